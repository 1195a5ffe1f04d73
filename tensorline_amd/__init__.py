"""tensorline_amd: a one-GPU inference engine for AMD MI355X (gfx950).

The public surface is small on purpose:

* :class:`tensorline_amd.engine.llm.LLM`: load a model folder, generate tokens.
* :class:`tensorline_amd.sampling.params.SamplingParams` / ``GenStats``: the
  request options of the reference engine (``tensorline/engine.py:24-39``).
* :func:`tensorline_amd.config.registry.load_model_config`: read ``config.json``
  and pick the architecture by its ``architectures[0]`` entry.
"""

__version__ = "0.1.0"

from tensorline_amd.sampling.params import GenStats, SamplingParams  # noqa: F401


def __getattr__(name):
    if name == "LLM":
        from tensorline_amd.engine.llm import LLM
        return LLM
    raise AttributeError(name)
