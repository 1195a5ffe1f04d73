"""Python entry to the HIP kernels.

Each function checks shapes, dtypes, devices and layout on the host, then calls one C entry
point of ``libtensorline_hip.so`` on torch's current stream.  There is no fallback: a missing
library, a tensor that is not on the GPU or a size a kernel does not take raises an error.
"""
from __future__ import annotations

import atexit
import ctypes
import glob
import os
import tempfile
import threading
import warnings
from dataclasses import dataclass

import torch

from tensorline_amd.ops import build as _build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_lib = None
_lib_lock = threading.Lock()


def library() -> ctypes.CDLL:
    """The loaded kernel library; built at the first call if no built one matches the sources."""
    global _lib
    if _lib is None:
        with _lib_lock:
            if _lib is None:
                path = _build.ensure_built()
                try:
                    lib = ctypes.CDLL(path)
                except OSError as e:
                    raise KernelError(f"cannot load the HIP kernel library {path}: {e}") from e
                lib.tl_last_error.restype = ctypes.c_char_p
                _lib = lib
    return _lib


def library_path() -> str | None:
    return _build.find_built()


def require_gpu(device) -> torch.device:
    """The engine runs on a ROCm GPU only."""
    dev = torch.device(device)
    if dev.type != "cuda":
        raise KernelError(f"tensorline_amd runs on a ROCm GPU (device 'cuda:N'), not on {dev}")
    if not torch.cuda.is_available():
        raise KernelError("no ROCm GPU is visible to torch: the engine has no CPU path")
    library()
    return dev


def _call(name: str, *args) -> None:
    fn = getattr(library(), name)
    rc = fn(*args)
    if rc != 0:
        raise KernelError(library().tl_last_error().decode("utf-8", "replace"))


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: torch.Tensor | None) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _on_gpu(*tensors: torch.Tensor | None) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        _check(t.is_cuda, f"tensor of shape {tuple(t.shape)} is on {t.device}, not on the GPU")
        dev = dev or t.device
        _check(t.device == dev, "tensors are on different devices")


def _i32(t: torch.Tensor, what: str, n: int | None = None) -> None:
    _check(t.dtype == torch.int32 and t.is_contiguous(), f"{what} must be a contiguous int32 tensor")
    if n is not None:
        _check(t.numel() >= n, f"{what} has {t.numel()} entries, {n} are needed")


# ---------------------------------------------------------------------------------------------
def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """x[t] = float(table[ids[t]]); the residual stream is float32 in every mode."""
    _on_gpu(ids, table, out)
    _i32(ids, "ids")
    _check(table.dim() == 2 and table.is_contiguous(), "embedding table must be a contiguous [V, H] matrix")
    T, (V, H) = ids.numel(), table.shape
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    _check(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, H), "embed: bad output")
    _call("tl_embed", _ptr(ids), _ptr(table), _code(table, "embed"), _ptr(out), T, H, V, _stream())
    return out


def add_rmsnorm(x: torch.Tensor, residual: "torch.Tensor | ShareSum | None", weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor:
    """Without ``rows``: ``x += residual`` in place (float32), returns ``RMSNorm(x) * weight``.
    With ``rows``: returns the norm of ``x[rows] + residual[rows]`` and leaves ``x`` alone.
    ``residual`` may be a :class:`ShareSum`: its shares are added in order, then to ``x``."""
    parts, part_stride = 1, 0
    if isinstance(residual, ShareSum):
        residual = residual.parts
        _check(residual.dim() == 3 and residual.is_contiguous(), "add_rmsnorm: shares must be a contiguous [P, T, H] tensor")
        parts, part_stride = residual.shape[0], residual.shape[1] * residual.shape[2]
        residual = residual[0]
    _on_gpu(x, residual, weight, rows, out)
    _check(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "add_rmsnorm: x must be contiguous float32 [T, H]")
    T, H = x.shape
    _check(weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() == H,
           f"add_rmsnorm: weight must be float32 of {H} entries")
    res_code = F32
    if residual is not None:
        _check(residual.is_contiguous() and tuple(residual.shape) == (T, H), "add_rmsnorm: residual must match x")
        res_code = _code(residual, "add_rmsnorm residual")
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty(n, H, dtype=out_dtype, device=x.device)
    _check(out.dtype == out_dtype and out.is_contiguous() and tuple(out.shape) == (n, H), "add_rmsnorm: bad output")
    _call("tl_add_rmsnorm", _ptr(x), _ptr(residual), res_code, parts, ctypes.c_longlong(part_stride), _ptr(weight),
          _ptr(out), _code(out, "add_rmsnorm out"),
          _ptr(rows), n, H, ctypes.c_float(eps), _stream())
    return out


def shuffle_weight(weight: torch.Tensor) -> torch.Tensor | None:
    """The copy of a bfloat16 [N, K] matrix that the few-row kernel streams: [ceil(N/16) tiles,
    ceil(K/32) chunks, 64 lanes, 8 values], lane 16*g + r holding row r of the tile at k = 32*chunk +
    8*g .. +8, zero where it pads.  None for matrices that kernel does not take."""
    if weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] % 8:
        return None
    N, K = weight.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        padded = torch.zeros(Np, Kp, dtype=weight.dtype, device=weight.device)
        padded[:N, :K] = weight
    else:
        padded = weight
    return padded.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()


def shuffle_weight_float(weight: torch.Tensor) -> torch.Tensor | None:
    """The copy of a float32 [N, K] matrix that the few-row float product streams: [ceil(N/16) tiles,
    ceil(K/16) steps, 64 lanes, 4 values], lane 16*g + r holding row r of the tile at k = 16*step + 4*g
    .. +4 (the lane's operands of the four products of a step), zero where it pads: one load of a wave
    is 1 KB of consecutive memory instead of 16 pieces of 64 bytes.  None for other matrices."""
    if weight.dtype != torch.float32 or weight.dim() != 2:
        return None
    N, K = weight.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 16) * 16
    if (Np, Kp) != (N, K):
        padded = torch.zeros(Np, Kp, dtype=weight.dtype, device=weight.device)
        padded[:N, :K] = weight
    else:
        padded = weight
    return padded.view(Np // 16, 16, Kp // 16, 4, 4).permute(0, 2, 3, 1, 4).contiguous()


def _check_shuffled(shuffled: torch.Tensor, N: int, K: int) -> None:
    if shuffled.dtype == torch.float32:
        _check(shuffled.is_contiguous() and tuple(shuffled.shape) == (-(-N // 16), -(-K // 16), 4, 16, 4),
               f"linear: the shuffled float weight copy does not belong to a [{N}, {K}] matrix")
        return
    _check(shuffled.dtype == torch.bfloat16 and shuffled.is_contiguous()
           and tuple(shuffled.shape) == (-(-N // 16), -(-K // 32), 4, 16, 8),
           f"linear: the shuffled weight copy does not belong to a [{N}, {K}] matrix")


@dataclass
class NormedRows:
    """Activations whose RMS normalisation is still owed.  ``rows`` [M, K] holds ``h * weight`` in
    the activation dtype and ``sumsq`` [parts, M] float32 partial sums of ``h^2``, row m's in column m; the
    product that takes them multiplies its result rows by ``1 / sqrt(sum(sumsq) / dim + eps)``,
    which equals the product of the normalised rows because the division is one factor per row."""
    rows: torch.Tensor
    sumsq: torch.Tensor
    dim: int
    eps: float
    stands_for_normed_rows = True      # a carry of this form is a norm's output; ``take`` picks rows of it

    def take(self, index: torch.Tensor) -> "NormedRows":
        """The rows ``index`` (int tensor) only."""
        idx = index.long()
        return NormedRows(self.rows.index_select(0, idx), self.sumsq.index_select(1, idx), self.dim, self.eps)


@dataclass
class NormSink:
    """What a product that ends a residual branch does instead of returning its result: add it to
    ``resid`` (float32 [M, N], in place) and hand the sum on as the :class:`NormedRows` of the next
    RMS norm (``weight`` float32 [N], ``eps``)."""
    resid: torch.Tensor
    weight: torch.Tensor
    eps: float


@dataclass
class ShareSum:
    """A product still in the shares of K it was computed in: ``parts`` [P, M, N] float32 stands for
    ``parts[0] + parts[1] + ...`` in that order.  The norm kernel adds the shares on its way
    (:func:`add_rmsnorm`), which saves the pass over memory that adding them first would take."""
    parts: torch.Tensor

    def sum(self) -> torch.Tensor:
        return self.parts.sum(0)


class _NormArgs(ctypes.Structure):
    _fields_ = [("ss_in", ctypes.c_void_p), ("ss_ld", ctypes.c_int), ("ss_n", ctypes.c_int),
                ("dim", ctypes.c_float), ("eps", ctypes.c_float),
                ("resid", ctypes.c_void_p), ("resid_ld", ctypes.c_int), ("next_weight", ctypes.c_void_p),
                ("a_out", ctypes.c_void_p), ("a_ld", ctypes.c_int), ("ss_out", ctypes.c_void_p),
                ("ss_out_ld", ctypes.c_int)]


def can_defer_norm(num_rows: int, dtype: torch.dtype) -> bool:
    """Whether the streaming products can carry the norms of a step of ``num_rows`` rows."""
    return dtype == torch.bfloat16 and 0 < num_rows <= ROWS64_MAX_ROWS


def _norm_args(owed: NormedRows | None, sink: NormSink | None, M: int, N: int, device, columns_per_partial: int = 16):
    """(ctypes argument, NormedRows the sink produces or None) for the streaming products' entry
    points; a sink leaves one partial sum of squares per row and ``columns_per_partial`` columns."""
    if owed is None and sink is None:
        return None, None
    na = _NormArgs()
    produced = None
    if owed is not None:
        _check(owed.sumsq.dtype == torch.float32 and owed.sumsq.dim() == 2 and owed.sumsq.shape[1] == M
               and owed.sumsq.stride(1) == 1 and owed.sumsq.stride(0) >= M,
               "owed norm: partial sums must be float32 [parts, M]")
        na.ss_in, na.ss_ld, na.ss_n = owed.sumsq.data_ptr(), owed.sumsq.stride(0), owed.sumsq.shape[0]
        na.dim, na.eps = float(owed.dim), float(owed.eps)
    if sink is not None:
        r, w = sink.resid, sink.weight
        _on_gpu(r, w)
        _check(r.dtype == torch.float32 and tuple(r.shape) == (M, N) and r.stride(1) == 1,
               f"residual sink: the residual must be float32 [{M}, {N}]")
        _check(w.dtype == torch.float32 and w.is_contiguous() and w.numel() == N,
               f"residual sink: the norm weight must be float32 of {N} entries")
        parts = -(-N // columns_per_partial)
        produced = NormedRows(torch.empty(M, N, dtype=torch.bfloat16, device=device),
                              torch.empty(parts, M, dtype=torch.float32, device=device), N, float(sink.eps))
        na.resid, na.resid_ld, na.next_weight = r.data_ptr(), r.stride(0), w.data_ptr()
        na.a_out, na.a_ld = produced.rows.data_ptr(), N
        na.ss_out, na.ss_out_ld = produced.sumsq.data_ptr(), M
    return ctypes.byref(na), produced


def linear(a: torch.Tensor | NormedRows, weight: torch.Tensor, bias: torch.Tensor | None = None,
           out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
           shuffled: torch.Tensor | None = None, sink: NormSink | None = None,
           keep_shares: bool = False) -> "torch.Tensor | NormedRows | ShareSum":
    """``a @ weight.T + bias``: a [M, K] (rows may be strided), weight [N, K], bias float32 [N].
    ``shuffled``: the copy of ``weight`` made by :func:`shuffle_weight`, which few-row bfloat16
    products stream instead of ``weight``.  ``a`` may be :class:`NormedRows` and ``sink`` a
    :class:`NormSink` (then the result is the next norm's :class:`NormedRows`); both need the few-row
    kernel (:func:`can_defer_norm` rows, a shuffled copy).  ``keep_shares``: the caller takes a
    :class:`ShareSum` where the product is computed in shares of K (many rows, a long K)."""
    owed = a if isinstance(a, NormedRows) else None
    if owed is not None:
        a = owed.rows
    _on_gpu(a, weight, bias, out, shuffled)
    _check(a.dim() == 2 and a.stride(1) == 1, "linear: input must be [M, K] with unit column stride")
    _check(weight.dim() == 2 and weight.is_contiguous(), "linear: weight must be a contiguous [N, K] matrix")
    M, K = a.shape
    N = weight.shape[0]
    _check(weight.shape[1] == K, f"linear: input has K={K}, weight has K={weight.shape[1]}")
    if bias is not None:
        _check(bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == N,
               f"linear: bias must be float32 of {N} entries")
    out_dtype = out_dtype or a.dtype
    if owed is not None or sink is not None:
        lda = a.stride(0) if M > 1 else K
        _check(out is None and (_skinny_ok(a, shuffled, M, K, lda) or _rows64_ok(a, shuffled, M, K, lda)),
               "linear: a deferred norm needs a streaming bfloat16 kernel (at most 64 rows, a shuffled weight copy)")
        _check_shuffled(shuffled, N, K)
        few = M <= SKINNY_MAX_ROWS and not (_few_rows_go_to_rows64(N, K) and _rows64_ok(a, shuffled, M, K, lda, few_too=True))
        # a sink's partials: per 16-column tile where the first kernel completes the sums, per 256 columns
        # where the mid-row product's second kernel does
        per = 16 if few or library().tl_gemm_rows64_shares(M, N, K) == 1 else 256
        norm, produced = _norm_args(owed, sink, M, N, a.device, per)
        if produced is None:
            out = torch.empty(M, N, dtype=out_dtype, device=a.device)
        if few:
            _call("tl_gemm_skinny", _ptr(a), _ptr(shuffled), _ptr(bias), _ptr(out),
                  F32 if out is None else _code(out, "linear output"), M, N, K, lda, N, norm, _stream())
        else:
            _rows64(a, shuffled, bias, out, M, N, K, lda, N, swiglu=False, norm=norm)
        return produced if produced is not None else out
    if out is None:
        if a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and (
                M > ROWS64_MAX_ROWS or (M > SKINNY_MAX_ROWS and shuffled is None)):
            return _library_linear(a, weight, bias, out_dtype, keep_shares)
        out = torch.empty(M, N, dtype=out_dtype, device=a.device)
    _check(out.dim() == 2 and tuple(out.shape) == (M, N) and out.stride(1) == 1 and out.dtype == out_dtype,
           "linear: bad output")
    lda = a.stride(0) if M > 1 else K
    ldc = out.stride(0) if M > 1 else N
    if shuffled is not None:
        _check_shuffled(shuffled, N, K)
    return _linear_dispatch(a, weight, bias, out, M, N, K, lda, ldc, shuffled)


MAX_KEY_SPLITS = 1024    # key splits the attention merge kernel takes
GENERIC_SPLIT_KEYS = 256  # keys per split of the any-shape attention kernel in steps of one token per sequence
SKINNY_MAX_ROWS = 16     # rows the few-row kernel serves (one 16-row MFMA tile)
ROWS64_MAX_ROWS = 64     # rows the 17..64-row kernel serves; above that the library


def _skinny_ok(a: torch.Tensor, shuffled: torch.Tensor | None, M: int, K: int, lda: int) -> bool:
    return (shuffled is not None and a.dtype == torch.bfloat16 and M <= SKINNY_MAX_ROWS
            and K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0)


def _rows64_ok(a: torch.Tensor, shuffled: torch.Tensor | None, M: int, K: int, lda: int, few_too: bool = False) -> bool:
    return (shuffled is not None and a.dtype == torch.bfloat16 and (few_too or SKINNY_MAX_ROWS < M) and M <= ROWS64_MAX_ROWS
            and K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0)


def _few_rows_go_to_rows64(N: int, K: int) -> bool:
    """Whether a plain product of at most 16 rows runs on the 17-to-64-row kernel.  The few-row
    kernel gives every 16-column tile to one work-group, so 320 tiles (5,120 columns) put two on 64
    of the 256 CUs and one on the rest, and the product takes as long as two tiles; the other
    kernel cuts K into shares as well and fills whole rounds of CUs, at the price of a second
    kernel.  That pays where the last round of tiles is far from full and K is long (measured at 8
    rows: 5,120 x 13,824: 31.6 against 38.0 us, 5,120 x 27,648: 59.4 against 70.4; not at 5,120 x
    5,120: 15.8 against 13.9).  The choice depends on the matrix alone, not on the rows."""
    tiles, steps = -(-N // 16), -(-K // 128)
    rounds = -(-tiles // 256)
    return 2 <= rounds <= 3 and tiles < 0.75 * rounds * 256 and rounds * steps >= 150


def _rows64(a, shuffled, bias, out, M, N, K, lda, ldc, swiglu: bool, norm=None):
    """17 to 64 rows: a 16-column tile per wave, rows shared through LDS, K split over the grid."""
    shares = library().tl_gemm_rows64_shares(M, N, K)
    ws = torch.empty(shares * M * N, dtype=torch.float32, device=a.device) if shares > 1 else None
    _call("tl_gemm_rows64", _ptr(a), _ptr(shuffled), _ptr(bias), _ptr(out), F32 if out is None else _code(out, "linear output"),
          _ptr(ws), M, N, K, lda, ldc, shares, 1 if swiglu else 0, norm, _stream())
    return out


def _linear_dispatch(a, weight, bias, out, M, N, K, lda, ldc, shuffled=None) -> torch.Tensor:
    """bfloat16 with few rows: the streaming MFMA kernel.  float32, and shapes that kernel does not
    take: the plain tiled kernel.  (bfloat16 with many rows went to the library before this, where
    the reference uses one too: tensorline/paged.py:179-188.)"""
    if _skinny_ok(a, shuffled, M, K, lda) and not _few_rows_go_to_rows64(N, K):
        _call("tl_gemm_skinny", _ptr(a), _ptr(shuffled), _ptr(bias), _ptr(out), _code(out, "linear output"),
              M, N, K, lda, ldc, None, _stream())
        return out
    if _rows64_ok(a, shuffled, M, K, lda, few_too=True):
        return _rows64(a, shuffled, bias, out, M, N, K, lda, ldc, swiglu=False)
    if (shuffled is not None and shuffled.dtype == torch.float32 and a.dtype == torch.float32 and out.dtype == torch.float32
            and M <= SKINNY_MAX_ROWS and library().tl_gemm_fewrows_takes(K)):
        _call("tl_gemm_fewrows_shuffled", _ptr(a), _ptr(shuffled), _ptr(bias), _ptr(out), M, N, K, lda, ldc, _stream())
        return out
    _call("tl_gemm_generic", _ptr(a), _code(a, "linear input"), _ptr(weight), _code(weight, "linear weight"),
          _ptr(bias), _ptr(out), _code(out, "linear output"), M, N, K, lda, ldc, _stream())
    return out


_MM_OUT_DTYPE_OK: bool | None = None


def _library_linear(a, weight, bias, out_dtype, keep_shares: bool = False):
    """hipBLASLt through torch for many-row bfloat16 products (float32 accumulation inside)."""
    global _MM_OUT_DTYPE_OK
    wt = weight.t()
    M, K = a.shape
    N = weight.shape[0]
    tiles = -(-M // 256) * -(-N // 256)
    if out_dtype == torch.float32 and _MM_OUT_DTYPE_OK and K >= 8192 and tiles < 200:
        # A long K with few output tiles leaves most of the 256 CUs idle in the library's product:
        # K is cut into 2, 4 or 8 shares run as one batched product, and the shares are added in order.
        ks = next((c for c in (2, 4, 8) if tiles * c >= 200), 8)
        if K % (8 * ks) == 0 and a.is_contiguous():
            kk = K // ks
            parts = torch.bmm(a.view(M, ks, kk).transpose(0, 1), weight.view(N, ks, kk).permute(1, 2, 0),
                              out_dtype=torch.float32)
            if keep_shares and bias is None:
                return ShareSum(parts)
            y = parts.sum(0)
            if bias is not None:
                y.add_(bias)
            return y
    if out_dtype == torch.float32:
        if _MM_OUT_DTYPE_OK is None:
            try:
                torch.mm(a[:1], wt[:, :16], out_dtype=torch.float32)
                _MM_OUT_DTYPE_OK = True
            except Exception:
                _MM_OUT_DTYPE_OK = False
        y = torch.mm(a, wt, out_dtype=torch.float32) if _MM_OUT_DTYPE_OK else torch.mm(a, wt).to(torch.float32)
        if bias is not None:
            y.add_(bias)
        return y
    y = torch.mm(a, wt)
    if bias is not None:
        y.add_(bias.to(y.dtype))
    return y


_TUNING_RECORD: str | None = None


def _keep_tuning_records_out_of_the_way(tn) -> None:
    """TunableOp records what it finds in a file, by default in the working directory: the record
    goes to a file of this process in the temporary directory instead and is removed at exit (a
    search is repeated in every process; nothing is read back)."""
    global _TUNING_RECORD
    if _TUNING_RECORD is not None:
        return
    if hasattr(tn, "write_file_on_exit"):
        tn.write_file_on_exit(False)
    _TUNING_RECORD = os.path.join(tempfile.gettempdir(), f"tensorline_amd_tuning_{os.getuid()}_{os.getpid()}.csv")
    tn.set_filename(_TUNING_RECORD)

    def remove():
        for path in glob.glob(_TUNING_RECORD[:-4] + "*"):
            try:
                os.remove(path)
            except OSError:
                pass
    atexit.register(remove)


def tune_library_linear(rows: int, weight: torch.Tensor, out_dtype: torch.dtype, seconds: float = 2.0) -> bool:
    """Have the library pick its kernel for the ``[rows, K] x [N, K]^T`` product by measurement
    (torch's TunableOp searches the hipBLASLt and rocBLAS solutions once and keeps the fastest for
    later calls of that shape) instead of by its heuristic: at 2,048 rows and the widths of a 7B
    model the heuristic's choice reaches about 1.0 PFLOP/s, the measured one 1.25.  Only the shape
    given is searched, here and now; other shapes keep the heuristic and are never searched at a
    request's cost.  Returns False when this torch has no TunableOp or the product does not go to
    the library."""
    tn = getattr(torch.cuda, "tunable", None)
    if tn is None or weight.dtype != torch.bfloat16 or rows <= ROWS64_MAX_ROWS:
        return False
    _on_gpu(weight)
    tn.enable(True)
    _keep_tuning_records_out_of_the_way(tn)
    tn.set_max_tuning_duration(int(seconds * 1000))
    tn.set_max_tuning_iterations(50)
    a = torch.randn(rows, weight.shape[1], device=weight.device).to(torch.bfloat16)
    tn.tuning_enable(True)
    try:
        _library_linear(a, weight, None, out_dtype)
        torch.cuda.synchronize(weight.device)
    except RuntimeError as e:                            # the search is optional: the heuristic choice stays
        warnings.warn(f"library tuning of the {tuple(weight.shape)} product failed and is skipped: {e}")
        return False
    finally:
        tn.tuning_enable(False)
    return True


def swiglu_gate_up(h: torch.Tensor | NormedRows, gate_up_weight: torch.Tensor,
                   shuffled: torch.Tensor | None = None) -> torch.Tensor:
    """``silu(h Wg^T) * (h Wu^T)`` for a fused [2I, K] weight (gate rows first): one kernel for
    few-row bfloat16 batches (it streams the ``shuffled`` copy), product then SiLU-multiply otherwise.
    ``h`` may be :class:`NormedRows` (few-row kernel only)."""
    owed = h if isinstance(h, NormedRows) else None
    if owed is not None:
        h = owed.rows
    _on_gpu(h, gate_up_weight, shuffled)
    _check(h.dim() == 2 and h.stride(1) == 1 and gate_up_weight.dim() == 2 and gate_up_weight.is_contiguous()
           and gate_up_weight.shape[0] % 2 == 0 and gate_up_weight.shape[1] == h.shape[1], "swiglu_gate_up: bad shapes")
    M, K = h.shape
    I = gate_up_weight.shape[0] // 2
    lda = h.stride(0) if M > 1 else K
    if shuffled is not None:
        _check_shuffled(shuffled, 2 * I, K)
    if _skinny_ok(h, shuffled, M, K, lda) and I % 16 == 0:
        out = torch.empty(M, I, dtype=h.dtype, device=h.device)
        norm, _ = _norm_args(owed, None, M, 2 * I, h.device)
        _call("tl_gemm_skinny_swiglu", _ptr(h), _ptr(shuffled), _ptr(out), M, I, K, lda, I, norm, _stream())
        return out
    if _rows64_ok(h, shuffled, M, K, lda) and (I % 16 == 0 or library().tl_gemm_rows64_shares(M, 2 * I, K) > 1):
        out = torch.empty(M, I, dtype=h.dtype, device=h.device)
        norm, _ = _norm_args(owed, None, M, 2 * I, h.device)
        return _rows64(h, shuffled, None, out, M, 2 * I, K, lda, I, swiglu=True, norm=norm)
    return silu_mul(linear(owed if owed is not None else h, gate_up_weight, shuffled=shuffled))


def _check_caches(k_cache, v_cache, dtype, num_kv_heads, head_dim, who: str) -> None:
    """Keys are paged as [pages, page, nkv, d]; values as [pages, nkv, d, page] (transposed in the page)."""
    _check(k_cache.dtype == dtype and k_cache.is_contiguous() and k_cache.dim() == 4
           and k_cache.shape[2] == num_kv_heads and k_cache.shape[3] == head_dim,
           f"{who}: key cache must be contiguous [pages, page, nkv, d] of the activation dtype")
    pages, page = k_cache.shape[0], k_cache.shape[1]
    _check(v_cache.dtype == dtype and v_cache.is_contiguous()
           and tuple(v_cache.shape) == (pages, num_kv_heads, head_dim, page),
           f"{who}: value cache must be contiguous [pages, nkv, d, page] matching the key cache")


def qkv_rope_store(h: torch.Tensor | NormedRows, shuffled: torch.Tensor, bias: torch.Tensor | None, pos: torch.Tensor,
                   inv_freq: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                   k_cache: torch.Tensor, v_cache: torch.Tensor, slots: torch.Tensor) -> torch.Tensor | None:
    """The projection, position encoding and cache write of a decode step in one kernel: returns the
    rotated queries [M, nq*d]; rotated keys and the values go into the cache at ``slots``.  Returns
    None when the kernel does not take the case (then the three separate kernels run): it needs
    bfloat16, at most 64 rows (above 16: a K long enough to be cut into shares), a head size that is
    a multiple of 32 and full-width rotation.
    ``h`` may be :class:`NormedRows`."""
    owed = h if isinstance(h, NormedRows) else None
    if owed is not None:
        h = owed.rows
    M, K = h.shape
    N = (num_heads + 2 * num_kv_heads) * head_dim
    if not (h.dtype == torch.bfloat16 and shuffled is not None and M <= ROWS64_MAX_ROWS and head_dim % 32 == 0
            and inv_freq is not None and 2 * inv_freq.numel() == head_dim and h.stride(1) == 1
            and K % 8 == 0 and h.data_ptr() % 16 == 0 and (M == 1 or h.stride(0) % 8 == 0)):
        return None
    shares = 1
    if M > SKINNY_MAX_ROWS:
        shares = library().tl_gemm_rows64_shares(M, N, K)
        if shares == 1:                                   # the mid-row product fuses only in its second kernel
            return None
    _on_gpu(h, shuffled, bias, pos, inv_freq, k_cache, v_cache, slots)
    _check_shuffled(shuffled, N, K)
    _check_caches(k_cache, v_cache, h.dtype, num_kv_heads, head_dim, "qkv_rope_store")
    _i32(pos, "pos", M)
    _i32(slots, "slots", M)
    _check(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "qkv_rope_store: inv_freq must be float32")
    if bias is not None:
        _check(bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == N, "qkv_rope_store: bad bias")
    q = torch.empty(M, num_heads * head_dim, dtype=h.dtype, device=h.device)
    norm, _ = _norm_args(owed, None, M, N, h.device)
    if M > SKINNY_MAX_ROWS:
        ws = torch.empty(shares * M * N, dtype=torch.float32, device=h.device)
        _call("tl_gemm_rows64_qkv_rope", _ptr(h), _ptr(shuffled), _ptr(bias), _ptr(pos), _ptr(inv_freq), _ptr(slots),
              _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(ws), M, K, h.stride(0), num_heads, num_kv_heads, head_dim,
              k_cache.shape[1], shares, norm, _stream())
        return q
    _call("tl_gemm_skinny_qkv_rope", _ptr(h), _ptr(shuffled), _ptr(bias), _ptr(pos), _ptr(inv_freq), _ptr(slots),
          _ptr(q), _ptr(k_cache), _ptr(v_cache), M, K, h.stride(0) if M > 1 else K, num_heads, num_kv_heads,
          head_dim, k_cache.shape[1], norm, _stream())
    return q


def rope_store(qkv: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor | None, num_heads: int,
               num_kv_heads: int, head_dim: int, k_cache: torch.Tensor | None, v_cache: torch.Tensor | None,
               slots: torch.Tensor | None, bias: torch.Tensor | None = None) -> None:
    """Rotate the query and key heads of the fused projection ``qkv`` [T, (nq + 2 nkv) d]; queries
    in place, rotated keys and the values into the paged cache at ``slots`` (negative: skip).
    ``bias`` (float32, one per column of ``qkv``) is a projection bias still owed: added first."""
    _on_gpu(qkv, pos, inv_freq, k_cache, v_cache, slots, bias)
    if bias is not None:
        _check(bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == qkv.shape[1],
               "rope_store: the bias must be float32 with one entry per column")
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _check(qkv.dim() == 2 and qkv.is_contiguous() and qkv.shape[1] == width,
           f"rope_store: qkv must be contiguous [T, {width}], got {tuple(qkv.shape)}")
    _i32(pos, "pos", T)
    rot = 0
    if inv_freq is not None:
        _check(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "rope_store: inv_freq must be float32")
        rot = 2 * inv_freq.numel()
        _check(rot <= head_dim, f"rope_store: rotary width {rot} exceeds the head size {head_dim}")
    write = k_cache is not None
    if write:
        _check(v_cache is not None and slots is not None, "rope_store: cache write needs k_cache, v_cache and slots")
        _check_caches(k_cache, v_cache, qkv.dtype, num_kv_heads, head_dim, "rope_store")
        _i32(slots, "slots", T)
    _call("tl_rope_store", _ptr(qkv), _code(qkv, "rope_store"), _ptr(pos), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache),
          _ptr(slots), T, num_heads, num_kv_heads, head_dim, rot, 1 if write else 0,
          k_cache.shape[1] if write else 0, _ptr(bias), _stream())


def one_token_sequences(facts) -> list[int]:
    """The sequences that bring one token to a step that also holds prompt portions (padding
    sequences among them); none in a step of one token per sequence."""
    if facts.decode_only:
        return []
    return [s for s, n in enumerate(facts.q_lens) if n == 1] + list(range(len(facts.q_lens), facts.num_seqs))


def _singles_get_own_launch(plan, singles: list[int], num_heads: int, num_kv_heads: int, head_dim: int,
                            window: int) -> bool:
    """Whether the one-token sequences of a step with prompt portions are worth a launch of their
    own.  Beside the portions each of them is walked by one work-group from its first key to its
    last, about 14 ns a key at a head size of 128 (and never faster than 1.5 times what their
    bytes take at the streaming rate); that time hides behind the portions' own, about 600 TFLOP/s
    of their scores and sums.  Alone they run split at the rate a decode step reads its cache,
    after about 9 us for the two launches, and the portions follow.  (Measured at 28 query and
    4 key/value heads of 128; only the choice of launches depends on it, not a result.)"""
    ctxs = [plan.starts[s] + 1 if s < len(plan.starts) else 1 for s in singles]
    if window > 0:
        ctxs = [min(c, window) for c in ctxs]
    stream_us = sum(ctxs) * 4 * num_kv_heads * head_dim / 4.5e6
    walk_us = max(0.014 * max(ctxs) * max(head_dim, 64) / 128, 1.5 * stream_us)
    portions_us = sum(n * (st + (n + 1) / 2) for n, st in zip(plan.q_lens, plan.starts) if n > 1) \
        * num_heads * head_dim * 4 / 6e8
    return walk_us > portions_us + 9 + stream_us + 5


LONG_SPLIT_KEYS = 1024    # the longest split the context scales a split to (64 pages of 16: a wave keeps their ids in its lanes)


def _key_splits(num_seqs: int, num_kv_heads: int, max_context: int, fit_context: int = 0) -> tuple[int, int]:
    """(keys per split, number of splits) for ``num_seqs`` one-token sequences; (0, 1): no split.
    The length follows the batch (enough waves for the GPU at a context of 4,096) and doubles with
    every doubling of the step's longest context beyond 4,096, up to LONG_SPLIT_KEYS: a context of
    32,768 is then cut into as many runs as one of 4,096, not eight times as many for the merge
    kernel to read back.  The doublings lie where the graphs' context buckets do, so an eager step
    and the graph captured for its bucket cut alike."""
    base = (1 << max(num_seqs - 1, 0).bit_length()) * num_kv_heads
    split_len = 64 if base <= 8 else 128 if base <= 32 else 256 if base <= 128 else 512 if base <= 512 else 0
    reach = 4096
    while split_len and reach < max_context and split_len < LONG_SPLIT_KEYS:
        split_len, reach = split_len * 2, reach * 2
    return _fit_key_splits(split_len, max_context, fit_context)


def _fit_key_splits(split_len: int, max_context: int, fit_context: int = 0) -> tuple[int, int]:
    """Splits get longer where there would be more than the merge kernel takes.  Their length is
    fitted to ``fit_context``, the longest context the engine ever runs, where the caller knows it
    (else to this step's longest): then every step of an engine, eager or replayed from a graph
    captured for the longest context, sums the same runs of keys together."""
    if not split_len:
        return 0, 1
    while -(-max(max_context, fit_context) // split_len) > MAX_KEY_SPLITS:
        split_len *= 2
    return split_len, max(1, -(-max_context // split_len))


def _tile16_chains(total128: int, num_kv_heads: int, path, longest_context: int = 1 << 30) -> int:
    """1 or 2: whether a work-group of the 16-columns-per-wave prompt kernel walks its keys as one
    chain of tiles or as two that take every other tile (twice the waves, put together at the end).
    Two where there is at most one work-group per CU: then the longest walk sets the time, and the
    second chain uses what a lone work-group leaves of its CU (1,024 tokens behind 4,096 at the 7B
    shape: 107 -> 96 us, 512 behind 8,192: 158 -> 131, 64 behind 3,000: 57 -> 50).  With more
    work-groups than CUs two of one chain per CU do as well or better (the two chains of a work-group
    pass their tiles' phases together, two work-groups drift apart and overlap them): a fresh prompt
    of 2,048 tokens takes 51 us either way, one of 3,072 94 against 113.  Nor with walks of fewer than
    16 tiles, where the second chain's waves and the hand-over at the end cost what they save (256
    fresh tokens: 12.3 against 11 us)."""
    if path == "mfma-tile16x2":
        return 2
    if path == "mfma-tile16":
        return 1
    return 2 if total128 * num_kv_heads <= 256 and longest_context >= 1024 else 1


def _tile32_waves(q_lens, starts, num_heads: int) -> int:
    """Whether a step's prompt portions run on the kernel with 32 columns per wave and work-groups of
    256 columns (8 waves; 0: no, they keep 16 columns per wave and work-groups of 128).  A work-group
    of 256 columns reads every key tile for twice the columns, which pays where the portions' columns
    see thousands of keys each and there are columns enough to fill the GPU with such groups;
    measured at 28 query and 4 key/value heads of 128: a 2,048-token portion behind 30,720 cached
    tokens 888 against 1,005 to 1,040 us, behind 14,336 483 against 500 to 530, a fresh prompt of
    8,192 tokens 490 against 510 to 526, of 4,096 165 against 155 to 163, of 2,048 66 against 52.
    Only the choice of kernel depends on it, never a result beyond rounding."""
    cols = sum(n for n in q_lens if n > 1)
    if cols == 0:
        return 0
    keys = sum(n * (st + (n + 1) / 2) for n, st in zip(q_lens, starts) if n > 1) / cols
    return 8 if keys >= 4096 and cols * num_heads >= 128 * 256 else 0          # at least 128 such work-groups


def attention_takes_head_dim(head_dim: int) -> bool:
    """The head sizes the attention kernels take: multiples of 16 up to 256 (32, 64 and 128 on the
    bfloat16 MFMA kernels, the others on the any-shape kernel)."""
    return head_dim > 0 and head_dim % 16 == 0 and head_dim <= 256


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, tables: torch.Tensor,
                    seq_of_token: torch.Tensor, pos: torch.Tensor, num_heads: int, num_kv_heads: int,
                    head_dim: int, scale: float, window: int = 0, out: torch.Tensor | None = None,
                    q_start: torch.Tensor | None = None, ctx_start: torch.Tensor | None = None, plan=None,
                    path: str | None = None, split_keys: int | None = None,
                    single_seqs: torch.Tensor | None = None, route_singles: bool | None = None) -> torch.Tensor:
    """Causal attention of each token over the cached keys of its sequence.

    ``q``: [T, >= nq*d] with the query heads in the first nq*d columns (row stride free);
    ``tables``: int32 [S, NB] page ids; ``seq_of_token``, ``pos``: int32 [T]; ``plan``: the step's
    host-side facts (``max_context``, ``max_query_len``, ``decode_only``, ``num_seqs``, ``q_lens``,
    ``starts``, ``fit_context``).  ``window`` > 0
    limits a token at position p to keys [p - window + 1, p].  Returns [T, nq*d].

    bfloat16 with a head size of 32, 64 or 128 and pages of a multiple of 8 tokens runs on the
    matrix cores; that kernel works per sequence and needs ``q_start`` [S+1], ``ctx_start`` [S]
    and the host-side ``plan`` (lengths of the step's sequences).  Everything else runs the
    any-shape kernel.  ``path`` forces one: "generic", "mfma" (prompt portions on the kernels that
    share key tiles through LDS where the page size allows; which of the two, see ``_tile32_waves``),
    "mfma-tile16" (16 columns per wave, work-groups of 128 columns walking their keys as one chain of
    tiles; "mfma-tile16x2": as two chains), "mfma-tile32" (32 columns per
    wave, work-groups of 256, head sizes 64 and 128) or "mfma-direct" (independent waves);
    ``split_keys`` forces the number of keys per split (0: no split).

    A step with prompt portions does not split keys: its one-token sequences would each be walked
    by one work-group from the first key to the last.  With ``single_seqs`` (int32, the indices
    ``one_token_sequences(plan)`` on the device) they are computed by a launch of their own where that is
    estimated to be faster (``_singles_get_own_launch``), split like a decode step of that many
    sequences, and the launch for the portions leaves them out.  ``route_singles`` forces that
    on or off."""
    _on_gpu(q, k_cache, v_cache, tables, seq_of_token, pos, out, q_start, ctx_start)
    T = q.shape[0]
    _check(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= num_heads * head_dim, "paged_attention: bad query layout")
    _check_caches(k_cache, v_cache, q.dtype, num_kv_heads, head_dim, "paged_attention")
    _check(tables.dim() == 2 and tables.dtype == torch.int32 and tables.is_contiguous(), "paged_attention: bad page table")
    _i32(seq_of_token, "seq_of_token", T)
    _i32(pos, "pos", T)
    if out is None:
        out = torch.empty(T, num_heads * head_dim, dtype=q.dtype, device=q.device)
    _check(out.dtype == q.dtype and out.dim() == 2 and out.shape[0] == T and out.stride(1) == 1, "paged_attention: bad output")
    q_stride = q.stride(0) if T > 1 else q.shape[1]
    o_stride = out.stride(0) if T > 1 else out.shape[1]
    page = k_cache.shape[1]
    mfma_ok = (q.dtype == torch.bfloat16 and head_dim in (32, 64, 128) and page % 8 == 0 and q_start is not None
               and ctx_start is not None and plan is not None and q_stride % 8 == 0 and o_stride % 4 == 0
               and q.data_ptr() % 16 == 0 and out.data_ptr() % 8 == 0)
    if path in ("mfma", "mfma-direct", "mfma-tile16", "mfma-tile16x2", "mfma-tile32"):
        _check(mfma_ok, "paged_attention: the matrix-core kernel does not take these arguments")
    if mfma_ok and path != "generic":
        S = tables.shape[0]
        _i32(q_start, "q_start", S + 1)
        _i32(ctx_start, "ctx_start", S)
        G = num_heads // num_kv_heads
        skip_single = 0
        singles = one_token_sequences(plan) if single_seqs is not None and split_keys is None else []
        if singles and route_singles is not False:
            _i32(single_seqs, "single_seqs", len(singles))
            ctx1 = max([plan.starts[s] + 1 for s in singles if s < len(plan.starts)] + [1])
            split_len, nsplit = _key_splits(len(singles), num_kv_heads, ctx1, plan.fit_context)
            if route_singles or (route_singles is None and nsplit > 1 and _singles_get_own_launch(
                    plan, singles, num_heads, num_kv_heads, head_dim, int(window))):
                nt1 = 1 if G <= 16 else 2
                ws = torch.empty(len(singles) * num_heads * nsplit * (head_dim + 2), dtype=torch.float32, device=q.device)
                n_o = len(singles) * num_heads * nsplit * head_dim
                _call("tl_attention_mfma", _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(tables), tables.shape[1],
                      _ptr(q_start), _ptr(ctx_start), _ptr(pos), _ptr(out), o_stride, _ptr(ws[:n_o]), _ptr(ws[n_o:]), T, S,
                      num_heads, num_kv_heads, head_dim, page, int(window), ctypes.c_float(scale), nt1,
                      -(-G // (16 * nt1)), nsplit, max(split_len // 32, 1), 0, 0, _ptr(single_seqs), len(singles), 0,
                      _stream())
                skip_single = 1
        q_lens = [n for n in plan.q_lens if n > 1] if skip_single else plan.q_lens
        nt = 1 if plan.max_query_len * G <= 16 else 2
        groups = [-(-n * G // (16 * nt)) for n in q_lens]
        pads = 0 if skip_single else max(0, S - len(groups))    # padding sequences bring one token each
        max_groups = max(groups + [1])
        total128 = sum(-(-n * G // 128) for n in q_lens) + pads
        # Splits are fixed runs of keys aligned to absolute positions, so the same keys are summed
        # together whatever the context length or the launch shape.  Pure decode steps split by the
        # batch size rounded up to a power of two (what a graph bucket pads to); steps with prompt
        # portions have enough columns and do not split.
        split_len, nsplit = 0, 1
        if split_keys is not None:
            _check(int(split_keys) % 32 == 0, "paged_attention: a split is a multiple of 32 keys")
            split_len, nsplit = _fit_key_splits(int(split_keys), plan.max_context, plan.fit_context)
        elif plan.decode_only:
            split_len, nsplit = _key_splits(S, num_kv_heads, plan.max_context, plan.fit_context)
        split_blocks = max(split_len // 32, 1)
        ws_o = ws_ml = None
        if nsplit > 1:
            ws = torch.empty(T * num_heads * nsplit * (head_dim + 2), dtype=torch.float32, device=q.device)
            ws_o, ws_ml = ws[:T * num_heads * nsplit * head_dim], ws[T * num_heads * nsplit * head_dim:]
        waves = 8 if path == "mfma-tile32" else _tile32_waves(plan.q_lens, plan.starts, num_heads) if path in (None, "mfma") else 0
        if (waves and nt == 2 and nsplit == 1 and total128 > 0
                and library().tl_attention_tile32_takes(head_dim, page, tables.shape[1], S, waves)):
            # prompt portions behind many keys, head size 64 or 128: 32 columns per wave on the 32x32
            # matrix-core instruction, work-groups of 256 columns
            cols = 32 * waves
            total = sum(-(-n * G // cols) for n in q_lens) + pads
            _call("tl_attention_tile32", _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(tables), tables.shape[1],
                  _ptr(q_start), _ptr(ctx_start), _ptr(out), o_stride, T, S, num_heads, num_kv_heads, head_dim, page,
                  int(window), ctypes.c_float(scale), waves, total, skip_single, _stream())
            return out
        _call("tl_attention_mfma", _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(tables), tables.shape[1],
              _ptr(q_start), _ptr(ctx_start), _ptr(pos), _ptr(out), o_stride, _ptr(ws_o), _ptr(ws_ml), T, S, num_heads,
              num_kv_heads, head_dim, page, int(window), ctypes.c_float(scale), nt, max_groups, nsplit, split_blocks,
              0 if path == "mfma-direct" else _tile16_chains(total128, num_kv_heads, path, plan.max_context), total128,
              _ptr(None), 0,
              skip_single, _stream())
        return out
    # The any-shape kernel tiles each sequence's tokens: it needs the first row of every sequence and the
    # most tokens one of them brings.  The engine has both; a bare call derives them from seq_of_token.
    S = tables.shape[0]
    if q_start is not None and plan is not None:
        _i32(q_start, "q_start", S + 1)
        max_query_len = int(plan.max_query_len)
    else:
        counts = torch.bincount(seq_of_token.long(), minlength=S)[:S]
        q_start = torch.zeros(S + 1, dtype=torch.int32, device=q.device)
        q_start[1:] = torch.cumsum(counts, 0)
        max_query_len = int(counts.max().item()) if T else 1
        # a row of a sequence the table does not have would be computed by nobody and merged from nothing
        _check(int(counts.sum().item()) == T, f"paged_attention: seq_of_token names sequences outside the {S} of the page table")
    _check(attention_takes_head_dim(head_dim), f"paged_attention: head size {head_dim} must be a multiple of 16, at most 256")
    # Steps of one token per sequence split the keys into runs of GENERIC_SPLIT_KEYS at absolute positions
    # (longer runs only where the longest context the engine ever runs would need more splits than a launch
    # takes), whatever the batch: one work-group per sequence and key/value head would walk a long context alone.
    split_len, nsplit, ws = 0, 1, None
    if plan is not None and plan.decode_only and max_query_len == 1 and split_keys != 0:
        split_len, nsplit = _fit_key_splits(int(split_keys) if split_keys else GENERIC_SPLIT_KEYS, plan.max_context,
                                            plan.fit_context)
        _check(split_len % 64 == 0, "paged_attention: a split of the any-shape kernel is a multiple of 64 keys")
        # Whether the runs go through the merge kernel is a matter of the longest context the engine
        # runs, not of this step's: a step of short contexts and its twin in a graph captured for long
        # ones take the same path and give the same bits (a second, empty run costs nothing).
        if nsplit == 1 and max(plan.max_context, plan.fit_context) > split_len:
            nsplit = 2
        if nsplit > 1:
            ws = torch.empty(T * num_heads * nsplit * (head_dim + 2), dtype=torch.float32, device=q.device)
    _call("tl_attention_generic", _ptr(q), q_stride, _ptr(k_cache), _ptr(v_cache), _ptr(tables), tables.shape[1],
          _ptr(q_start), _ptr(pos), _ptr(out), o_stride, _code(q, "paged_attention"), T, S, max(max_query_len, 1), num_heads,
          num_kv_heads, head_dim, page, int(window), ctypes.c_float(scale), nsplit, split_len, _ptr(ws), _stream())
    return out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``silu(gate_up[:, :I]) * gate_up[:, I:]`` for a fused [T, 2I] projection."""
    _on_gpu(gate_up, out)
    _check(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0,
           "silu_mul: input must be contiguous [T, 2I]")
    T, I2 = gate_up.shape
    if out is None:
        out = torch.empty(T, I2 // 2, dtype=gate_up.dtype, device=gate_up.device)
    _check(out.dtype == gate_up.dtype and out.is_contiguous() and tuple(out.shape) == (T, I2 // 2), "silu_mul: bad output")
    _call("tl_silu_mul", _ptr(gate_up), _ptr(out), _code(gate_up, "silu_mul"), T, I2 // 2, _stream())
    return out


def argmax(logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """Row-wise arg-max of float32 logits [R, V] -> int32 [R]; the lowest index wins a tie."""
    _on_gpu(logits, out)
    _check(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax: logits must be float32 [R, V]")
    R, V = logits.shape
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _i32(out, "argmax output", R)
    sv = si = None
    if V > 8192:            # wide rows: per-chunk bests, then the row's best among them
        sv = torch.empty(R * 64, dtype=torch.float32, device=logits.device)
        si = torch.empty(R * 64, dtype=torch.int32, device=logits.device)
    _call("tl_argmax", _ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(out), _ptr(sv), _ptr(si), _stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor | None = None, any_top_p: bool | None = None, any_greedy: bool = True) -> torch.Tensor:
    """One token per row of float32 logits [R, V]: greedy where temperature <= 0, else a draw from
    softmax(logits / temperature) cut by top-p, using the uniform number given for the row.
    ``any_top_p``: whether some row has top_p < 1, if the caller knows (saves three kernels when
    none has, and a look at the device when not given); ``any_greedy`` False promises that no row
    is greedy (saves the arg-max)."""
    _on_gpu(logits, temperature, top_p, uniform, out)
    _check(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be float32 [R, V]")
    R, V = logits.shape
    for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        _check(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == R, f"sample: {name} must be float32 [R]")
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _i32(out, "sample output", R)
    if any_top_p is None:
        any_top_p = bool((top_p < 1).any().item())
    chunks = library().tl_sample_chunks(V)
    pmax = torch.empty(R * chunks, dtype=torch.float32, device=logits.device)
    ws = torch.zeros(R * (3080 + 3 * chunks), dtype=torch.int64, device=logits.device)
    _call("tl_sample", _ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(temperature), _ptr(top_p),
          _ptr(uniform), _ptr(out), _ptr(pmax), _ptr(ws), 1 if any_greedy else 0, 1 if any_top_p else 0, _stream())
    return out
