"""Each HIP kernel alone against its plain reference, at sizes other than the engine's."""
import math

import pytest
import torch

from tests import plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def K():
    from tensorline_amd.ops import kernels
    return kernels


def tol(dtype, f32=1e-5, bf16=2e-2):
    return dict(atol=f32, rtol=f32) if dtype == torch.float32 else dict(atol=bf16, rtol=bf16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    torch.manual_seed(0)
    table = torch.randn(1000, 192, device=DEV).to(dtype)
    ids = torch.tensor([0, 999, 5, 5, 17], dtype=torch.int32, device=DEV)
    x = K().embed(ids, table)
    assert x.dtype == torch.float32
    torch.testing.assert_close(x, table[ids.long()].float(), atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [1, 5, 64])
def test_add_rmsnorm_reference_vector(dtype, T):
    # sizes of the reference's own test: H=896, eps=1e-6, w ~ U(0.5, 1.5) (tests/test_quant.py:100-113)
    torch.manual_seed(0)
    H, eps = 896, 1e-6
    w = torch.empty(H, device=DEV).uniform_(0.5, 1.5)
    x = torch.randn(T, H, device=DEV)
    r = torch.randn(T, H, device=DEV).to(dtype)
    want_x = x + r.float()
    want = plain.rmsnorm(want_x.double(), w.double(), eps)
    got = K().add_rmsnorm(x, r, w, eps, dtype)
    torch.testing.assert_close(x, want_x, atol=0, rtol=0)          # updated in place, exactly
    torch.testing.assert_close(got.double(), want, **tol(dtype, 2e-6, 2e-2))
    # no residual, odd width, rows picked
    H2 = 193
    x2 = torch.randn(7, H2, device=DEV)
    w2 = torch.randn(H2, device=DEV)
    keep = x2.clone()
    got2 = K().add_rmsnorm(x2, None, w2, 1e-5, dtype)
    torch.testing.assert_close(x2, keep, atol=0, rtol=0)
    torch.testing.assert_close(got2.double(), plain.rmsnorm(keep.double(), w2.double(), 1e-5), **tol(dtype, 2e-6, 2e-2))
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    r2 = torch.randn(7, H2, device=DEV).to(dtype)
    got3 = K().add_rmsnorm(x2, r2, w2, 1e-5, dtype, rows=rows)
    torch.testing.assert_close(x2, keep, atol=0, rtol=0)            # with rows, x is left alone
    want3 = plain.rmsnorm((keep + r2.float())[rows.long()].double(), w2.double(), 1e-5)
    torch.testing.assert_close(got3.double(), want3, **tol(dtype, 2e-6, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [1, 3, 16, 17, 64, 130])
@pytest.mark.parametrize("N,Kd", [(176, 64), (1000, 192), (64, 100), (3, 7)])
def test_linear(dtype, M, N, Kd):
    torch.manual_seed(M * 1000 + N)
    a = torch.randn(M, Kd, device=DEV).to(dtype)
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(dtype)
    b = torch.randn(N, device=DEV)
    want = a.double() @ w.double().T + b.double()
    got = K().linear(a, w, b)
    assert got.dtype == dtype
    torch.testing.assert_close(got.double(), want, **tol(dtype, 1e-5, 3e-2))
    got32 = K().linear(a, w, None, out_dtype=torch.float32)
    torch.testing.assert_close(got32.double(), a.double() @ w.double().T, **tol(dtype, 1e-5, 1e-5))


@pytest.mark.parametrize("H", [896, 193, 3584])
def test_add_rmsnorm_takes_a_product_in_its_shares(H):
    """A residual given as the K shares of a product: the shares are added in order, then to x; the
    result has the bits of adding them first."""
    torch.manual_seed(H)
    T, eps = 37, 1e-6
    w = torch.empty(H, device=DEV).uniform_(0.5, 1.5)
    for P in (2, 3):
        x = torch.randn(T, H, device=DEV)
        x2 = x.clone()
        parts = torch.randn(P, T, H, device=DEV)
        got = K().add_rmsnorm(x, K().ShareSum(parts), w, eps, torch.bfloat16)
        want = K().add_rmsnorm(x2, parts.sum(0), w, eps, torch.bfloat16)
        torch.testing.assert_close(x, x2, atol=0, rtol=0)
        torch.testing.assert_close(got, want, atol=0, rtol=0)
        rows = torch.tensor([5, 0, 36], dtype=torch.int32, device=DEV)
        got_r = K().add_rmsnorm(x, K().ShareSum(parts), w, eps, torch.float32, rows=rows)
        want_r = K().add_rmsnorm(x2, parts.sum(0), w, eps, torch.float32, rows=rows)
        torch.testing.assert_close(got_r, want_r, atol=0, rtol=0)


def test_linear_many_rows_keeps_its_shares_on_request():
    """A many-row product with a long K and few output tiles runs as shares of K: on request they
    come back unsummed, and their sum is the product."""
    torch.manual_seed(3)
    M, N, Kd = 256, 512, 9216
    a = torch.randn(M, Kd, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(torch.bfloat16)
    want = a.double() @ w.double().T
    whole = K().linear(a, w, None, out_dtype=torch.float32)
    kept = K().linear(a, w, None, out_dtype=torch.float32, keep_shares=True)
    assert isinstance(kept, K().ShareSum) and kept.parts.shape[1:] == (M, N) and kept.parts.shape[0] > 1
    torch.testing.assert_close(kept.sum(), whole, atol=0, rtol=0)
    torch.testing.assert_close(whole.double(), want, atol=2e-3, rtol=2e-3)
    # a product that is not cut into shares comes back as a tensor either way
    small = K().linear(a[:, :1024].contiguous(), w[:, :1024].contiguous(), None, out_dtype=torch.float32, keep_shares=True)
    assert isinstance(small, torch.Tensor)


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("N,Kd", [(1000, 1184), (3584, 18944), (50, 1030), (70, 513), (130, 7), (16, 512), (37, 40000)])
def test_linear_few_rows_float32(M, N, Kd):
    """The float product for at most 16 rows: K in segments of 512 shared by a work-group's waves (one
    segment, a partial last one, more segments than waves, a K that is no multiple of 4 and one too
    long for the segments' sums in LDS, which the many-row kernel takes), N no multiple of 16.  A
    row's result has the same bits whatever other rows come along."""
    torch.manual_seed(M + N)
    a = torch.randn(M, Kd, device=DEV)
    w = torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)
    b = torch.randn(N, device=DEV)
    want = a.double() @ w.double().T + b.double()
    got = K().linear(a, w, b)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double(), want, atol=1e-5, rtol=1e-5)
    alone = K().linear(a[M - 1:].contiguous(), w, b)
    torch.testing.assert_close(alone[0], got[M - 1], atol=0, rtol=0)
    # from the matrix-core ordered copy of the weight (what the engine's decode steps stream): the same bits
    ws = K().shuffle_weight_float(w)
    assert ws.shape == (-(-N // 16), -(-Kd // 16), 4, 16, 4)
    torch.testing.assert_close(K().linear(a, w, b, shuffled=ws), got, atol=0, rtol=0)
    strided = torch.randn(M, Kd + 5, device=DEV)[:, 1:Kd + 1]          # rows neither aligned nor contiguous
    torch.testing.assert_close(K().linear(strided, w, b, shuffled=ws), K().linear(strided, w, b), atol=0, rtol=0)


@pytest.mark.parametrize("M", [1, 2, 8, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("N,Kd", [(1000, 1184), (4608, 3584), (136, 8), (50, 264), (3584, 18944), (5120, 1184), (2090, 72),
                                  (5120, 9728)])
def test_linear_few_rows_bfloat16(M, N, Kd):
    """The streaming MFMA kernels (up to 16 rows, and 17 to 64): N no multiple of 16 or 128, K with a
    partial chunk, K cut into shares; numbers of tiles that fill the CUs unevenly (224, 288, 320, 131),
    the last with a K so long that few rows too go to the kernel that cuts K into shares."""
    assert K()._few_rows_go_to_rows64(N, Kd) == ((N, Kd) == (5120, 9728))
    torch.manual_seed(M + N)
    a = torch.randn(M, Kd, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(torch.bfloat16)
    b = torch.randn(N, device=DEV)
    want = a.double() @ w.double().T + b.double()
    ws = K().shuffle_weight(w)
    got = K().linear(a, w, b, out_dtype=torch.float32, shuffled=ws)
    torch.testing.assert_close(got.double(), want, atol=2e-4 * math.sqrt(Kd / 1000 + 1), rtol=2e-4)
    got16 = K().linear(a, w, b, shuffled=ws)
    torch.testing.assert_close(got16.double(), want, atol=3e-2, rtol=3e-2)
    # the value of a row does not depend on the rows beside it
    alone = K().linear(a[M - 1:M].contiguous(), w, b, out_dtype=torch.float32, shuffled=ws)
    same_class = M <= 16          # up to 16 rows run the same code with the same split of K: same bits
    t = 0 if same_class else 2e-4 * math.sqrt(Kd / 1000 + 1)
    torch.testing.assert_close(alone[0], got[M - 1], atol=t, rtol=t)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [1, 8, 40, 64, 200])
@pytest.mark.parametrize("I,Kd", [(176, 64), (1184, 3584), (100, 48), (48, 136)])
def test_swiglu_gate_up(dtype, M, I, Kd):
    torch.manual_seed(M + I)
    h = torch.randn(M, Kd, device=DEV).to(dtype)
    w = (torch.randn(2 * I, Kd, device=DEV) / math.sqrt(Kd) * 2).to(dtype)
    got = K().swiglu_gate_up(h, w, K().shuffle_weight(w))
    gu = h.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
    assert got.dtype == dtype and tuple(got.shape) == (M, I)
    # float32 accumulation over K terms: the error grows with sqrt(K)
    torch.testing.assert_close(got.double(), want, **tol(dtype, 2e-6 * math.sqrt(Kd) + 1e-5, 4e-2))


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_strided_rows(dtype):
    torch.manual_seed(1)
    big = torch.randn(9, 300, device=DEV).to(dtype)
    a = big[:, 20:120]
    w = torch.randn(33, 100, device=DEV).to(dtype)
    got = K().linear(a, w, None, out_dtype=torch.float32)
    torch.testing.assert_close(got.double(), a.double() @ w.double().T, **tol(dtype, 2e-5, 2e-5))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,rot", [(14, 2, 64, 64), (5, 1, 48, 48), (4, 4, 16, 8), (28, 4, 128, 128)])
def test_rope_store(dtype, nq, nkv, d, rot):
    torch.manual_seed(0)
    T, bs, pages, theta = 37, 8, 12, 50000.0
    qkv = torch.randn(T, (nq + 2 * nkv) * d, device=DEV).to(dtype)
    pos = torch.randint(0, 3000, (T,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * bs, device=DEV)[:T].to(torch.int32)
    slots[5] = -1
    kc = torch.full((pages, bs, nkv, d), 7.0, device=DEV).to(dtype)
    vc = torch.full((pages, nkv, d, bs), 7.0, device=DEV).to(dtype)       # values: transposed within the page
    i = torch.arange(0, rot, 2, dtype=torch.float64)
    inv_freq = (theta ** (-i / rot)).float().to(DEV)
    heads = qkv.float().cpu().view(T, nq + 2 * nkv, d)
    want_q = plain.rope(heads[:, :nq], pos.cpu(), theta, rot)
    want_k = plain.rope(heads[:, nq:nq + nkv], pos.cpu(), theta, rot)
    want_v = heads[:, nq + nkv:]
    K().rope_store(qkv, pos, inv_freq, nq, nkv, d, kc, vc, slots)
    got = qkv.float().cpu().view(T, nq + 2 * nkv, d)
    t = tol(dtype, 2e-5, 2e-2)
    torch.testing.assert_close(got[:, :nq], want_q, **t)
    kf, vf = kc.float().cpu().view(-1, nkv, d), vc.float().cpu().permute(0, 3, 1, 2).reshape(-1, nkv, d)
    ok = slots.cpu() >= 0
    torch.testing.assert_close(kf[slots.cpu()[ok].long()], want_k[ok], **t)
    torch.testing.assert_close(vf[slots.cpu()[ok].long()], want_v[ok], atol=0, rtol=0)
    untouched = torch.ones(pages * bs, dtype=torch.bool)
    untouched[slots.cpu()[ok].long()] = False
    assert torch.all(kf[untouched] == 7.0) and torch.all(vf[untouched] == 7.0)
    # position 0 is the identity
    qkv0 = torch.randn(3, (nq + 2 * nkv) * d, device=DEV).to(dtype)
    keep = qkv0.clone()
    K().rope_store(qkv0, torch.zeros(3, dtype=torch.int32, device=DEV), inv_freq, nq, nkv, d, None, None, None)
    torch.testing.assert_close(qkv0, keep, atol=0, rtol=0)
    # an owed bias: the same as adding it beforehand (in float32: to the bit)
    bias = torch.randn((nq + 2 * nkv) * d, device=DEV)
    outs = []
    for owed in (True, False):
        x = qkv.clone() if owed else (qkv.float() + bias).to(dtype)      # qkv holds rotated queries by now: any input will do
        kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
        K().rope_store(x, pos, inv_freq, nq, nkv, d, kc2, vc2, slots, bias if owed else None)
        outs.append((x[:, :nq * d], kc2, vc2))
    for a, b in zip(*outs):
        if dtype == torch.float32:
            torch.testing.assert_close(a, b, atol=0, rtol=0)
        else:
            torch.testing.assert_close(a.float(), b.float(), atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("M", [1, 5, 16, 17, 40, 64])
@pytest.mark.parametrize("nq,nkv,d,Kd", [(6, 2, 32, 192), (28, 4, 128, 3584), (4, 4, 64, 264), (5, 1, 96, 120)])
def test_fused_projection_rotation_and_cache_write(M, nq, nkv, d, Kd):
    """One kernel for q/k/v projection + bias + RoPE + cache write against the three separate kernels."""
    torch.manual_seed(M + nq)
    bs, pages, theta = 8, 12, 1e6
    pages = max(pages, M // bs + 4)
    N = (nq + 2 * nkv) * d
    h = torch.randn(M, Kd, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(torch.bfloat16)
    b = torch.randn(N, device=DEV)
    pos = torch.randint(0, 4000, (M,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * bs, device=DEV)[:M].to(torch.int32)
    if M > 2:
        slots[2] = -1
    inv_freq = (theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)).float().to(DEV)
    mk = lambda: (torch.full((pages, bs, nkv, d), 7.0, device=DEV).to(torch.bfloat16),
                  torch.full((pages, nkv, d, bs), 7.0, device=DEV).to(torch.bfloat16))
    kc, vc = mk()
    q = K().qkv_rope_store(h, K().shuffle_weight(w), b, pos, inv_freq, nq, nkv, d, kc, vc, slots)
    if M > 16 and K().library().tl_gemm_rows64_shares(M, N, Kd) == 1:
        assert q is None                                      # K too short to be cut: the separate kernels serve
        return
    assert q is not None and tuple(q.shape) == (M, nq * d)
    # the same from the plain formulas in float64
    qkv = (h.double() @ w.double().T + b.double()).cpu().view(M, nq + 2 * nkv, d)
    want_q = plain.rope(qkv[:, :nq], pos.cpu(), theta)
    want_k = plain.rope(qkv[:, nq:nq + nkv], pos.cpu(), theta)
    torch.testing.assert_close(q.double().cpu().view(M, nq, d), want_q, atol=3e-2, rtol=3e-2)
    ok = slots.cpu() >= 0
    sl = slots.cpu()[ok].long()
    kf = kc.double().cpu().view(-1, nkv, d)
    vf = vc.double().cpu().permute(0, 3, 1, 2).reshape(-1, nkv, d)
    torch.testing.assert_close(kf[sl], want_k[ok], atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(vf[sl], qkv[:, nq + nkv:][ok], atol=3e-2, rtol=3e-2)
    untouched = torch.ones(pages * bs, dtype=torch.bool)
    untouched[sl] = False
    assert torch.all(kf[untouched] == 7.0) and torch.all(vf[untouched] == 7.0)
    # cases it declines: float32, too many rows, partial rotation
    assert K().qkv_rope_store(h.float(), None, b, pos, inv_freq, nq, nkv, d, kc, vc, slots) is None
    assert K().qkv_rope_store(h, K().shuffle_weight(w), b, pos, inv_freq[: d // 4].contiguous(), nq, nkv, d, kc, vc, slots) is None


def _normed_rows(h, gamma, eps, parts):
    """NormedRows of float rows ``h`` as a product's residual sink would leave them, with the sum of
    squares cut into ``parts`` uneven partials."""
    M, H = h.shape
    cuts = sorted(set([0, H] + torch.randint(1, H, (parts - 1,)).tolist()))
    ss = torch.stack([(h[:, a:b].double() ** 2).sum(1) for a, b in zip(cuts[:-1], cuts[1:])], 0).float()
    return K().NormedRows((h * gamma).to(torch.bfloat16), ss.contiguous(), H, eps)


@pytest.mark.parametrize("M", [1, 7, 16, 17, 40, 64])
@pytest.mark.parametrize("N,Kd,parts", [(176, 64, 4), (1000, 1184, 74), (3584, 3584, 224), (50, 264, 1), (37888, 3584, 14),
                                        (5120, 9728, 38)])
def test_products_apply_an_owed_norm(M, N, Kd, parts):
    """A product of rows h * g with the division by rms(h) owed equals the product of RMSNorm(h) * g:
    plain, gate/up with SiLU, and q/k/v with rotation and cache write."""
    torch.manual_seed(M * 1000 + N)
    eps = 1e-5
    h = torch.randn(M, Kd, device=DEV) * torch.logspace(-1, 2, M, device=DEV)[:, None]   # rows of very different size
    if N > 30000 and M not in (16, 64):
        pytest.skip("the wide case is for the fullest row counts")
    gamma = 1 + 0.1 * torch.randn(Kd, device=DEV)
    owed = _normed_rows(h, gamma, eps, parts)
    rstd = 1 / torch.sqrt((h.double() ** 2).mean(1, keepdim=True) + eps)
    x = owed.rows.double() * rstd                        # what the product must multiply, given the rounded rows
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(torch.bfloat16)
    b = torch.randn(N, device=DEV)
    sh = K().shuffle_weight(w)
    got = K().linear(owed, w, b, out_dtype=torch.float32, shuffled=sh)
    torch.testing.assert_close(got.double(), x @ w.double().T + b.double(), atol=2e-3, rtol=2e-3)
    if N % 32 == 0:
        act = K().swiglu_gate_up(owed, w, sh)
        y = x @ w.double().T
        want = torch.nn.functional.silu(y[:, :N // 2]) * y[:, N // 2:]
        torch.testing.assert_close(act.double(), want, atol=2e-2, rtol=2e-2)
    with pytest.raises(K().KernelError, match="streaming"):
        K().linear(owed, w, b, out_dtype=torch.float32, shuffled=None)


@pytest.mark.parametrize("M,Kd", [(5, 192), (40, 1184)])
def test_fused_projection_applies_an_owed_norm(M, Kd):
    torch.manual_seed(3)
    nq, nkv, d, bs, pages, eps = 6, 2, 32, 8, 12, 1e-6
    N = (nq + 2 * nkv) * d
    h = torch.randn(M, Kd, device=DEV) * 30
    gamma = 1 + 0.1 * torch.randn(Kd, device=DEV)
    owed = _normed_rows(h, gamma, eps, 12)
    x = (owed.rows.double() / torch.sqrt((h.double() ** 2).mean(1, keepdim=True) + eps)).to(torch.bfloat16)
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(torch.bfloat16)
    b = torch.randn(N, device=DEV)
    pos = torch.randint(0, 4000, (M,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * bs, device=DEV)[:M].to(torch.int32)
    inv_freq = (1e6 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)).float().to(DEV)
    out = []
    for inp in (owed, x):
        kc = torch.zeros(pages, bs, nkv, d, device=DEV, dtype=torch.bfloat16)
        vc = torch.zeros(pages, nkv, d, bs, device=DEV, dtype=torch.bfloat16)
        q = K().qkv_rope_store(inp, K().shuffle_weight(w), b, pos, inv_freq, nq, nkv, d, kc, vc, slots)
        assert q is not None
        out.append((q, kc, vc))
    for a, c in zip(out[0], out[1]):                     # against the same kernel on rows normalised beforehand
        torch.testing.assert_close(a.float(), c.float(), atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("M", [1, 6, 16, 17, 33, 64])
@pytest.mark.parametrize("N,Kd", [(176, 64), (1000, 1184), (3584, 18944), (40, 264), (5000, 256), (5120, 520), (5120, 9728)])
def test_product_adds_into_the_residual_and_prepares_the_next_norm(M, N, Kd):
    torch.manual_seed(M + N)
    eps = 1e-6
    a = torch.randn(M, Kd, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(torch.bfloat16)
    b = torch.randn(N, device=DEV)
    gamma = 1 + 0.1 * torch.randn(N, device=DEV)
    resid0 = torch.randn(M, N, device=DEV) * 5
    resid = resid0.clone()
    nxt = K().linear(a, w, b, out_dtype=torch.float32, shuffled=K().shuffle_weight(w), sink=K().NormSink(resid, gamma, eps))
    want = resid0.double() + a.double() @ w.double().T + b.double()
    torch.testing.assert_close(resid.double(), want, atol=1e-3, rtol=1e-4)
    assert isinstance(nxt, K().NormedRows) and nxt.dim == N and nxt.eps == eps
    torch.testing.assert_close(nxt.rows.float(), (resid * gamma).to(torch.bfloat16).float(), atol=0, rtol=2 ** -7)
    assert nxt.sumsq.shape[1] == M and nxt.sumsq.shape[0] in (-(-N // 16), -(-N // 256))
    torch.testing.assert_close(nxt.sumsq.double().sum(0), (resid.double() ** 2).sum(1), atol=0, rtol=1e-5)
    # handed on: the next product's result equals that of the norm kernel followed by the product
    w2 = (torch.randn(48, N, device=DEV) / math.sqrt(N)).to(torch.bfloat16)
    got = K().linear(nxt, w2, None, out_dtype=torch.float32, shuffled=K().shuffle_weight(w2))
    x = K().add_rmsnorm(resid.clone(), None, gamma, eps, torch.bfloat16)
    want2 = K().linear(x, w2, None, out_dtype=torch.float32, shuffled=K().shuffle_weight(w2))
    torch.testing.assert_close(got, want2, atol=2e-2, rtol=2e-2)


def _attention_case(dtype, nq, nkv, d, bs, lens, q_lens=None, window=0, seed=0, spike=False, path=None, split_keys=None,
                    route_singles=None, pool_pages=None, spike_at=None):
    """Sequences of context ``lens``; the last ``q_lens[i]`` positions of each are queries.
    pool_pages: the sequences' pages are the last ones of a pool of that many.  ``spike``: the key
    at position 1 (or at ``spike_at(position of the query)``, if that is a key at all) is made to
    match its query, so that it dominates the sum if it is seen."""
    torch.manual_seed(seed)
    S = len(lens)
    q_lens = q_lens or [1] * S
    nb = max(-(-n // bs) for n in lens)
    num_blocks = S * nb + 8
    kc = torch.randn(num_blocks, bs, nkv, d, device=DEV).to(dtype)
    vc = torch.randn(num_blocks, nkv, d, bs, device=DEV).to(dtype)
    tables = torch.randperm(num_blocks, device=DEV)[:S * nb].view(S, nb).to(torch.int32)   # scattered pages
    if pool_pages:
        first = pool_pages - num_blocks
        big_k = torch.zeros(pool_pages, bs, nkv, d, dtype=dtype, device=DEV)
        big_v = torch.zeros(pool_pages, nkv, d, bs, dtype=dtype, device=DEV)
        big_k[first:], big_v[first:] = kc, vc
        kc, vc, tables = big_k, big_v, tables + first
    seq_of, pos = [], []
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        for p in range(n - ql, n):
            seq_of.append(s)
            pos.append(p)
    T = len(pos)
    q = torch.randn(T, nq * d, device=DEV).to(dtype)
    if spike:
        # one far key among hundreds must dominate: scale a query and a matching early key
        kflat = kc.view(-1, nkv, d)
        for t in range(T):
            s = seq_of[t]
            far = 1 if lens[s] > 2 else 0
            if spike_at is not None:
                far = spike_at(pos[t])
                if not 0 <= far < lens[s]:
                    continue
            row = int(tables[s, far // bs]) * bs + far % bs
            kflat[row] = (q[t].view(nq, d)[:nkv].float() * 4).to(dtype)
    from tensorline_amd.engine.batch import StepFacts
    qs = [0]
    for ql in q_lens:
        qs.append(qs[-1] + ql)
    plan = StepFacts(max_context=max(lens), max_query_len=max(q_lens), decode_only=max(q_lens) == 1,
                     num_seqs=S, q_lens=list(q_lens), starts=[n - ql for n, ql in zip(lens, q_lens)])
    single_seqs = None
    if K().one_token_sequences(plan):
        single_seqs = torch.tensor(K().one_token_sequences(plan), dtype=torch.int32, device=DEV)
    out = K().paged_attention(q, kc, vc, tables, torch.tensor(seq_of, dtype=torch.int32, device=DEV),
                              torch.tensor(pos, dtype=torch.int32, device=DEV), nq, nkv, d, d ** -0.5, window=window,
                              q_start=torch.tensor(qs, dtype=torch.int32, device=DEV),
                              ctx_start=torch.tensor(plan.starts, dtype=torch.int32, device=DEV), plan=plan,
                              path=path, split_keys=split_keys, single_seqs=single_seqs, route_singles=route_singles)
    if pool_pages:
        kc, vc, tables = kc[first:], vc[first:], tables - first
    kf, vf = kc.double().cpu().view(-1, nkv, d), vc.double().cpu().permute(0, 3, 1, 2).reshape(-1, nkv, d)
    want = torch.empty(T, nq, d, dtype=torch.float64)
    tcpu = tables.cpu().long()
    t0 = 0
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        keys = torch.arange(n)
        rows = tcpu[s][keys // bs] * bs + keys % bs
        qs = q[t0:t0 + ql].double().cpu().view(ql, nq, d)
        want[t0:t0 + ql] = plain.causal_attention(qs, kf[rows], vf[rows], d ** -0.5, window=window, q_offset=n - ql)
        t0 += ql
    return out.double().cpu().view(T, nq, d), want


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads", [(14, 2), (12, 2), (16, 2), (4, 4)])
@pytest.mark.parametrize("lens", [[1], [15, 16, 17], [63, 64, 65, 300], [1400] * 3 + [2, 129]])
def test_attention_decode_reference_cases(dtype, heads, lens):
    # the cases of the reference's kernel test (tests/test_paged_attn.py:22-38): D=64, page 16
    got, want = _attention_case(dtype, heads[0], heads[1], 64, 16, lens)
    torch.testing.assert_close(got, want, **tol(dtype, 2e-5, 1e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,bs", [(5, 1, 48, 16), (4, 2, 16, 8), (28, 4, 128, 16), (6, 2, 32, 8), (3, 3, 80, 4)])
def test_attention_portions_and_spike(dtype, nq, nkv, d, bs):
    lens, q_lens = [70, 9, 300, 2], [33, 9, 2, 1]
    got, want = _attention_case(dtype, nq, nkv, d, bs, lens, q_lens, spike=True, seed=3)
    torch.testing.assert_close(got, want, **tol(dtype, 3e-5, 2e-2))


def _pages_beyond_32_bits(bs, nkv, d):
    """Pages of a pool whose planes hold more than 2^31 elements (2^32 bytes and more)."""
    return (1 << 31) // (bs * nkv * d) + 4096


@pytest.mark.parametrize("dtype,path", [(torch.bfloat16, "mfma"), (torch.bfloat16, "generic"), (torch.float32, "generic")])
def test_attention_reads_pages_at_offsets_beyond_32_bits(dtype, path):
    """The sequences' pages are the last ones of a pool of several GB per plane: a page's offset in
    elements is above 2^31 and must be computed in 64 bits, in one-token steps and in portions."""
    nq, nkv, d, bs = 4, 2, 128, 16
    pool = _pages_beyond_32_bits(bs, nkv, d)
    try:
        for lens, q_lens in (([700, 33], None), ([300, 40, 65], [33, 40, 1])):
            got, want = _attention_case(dtype, nq, nkv, d, bs, lens, q_lens, spike=True, seed=11, path=path, pool_pages=pool)
            torch.testing.assert_close(got, want, **tol(dtype, 3e-5, 2e-2))
    finally:
        torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", DTYPES)
def test_cache_writes_at_offsets_beyond_32_bits(dtype):
    """The kernels that write the cache (rotation and store; the fused projections for few rows and
    for 17 to 64 rows) with slots on the last pages of a pool of several GB per plane leave there
    what they leave in a small pool, and nothing anywhere else."""
    nq, nkv, d, bs, Kd, small = 4, 2, 128, 16, 3584, 12
    pool = _pages_beyond_32_bits(bs, nkv, d)
    first = pool - small
    torch.manual_seed(4)
    inv_freq = (1e6 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)).float().to(DEV)
    N = (nq + 2 * nkv) * d
    try:
        big_k = torch.zeros(pool, bs, nkv, d, dtype=dtype, device=DEV)
        big_v = torch.zeros(pool, nkv, d, bs, dtype=dtype, device=DEV)
        for M in (5, 40):
            pos = torch.randint(0, 4000, (M,), dtype=torch.int32, device=DEV)
            slots = torch.randperm(small * bs, device=DEV)[:M].to(torch.int32)
            writers = [lambda kc, vc, sl: K().rope_store(qkv.clone(), pos, inv_freq, nq, nkv, d, kc, vc, sl)]
            qkv = torch.randn(M, N, device=DEV).to(dtype)
            if dtype == torch.bfloat16:
                h = torch.randn(M, Kd, device=DEV).to(dtype)
                ws = K().shuffle_weight((torch.randn(N, Kd, device=DEV) / math.sqrt(Kd)).to(dtype))
                b = torch.randn(N, device=DEV)
                fused = lambda kc, vc, sl: K().qkv_rope_store(h, ws, b, pos, inv_freq, nq, nkv, d, kc, vc, sl)
                assert fused(torch.zeros(small, bs, nkv, d, dtype=dtype, device=DEV),
                             torch.zeros(small, nkv, d, bs, dtype=dtype, device=DEV), slots) is not None
                writers.append(fused)
            for write in writers:
                kc = torch.zeros(small, bs, nkv, d, dtype=dtype, device=DEV)
                vc = torch.zeros(small, nkv, d, bs, dtype=dtype, device=DEV)
                write(kc, vc, slots)
                assert kc.abs().sum() > 0 and vc.abs().sum() > 0
                big_k[first:].zero_()
                big_v[first:].zero_()
                write(big_k, big_v, slots + first * bs)
                assert torch.equal(big_k[first:], kc) and torch.equal(big_v[first:], vc)
        # nothing was written below the last pages (a 32-bit offset would land there)
        assert not big_k[:first].any() and not big_v[:first].any()
    finally:
        del big_k, big_v
        torch.cuda.empty_cache()


@pytest.mark.parametrize("lens,split", [([33000], None), ([70001, 9], None), ([70001], 32)])
def test_attention_decode_long_contexts(lens, split):
    """Decoded tokens over tens of thousands of keys: hundreds of key splits, and beyond the most
    splits the merge takes the splits grow; a far key dominates."""
    got, want = _attention_case(torch.bfloat16, 28, 4, 128, 16, lens, None, spike=True, seed=5, path="mfma", split_keys=split)
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lens,split,d,bs", [([33000], None, 128, 16), ([5000, 9, 257], None, 48, 8), ([5000, 256], 512, 64, 24),
                                              ([1300, 70], 0, 128, 16), ([700, 9, 257], None, 256, 16), ([1025], None, 144, 24)])
def test_attention_any_shape_kernel_splits_keys_in_one_token_steps(dtype, lens, split, d, bs):
    """The any-shape kernel (the float32 path's attention) in steps of one token per sequence: keys in
    runs of 256 (or as asked) at absolute positions, a work-group per run, merged by a second kernel;
    a far key dominates, contexts of a few keys beside thousands, a context that ends exactly at a
    run's edge, pages of no power of two, head sizes above 128 (tiles of 32 keys: two of the four
    waves have a key block).  0: no split, the same kernel walking all keys."""
    got, want = _attention_case(dtype, 6, 2, d, bs, lens, None, spike=True, seed=11, path="generic", split_keys=split)
    torch.testing.assert_close(got, want, **tol(dtype, 3e-5, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 100, 101, 300])
@pytest.mark.parametrize("split", [None, 64])
def test_attention_any_shape_kernel_window_with_split_keys(dtype, window, split):
    """A window in steps of one token per sequence on the any-shape kernel, where the keys are split
    into runs: the window's first key inside a run (700 keys, window 100: key 600 of the run from
    512), exactly on a run's edge (357 keys, window 101: key 256), whole leading runs empty, a
    window longer than the context.  The key just outside the window matches its query: seen, it
    would carry the sum."""
    lens = [700, 257, 256, 9, 357]
    got, want = _attention_case(dtype, 6, 2, 32, 8, lens, None, window=window, seed=21, spike=True, path="generic",
                                split_keys=split, spike_at=lambda p: p - window)
    torch.testing.assert_close(got, want, **tol(dtype, 3e-5, 2e-2))
    inside, _ = _attention_case(dtype, 6, 2, 32, 8, lens, None, window=window, seed=21, spike=True, path="generic",
                                split_keys=split, spike_at=lambda p: p - window + 1)
    if window > 1:
        assert not torch.allclose(inside, got, atol=1e-3)      # the same key one place further in is seen, and shows


@pytest.mark.parametrize("d,bs", [(128, 8), (128, 16), (128, 32), (128, 64), (128, 128), (128, 24), (64, 8), (64, 16),
                                  (64, 32), (64, 64), (32, 16), (32, 32), (32, 64), (32, 256)])
def test_attention_prompt_tiles_page_sizes_and_long_tables(d, bs):
    """Prompt portions on the kernel that stages 64-key tiles in LDS: pages smaller than, equal to
    and larger than a tile, a page table of more than 512 entries (8 and 16-token pages), a far key
    that dominates, a portion that starts and ends inside a tile, a short sequence beside it.  Pages
    of 24 tokens (no power of two) take the independent-wave kernel instead.  Where the 64 units of
    each of a wave's loads lie in one page (head size x page size >= 2048) the loader works with one
    page id per load, and the values' tile in LDS is cut by pages; elsewhere with one per lane."""
    lens, q_lens = [9000, 131, 70], [300, 131, 3]
    # 16 columns per wave, one chain of tiles per work-group and two; 32 (head sizes 64 and 128, else as before)
    for path in ("mfma-tile16", "mfma-tile16x2", "mfma-tile32"):
        got, want = _attention_case(torch.bfloat16, 28, 4, d, bs, lens, q_lens, spike=True, seed=bs, path=path)
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("path", ["generic", "mfma", "mfma-direct", "mfma-tile16x2", "mfma-tile32"])
@pytest.mark.parametrize("heads", [(14, 2), (12, 2), (16, 2), (4, 4), (28, 4)])
@pytest.mark.parametrize("d", [32, 64, 128])
def test_attention_matrix_core_kernel(path, heads, d):
    """The matrix-core kernel against the plain attention: decode rows and prompt portions in one
    batch, scattered pages, a key that dominates, contexts around block and page edges, and the
    key range split 1, 3 and many ways."""
    dtype = torch.bfloat16
    lens = [1, 31, 32, 33, 65, 300, 1400, 2, 129]
    q_lens = [1, 1, 32, 5, 64, 1, 9, 2, 100]
    for split_keys in (0, 32, 96, None):
        got, want = _attention_case(dtype, heads[0], heads[1], d, 16, lens, q_lens, seed=7, spike=True, path=path,
                                    split_keys=split_keys)
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
    lens = [63, 64, 65, 300, 1400, 1400, 17]                  # decode only, page of 8
    for split_keys in (0, 64, 256, None):
        got, want = _attention_case(dtype, heads[0], heads[1], d, 8, lens, seed=8, path=path, split_keys=split_keys)
        torch.testing.assert_close(got, want, atol=1e-2, rtol=1e-2)
    for window in (1, 7, 32, 100):
        for split_keys in (0, 64):
            got, want = _attention_case(dtype, heads[0], heads[1], d, 16, [50, 7, 130, 700], [20, 7, 1, 33],
                                        window=window, seed=9, path=path, split_keys=split_keys)
            torch.testing.assert_close(got, want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("heads", [(14, 2), (4, 4), (28, 4), (40, 2)])
@pytest.mark.parametrize("d,bs", [(32, 16), (64, 24), (128, 16), (128, 8)])
def test_attention_one_token_sequences_beside_prompt_portions(heads, d, bs):
    """In a step with prompt portions the one-token sequences may be computed by a launch of their
    own with split keys (they are, by default, when their contexts are long beside the portions): first,
    last and between portions, contexts of one key and of thousands, a dominating far key, a
    window, pages of no power of two (where the portions run on independent waves)."""
    dtype = torch.bfloat16
    lens = [5000, 40, 1, 1400, 700, 31, 2, 1025]
    q_lens = [1, 40, 1, 1, 300, 1, 2, 1]
    for window in (0, 100):
        outs = []
        for route in (True, False, None):
            got, want = _attention_case(dtype, heads[0], heads[1], d, bs, lens, q_lens, window=window, seed=11,
                                        spike=window == 0, route_singles=route)
            torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
            outs.append(got)
        # the same with the portions on the kernel of 32 columns per wave
        got, want = _attention_case(dtype, heads[0], heads[1], d, bs, lens, q_lens, window=window, seed=11,
                                    spike=window == 0, route_singles=True, path="mfma-tile32")
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
        if window == 0:
            assert torch.equal(outs[0], outs[2])              # 5,000 keys: routed when left to choose
        portion_rows = [r for r in range(sum(q_lens)) if r not in (0, 41, 42, 343, sum(q_lens) - 1)]
        assert torch.equal(outs[0][portion_rows], outs[1][portion_rows])
    short = _attention_case(dtype, heads[0], heads[1], d, bs, [500, 40, 9], [1, 40, 1], seed=12, route_singles=None)
    unrouted = _attention_case(dtype, heads[0], heads[1], d, bs, [500, 40, 9], [1, 40, 1], seed=12, route_singles=False)
    assert torch.equal(short[0], unrouted[0])                 # short contexts stay with the portions


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 7, 16, 100])
def test_attention_window(dtype, window):
    got, want = _attention_case(dtype, 6, 2, 32, 8, [50, 7, 130], [20, 7, 1], window=window, seed=5)
    torch.testing.assert_close(got, want, **tol(dtype, 2e-5, 1e-2))


def test_attention_special_cases():
    # one key: o = v;  q = 0: o = mean of the visible values
    dtype, nq, nkv, d, bs = torch.float32, 4, 2, 16, 8
    kc = torch.randn(4, bs, nkv, d, device=DEV)
    vc = torch.randn(4, nkv, d, bs, device=DEV)
    tables = torch.tensor([[2, 0]], dtype=torch.int32, device=DEV)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    q = torch.randn(1, nq * d, device=DEV)
    o = K().paged_attention(q, kc, vc, tables, z, z, nq, nkv, d, 0.25).view(nq, d)
    torch.testing.assert_close(o, vc[2, :, :, 0].repeat_interleave(2, 0), atol=1e-6, rtol=1e-6)
    p = torch.tensor([10], dtype=torch.int32, device=DEV)
    o = K().paged_attention(torch.zeros_like(q), kc, vc, tables, z, p, nq, nkv, d, 0.25).view(nq, d)
    vis = torch.cat([vc[2].permute(2, 0, 1), vc[0].permute(2, 0, 1)[:3]]).mean(0)
    torch.testing.assert_close(o, vis.repeat_interleave(2, 0), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    torch.manual_seed(0)
    gu = (torch.randn(9, 2 * 176, device=DEV) * 3).to(dtype)
    got = K().silu_mul(gu)
    g, u = gu[:, :176].double(), gu[:, 176:].double()
    torch.testing.assert_close(got.double(), torch.nn.functional.silu(g) * u, **tol(dtype, 1e-5, 2e-2))


def test_argmax_and_ties():
    torch.manual_seed(0)
    lg = torch.randn(6, 1000, device=DEV)
    lg[2, 17] = lg[2, 900] = 50.0        # tie: the lower index wins
    got = K().argmax(lg)
    want = lg.argmax(-1)
    want[2] = 17
    assert got.tolist() == want.tolist()
    big = torch.randn(3, 152064, device=DEV)
    assert K().argmax(big).tolist() == big.argmax(-1).tolist()


def test_sample_keep_rule_and_draws():
    # hand vector of the keep rule: p = [.5, .3, .2]; top_p .5 keeps one token, .51 keeps two
    lg = torch.log(torch.tensor([[0.5, 0.3, 0.2]], device=DEV))
    one = torch.ones(1, device=DEV)
    for tp, u, want in [(0.5, 0.99, 0), (0.51, 0.99, 1), (0.51, 0.1, 0), (0.81, 0.99, 2), (1.0, 0.99, 2), (1.0, 0.6, 1)]:
        got = K().sample(lg, one, one * tp, one * u)
        assert got.tolist() == [want], (tp, u, got.tolist())
    # greedy rows inside a sampling batch, and agreement with the plain rule on random rows
    torch.manual_seed(1)
    R, V = 64, 1000
    lg = torch.randn(R, V, device=DEV) * 3
    temp = torch.rand(R, device=DEV) + 0.3
    temp[::7] = 0.0
    tp = torch.rand(R, device=DEV) * 0.9 + 0.1
    tp[::5] = 1.0
    u = torch.rand(R, device=DEV)
    got = K().sample(lg, temp, tp, u).tolist()
    miss = 0
    for r in range(R):
        want = plain.sample_with_uniform(lg[r].cpu(), float(temp[r]), float(tp[r]), float(u[r]))
        if temp[r] <= 0:
            assert got[r] == want
        elif got[r] != want:
            # a float32 running sum may land on the other side of a boundary next to the target
            probs = torch.softmax(lg[r].double().cpu() / float(temp[r]), -1)
            if tp[r] < 1:
                assert plain.top_p_keep(probs, float(tp[r]))[got[r]], "drew a token outside the kept set"
            miss += 1
    assert miss <= 2
    # same inputs, same tokens, whatever else is in the batch
    again = K().sample(lg[10:20].contiguous(), temp[10:20].contiguous(), tp[10:20].contiguous(), u[10:20].contiguous())
    assert again.tolist() == got[10:20]


def test_sample_wide_rows_ties_and_masked_logits():
    """Rows of several chunks: agreement with the plain rule, a row of equal logits (the kept set is
    a number of ties, lowest indices first), a row with all but two logits at -inf, a dominant token."""
    torch.manual_seed(4)
    V = 10007
    R = 12
    lg = torch.randn(R, V, device=DEV) * 4
    temp = torch.rand(R, device=DEV) * 1.2 + 0.2
    tp = torch.rand(R, device=DEV) * 0.95 + 0.04
    tp[::4] = 1.0
    u = torch.rand(R, device=DEV)
    got = K().sample(lg, temp, tp, u).tolist()
    miss = 0
    for r in range(R):
        want = plain.sample_with_uniform(lg[r].cpu(), float(temp[r]), float(tp[r]), float(u[r]))
        if got[r] != want:
            probs = torch.softmax(lg[r].double().cpu() / float(temp[r]), -1)
            if tp[r] < 1:
                assert plain.top_p_keep(probs, float(tp[r]))[got[r]], "drew a token outside the kept set"
            miss += 1
    assert miss <= 1
    # equal logits: top_p 0.3 keeps tokens while k / V < 0.3, that is the first 3003; u picks evenly among them
    us = torch.tensor([0.0, 0.25, 0.5, 0.999999], device=DEV)
    n = us.numel()
    flat = torch.zeros(n, V, device=DEV)
    got = K().sample(flat, torch.ones(n, device=DEV), torch.full((n,), 0.3, device=DEV), us).tolist()
    assert got == [int(float(x) * 3003) for x in us.tolist()]
    got = K().sample(flat, torch.ones(n, device=DEV), torch.ones(n, device=DEV), us).tolist()
    assert got == [int(float(x) * V) for x in us.tolist()]
    # two live tokens far apart, the rest -inf: p = (0.25, 0.75)
    two = torch.full((3, V), float("-inf"), device=DEV)
    two[:, 5000] = math.log(0.25)
    two[:, 9999] = math.log(0.75)
    one = torch.ones(3, device=DEV)
    assert K().sample(two, one, one, torch.tensor([0.1, 0.3, 0.9], device=DEV)).tolist() == [5000, 9999, 9999]
    assert K().sample(two, one, one * 0.7, torch.tensor([0.1, 0.3, 0.9], device=DEV)).tolist() == [9999] * 3
    # the vocabulary of the 7B shape: a dominant token wins whatever u is
    big = torch.randn(2, 152064, device=DEV)
    big[0, 151000] = 60.0
    big[1, 3] = 60.0
    assert K().sample(big, torch.ones(2, device=DEV), torch.tensor([0.9, 1.0], device=DEV),
                      torch.tensor([0.9999, 0.5], device=DEV)).tolist() == [151000, 3]


def test_sample_frequencies():
    torch.manual_seed(2)
    V, R = 50, 20000
    row = torch.randn(V, device=DEV) * 2
    lg = row.repeat(R, 1)
    u = torch.rand(R, device=DEV)
    t = torch.full((R,), 0.8, device=DEV)
    got = K().sample(lg, t, torch.ones(R, device=DEV), u)
    freq = torch.bincount(got.long(), minlength=V).double().cpu() / R
    probs = torch.softmax(row.double().cpu() / 0.8, -1)
    assert (freq - probs).abs().max() < 0.015
    # temperature -> 0+ is arg-max
    cold = K().sample(lg[:4], torch.full((4,), 1e-4, device=DEV), torch.ones(4, device=DEV), u[:4])
    assert cold.tolist() == [int(row.argmax())] * 4


def test_bad_arguments_are_refused():
    from tensorline_amd.ops.kernels import KernelError
    with pytest.raises(KernelError):
        K().linear(torch.randn(2, 8, device=DEV), torch.randn(4, 9, device=DEV))
    with pytest.raises(KernelError):
        K().embed(torch.zeros(2, dtype=torch.int64, device=DEV), torch.randn(4, 8, device=DEV))
    with pytest.raises(KernelError):
        K().add_rmsnorm(torch.randn(2, 8), None, torch.ones(8), 1e-6, torch.float32)
    with pytest.raises(KernelError):
        kc = torch.randn(2, 4, 1, 512, device=DEV)
        K().paged_attention(torch.randn(1, 512, device=DEV), kc, kc.permute(0, 2, 3, 1).contiguous(), torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                            torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                            1, 1, 512, 1.0)


def test_attention_long_portions_take_the_kernel_of_32_columns_per_wave(monkeypatch):
    """Left to choose, a long prompt portion behind thousands of keys runs on the kernel with 32
    columns per wave and work-groups of 256 columns, a short one on that with 16 and 128; both give
    the plain attention, a dominating far key included, and a prompt with a window too."""
    called = []
    call = K()._call
    monkeypatch.setattr(K(), "_call", lambda name, *a: (called.append(name), call(name, *a))[1])
    got, want = _attention_case(torch.bfloat16, 28, 4, 128, 16, [10000, 40], [1300, 40], spike=True, seed=4)
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
    assert called == ["tl_attention_tile32"]
    called.clear()
    got, want = _attention_case(torch.bfloat16, 28, 4, 128, 16, [3000, 40], [1300, 40], spike=True, seed=4)
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
    assert called == ["tl_attention_mfma"]
    got, want = _attention_case(torch.bfloat16, 8, 2, 64, 32, [9000], [1200], window=700, seed=5, path="mfma-tile32")
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


def test_attention_short_portions_behind_long_contexts_walk_their_keys_as_two_chains(monkeypatch):
    """Left to choose, a step with at most one work-group of 128 columns per CU and a walk of 16 tiles
    or more asks the prompt kernel for two chains of tiles per work-group, a step with more
    work-groups or only short walks for one; all give the plain attention where one far key
    dominates, with an odd number of tiles (the second chain has one fewer), a window, and a
    one-token sequence beside the portion."""
    asked = []
    call = K()._call
    monkeypatch.setattr(K(), "_call", lambda name, *a: (asked.append((name, a[25] if len(a) > 25 else None)), call(name, *a))[1])
    for lens, q_lens, window in (([4200, 40], [300, 40], 0), ([2900, 1], [64, 1], 0), ([1100], [33], 0), ([5000], [500], 700)):
        asked.clear()
        got, want = _attention_case(torch.bfloat16, 28, 4, 128, 16, lens, q_lens, window=window, spike=True, seed=6)
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
        assert asked == [("tl_attention_mfma", 2)], asked
    for lens, q_lens in (([3000, 40], [1300, 40]), ([60], [33]), ([1000, 9], [700, 9])):
        asked.clear()
        got, want = _attention_case(torch.bfloat16, 28, 4, 128, 16, lens, q_lens, spike=True, seed=4)
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
        assert asked == [("tl_attention_mfma", 1)], asked
