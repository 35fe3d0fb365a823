"""Each HIP kernel alone against a plain float64 torch computation of the same
operation, at sizes other than the tiny models': widths and vocabularies that are
no power of two, head sizes in steps of 16, MQA/GQA/MHA, fragmented block tables,
NaN-filled pages (a read of an unwritten or foreign slot poisons the result).
"""

from __future__ import annotations

import math
from types import SimpleNamespace

import pytest
import torch

import plain_qwen2 as plain
from qkv_reference import check_qkv, qkv_reference

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
    # one rounding to bfloat16 is 2^-9 relative; float32 kernels differ from float64 by ~1e-6
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=1e-2, rtol=1.6e-2)


@pytest.fixture(scope="module")
def ops_for(gpu_device):
    from mini_llm_runtime_amd.kernels.ops import HipOps

    cache = {}

    def get(dtype):
        if dtype not in cache:
            cache[dtype] = HipOps(dtype, gpu_device)
        return cache[dtype]

    return get


def _attend(ops, *args, **kw):
    """`paged_attention` with the launch plan that these tests keep on the batch description itself."""
    kw.setdefault("plan", args[4])
    return ops.paged_attention(*args, **kw)


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# ---- embedding, norm, elementwise -----------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(ops_for, dtype):
    ops = ops_for(dtype)
    table = _rand((517, 96), dtype, 1)
    ids = torch.tensor([0, 516, 3, 3, 200], dtype=torch.int32)
    out = ops.embedding(table.cuda(), ids.cuda()).cpu()
    assert out.dtype == torch.float32
    assert torch.equal(out, table[ids.long()].float())
    bad = ops.embedding(table.cuda(), torch.tensor([517, -1], dtype=torch.int32).cuda()).cpu()
    assert torch.isnan(bad).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [64, 96, 896, 1000, 5120])
@pytest.mark.parametrize("weight_f32", [False, True])
def test_rmsnorm(ops_for, dtype, hidden, weight_f32):
    ops = ops_for(dtype)
    x = _rand((5, hidden), torch.float32, 2, 3.0)
    delta = _rand((5, hidden), dtype, 3)
    w = (1 + _rand((hidden,), torch.float32, 4, 0.1)).to(torch.float32 if weight_f32 or dtype == torch.float32 else dtype)
    eps = 1e-5
    ref = plain.rms_norm(x.double(), w.double(), eps)
    got = ops.rmsnorm(x.cuda().clone(), w.cuda(), eps).cpu()
    assert got.dtype == dtype
    torch.testing.assert_close(got.double(), ref, **_tol(dtype))
    xd = x.cuda().clone()
    got = ops.rmsnorm(xd, w.cuda(), eps, delta=delta.cuda()).cpu()
    summed = x.double() + delta.double()
    torch.testing.assert_close(xd.cpu().double(), summed, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(got.double(), plain.rms_norm(summed, w.double(), eps), **_tol(dtype))


def test_rmsnorm_vectors(ops_for):
    """x=[3,4], w=[2,0.5], eps=0 and ones-stay-ones (reference tests/test_manual_qwen_decoder_layer.py:8-18)."""
    ops = ops_for(torch.float32)
    x = torch.tensor([[3.0, 4.0]]).cuda()
    got = ops.rmsnorm(x, torch.tensor([2.0, 0.5]).cuda(), 0.0).cpu()
    rms = math.sqrt(12.5)
    torch.testing.assert_close(got, torch.tensor([[2 * 3 / rms, 0.5 * 4 / rms]]))
    ones = ops.rmsnorm(torch.ones(1, 8).cuda(), torch.ones(8).cuda(), 0.0).cpu()
    torch.testing.assert_close(ones, torch.ones(1, 8))


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_gather_silu(ops_for, dtype):
    ops = ops_for(dtype)
    x = _rand((7, 100), torch.float32, 5)
    d = _rand((7, 100), dtype, 6)
    xd = x.cuda().clone()
    ops.add_(xd, d.cuda())
    torch.testing.assert_close(xd.cpu(), x + d.float())
    rows = torch.tensor([6, 0, 3, 3], dtype=torch.int32)
    assert torch.equal(ops.gather_rows(x.cuda(), rows.cuda()).cpu(), x[rows.long()])
    assert torch.equal(ops.gather_rows(d.cuda(), rows.cuda()).cpu(), d[rows.long()])
    gu = _rand((9, 2 * 352), dtype, 7, 2.0)
    g, u = gu[:, :352].double(), gu[:, 352:].double()
    ref = g * torch.sigmoid(g) * u
    torch.testing.assert_close(ops.silu_mul(gu.cuda()).cpu().double(), ref, **_tol(dtype))
    # identity-weight SwiGLU vector: silu(x) * 2x (reference tests/test_manual_qwen_decoder_layer.py:21-36)
    xv = torch.tensor([[-1.0, 0.5, 2.0]])
    both = torch.cat([xv, 2 * xv], dim=1).to(dtype)
    ref = torch.nn.functional.silu(both[:, :3].double()) * both[:, 3:].double()
    torch.testing.assert_close(ops.silu_mul(both.cuda()).cpu().double(), ref, **_tol(dtype))


# ---- matrix product -----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 17, 8), (5, 64, 96), (63, 352, 129), (65, 517, 96), (200, 130, 1000), (2, 1152, 896)])
def test_linear(ops_for, dtype, m, n, k):
    ops = ops_for(dtype)
    x = _rand((m, k), dtype, 8)
    w = _rand((n, k), dtype, 9, 0.1)
    for bias_dtype in (None, dtype, torch.float32):
        b = None if bias_dtype is None else _rand((n,), bias_dtype, 10)
        ref = x.double() @ w.double().t() + (0 if b is None else b.double())
        for out_dtype in {dtype, torch.float32}:
            got = ops.linear(x.cuda(), w.cuda(), None if b is None else b.cuda(), out_dtype=out_dtype).cpu()
            assert got.dtype == out_dtype and got.shape == (m, n)
            tol = _tol(out_dtype if dtype == torch.bfloat16 else dtype)
            if dtype == torch.float32:
                tol = dict(atol=1e-4, rtol=1e-5)  # k-long float32 sums against float64
            torch.testing.assert_close(got.double(), ref, **tol)


@pytest.mark.parametrize(
    "m,n,k",
    [(1, 1152, 896), (8, 896, 4864), (3, 17, 8), (16, 130, 136), (17, 64, 96), (33, 517, 2056), (64, 9728, 896),
     (65, 100, 64), (128, 128, 64), (200, 352, 1000), (300, 1152, 896), (2048, 896, 4864), (129, 151936, 96)],
)
def test_linear_bf16_matrix_cores(ops_for, m, n, k):
    """The MFMA kernels (skinny for up to 64 tokens, tiled above) against float64 and against the FMA kernel."""
    ops = ops_for(torch.bfloat16)
    x = _rand((m, k), torch.bfloat16, 40)
    w = _rand((n, k), torch.bfloat16, 41, 0.05)
    b = _rand((n,), torch.float32, 42)
    ref = x.double() @ w.double().t() + b.double()
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    got32 = ops.linear(xd, wd, bd, out_dtype=torch.float32).cpu().double()
    # exact bfloat16 products, float32 accumulation: only the order of the k-long sums differs
    torch.testing.assert_close(got32, ref, atol=1e-3 * (k / 1000) ** 0.5 + 1e-4, rtol=1e-4)
    fma = ops.linear(xd, wd, bd, out_dtype=torch.float32, kernel="fma").cpu().double()
    torch.testing.assert_close(got32, fma, atol=1e-3 * (k / 1000) ** 0.5 + 1e-4, rtol=1e-4)
    got16 = ops.linear(xd, wd, None).cpu().double()
    torch.testing.assert_close(got16, ref - b.double(), **_tol(torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,inter,k", [(1, 352, 96), (8, 4864, 896), (40, 130, 64), (200, 352, 136), (300, 64, 1000)])
def test_linear_swiglu_epilogue(ops_for, dtype, m, inter, k):
    """silu(gate) * up as the product's epilogue over rows woven in pairs (g g u u ...), on every
    kernel: matrix cores (skinny and tiled) and plain FMA."""
    ops = ops_for(dtype)
    x = _rand((m, k), dtype, 43)
    gate = _rand((inter, k), dtype, 44, 0.1)
    up = _rand((inter, k), dtype, 45, 0.1)
    woven = torch.empty(2 * inter, k, dtype=dtype)
    idx = torch.arange(inter)
    woven[(idx // 2) * 4 + idx % 2] = gate
    woven[(idx // 2) * 4 + 2 + idx % 2] = up
    g = x.double() @ gate.double().t()
    ref = g * torch.sigmoid(g) * (x.double() @ up.double().t())
    for kernel in ("auto", "fma"):
        got = ops.linear(x.cuda(), woven.cuda(), None, swiglu=True, kernel=kernel).cpu()
        assert got.shape == (m, inter)
        tol = dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else _tol(dtype)
        torch.testing.assert_close(got.double(), ref, **tol)


@pytest.mark.parametrize(
    "m,n,k",
    [(1, 896, 4864), (8, 896, 896), (16, 130, 2056), (33, 517, 2056), (64, 896, 4864), (8, 151936, 96),
     (300, 517, 4104), (2048, 896, 4864), (130, 130, 1032), (1000, 1030, 8200), (2040, 3000, 8192),
     (520, 1030, 9480), (96, 3584, 3584)],
)
def test_linear_partial_sums_feed_the_norm(ops_for, m, n, k):
    """A narrow product of a few tokens may come back as float32 partial sums over slices of k;
    the norm kernel adds them, in order, to the residual stream."""
    ops = ops_for(torch.bfloat16)
    x = _rand((m, k), torch.bfloat16, 46)
    w = _rand((n, k), torch.bfloat16, 47, 0.05)
    b = _rand((n,), torch.float32, 48)
    ref = x.double() @ w.double().t() + b.double()
    got = ops.linear(x.cuda(), w.cuda(), b.cuda(), partial_sums=True)
    if got.dim() == 3:
        assert got.dtype == torch.float32 and got.shape[1:] == (m, n) and got.shape[0] > 1
        total = got.cpu().double().sum(0)
    else:
        assert got.shape == (m, n)  # wide enough: not cut
        total = got.cpu().double()
    torch.testing.assert_close(total, ref, **(_tol(torch.bfloat16) if got.dim() == 2 else dict(atol=2e-3, rtol=1e-4)))
    if k >= 4104 and (m <= 300 or k >= 8192):
        assert got.dim() == 3, "a long, narrow product should be cut along k"
    stream = _rand((m, n), torch.float32, 49, 2.0)
    nw = (1 + _rand((n,), torch.float32, 50, 0.1)).to(torch.bfloat16)
    sd = stream.cuda().clone()
    h = ops.rmsnorm(sd, nw.cuda(), 1e-6, delta=got).cpu()
    summed = stream.double() + (total if got.dim() == 3 else got.cpu().double())
    torch.testing.assert_close(sd.cpu().double(), summed, atol=1e-5, rtol=1e-6)
    torch.testing.assert_close(h.double(), plain.rms_norm(summed, nw.double(), 1e-6), **_tol(torch.bfloat16))
    again = ops.linear(x.cuda(), w.cuda(), b.cuda(), partial_sums=True)
    assert torch.equal(again, got), "partial sums must not depend on timing"
    rows = torch.tensor([m - 1, 0], dtype=torch.int32).cuda()
    picked = ops.gather_rows(got, rows).cpu()
    assert torch.equal(picked, got.cpu()[..., [m - 1, 0], :])


def test_k_slices_chosen_for_many_tokens(ops_for):
    """The estimate that picks a tiling and a number of k slices for more than 64 tokens: never more
    slices than the consumer takes or than keep a few steps of k each, one slice for a wide
    product that fills the compute units by itself, several for a narrow one with a long k."""
    lib = ops_for(torch.bfloat16).lib
    for m in (65, 96, 300, 1000, 2048, 16384):
        for n, k in ((896, 896), (896, 4864), (3584, 18944), (37888, 3584), (130, 520), (5120, 27648)):
            for most in (1, 2, 3, 8):
                slices = lib.mlr_gemm_bf16_slices(m, n, k, most)
                assert 1 <= slices <= min(most, 4)
                assert slices == 1 or (k + 63) // 64 // slices >= 3
    assert lib.mlr_gemm_bf16_slices(2048, 37888, 3584, 8) == 1
    assert lib.mlr_gemm_bf16_slices(1024, 3584, 18944, 8) > 1
    assert lib.mlr_gemm_bf16_slices(96, 3584, 18944, 8) > 1


@pytest.mark.parametrize("kernel", [16, 14, 11, 22, 23, 44, 45, 46, 47, 48, 62, 63, 64, 65, 66, 67, 68])
@pytest.mark.parametrize("slices", [1, 3])
def test_each_matrix_core_kernel_at_odd_sizes(ops_for, kernel, slices):
    """Every bfloat16 kernel forced at sizes that are no multiple of its tile, with a tail of k
    shorter than an LDS slice, whole and cut along k."""
    ops = ops_for(torch.bfloat16)
    m, n, k = (13 if kernel == 16 else (300 if 44 <= kernel < 60 else 150)), (203 if kernel < 44 else 530), 1208
    x = _rand((m, k), torch.bfloat16, 61)
    w = _rand((n, k), torch.bfloat16, 62, 0.05)
    b = _rand((n,), torch.float32, 63)
    ref = x.double() @ w.double().t() + b.double()
    got = ops.linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, partial_sums=True, mfma_kernel=kernel, slices=slices)
    assert got.shape == ((slices, m, n) if slices > 1 else (m, n))
    total = got.cpu().double().sum(0) if slices > 1 else got.cpu().double()
    torch.testing.assert_close(total, ref, atol=2e-3, rtol=1e-4)
    if kernel != 16:
        with pytest.raises(Exception, match="64 tokens"):
            ops.linear(x.cuda(), w.cuda(), mfma_kernel=16)


@pytest.mark.parametrize("kernel,m,n", [(44, 2080, 1100), (44, 530, 3000), (44, 257, 256), (22, 1050, 700), (11, 532, 2373),
                                        (11, 90, 640), (44, 2112, 520), (44, 2113, 520), (45, 2080, 1100),
                                        (45, 530, 3000), (45, 257, 256), (23, 1050, 700), (23, 532, 2373), (23, 140, 640),
                                        (45, 2112, 520), (45, 2113, 520), (46, 2080, 1100), (46, 257, 192), (46, 2112, 520),
                                        (46, 2113, 400), (47, 2080, 1100), (47, 530, 3000), (47, 2176, 330), (47, 2177, 330), (48, 2080, 1100),
                                        (48, 2112, 700), (48, 2113, 330)])
@pytest.mark.parametrize("slices", [1, 2])
def test_tiles_with_few_tokens_at_the_lower_edge(ops_for, kernel, m, n, slices):
    """A last token tile whose tokens fit the first row of wavefronts (a prompt portion beside a few
    decoding requests) skips the matrix-core work of the others and is dealt out over the XCDs apart
    from the full tiles: every tile of every slice is still computed exactly once.  (Beside them: 64
    tokens in the last tile, which is light where a row of wavefronts has 64 tokens, and 65, which is
    not; 128 and 129 where it has 128.)"""
    ops = ops_for(torch.bfloat16)
    k = 200
    x = _rand((m, k), torch.bfloat16, 81)
    w = _rand((n, k), torch.bfloat16, 82, 0.05)
    b = _rand((n,), torch.float32, 83)
    ref = x.double() @ w.double().t() + b.double()
    got = ops.linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, partial_sums=True, mfma_kernel=kernel, slices=slices)
    total = got.cpu().double().sum(0) if slices > 1 else got.cpu().double()
    torch.testing.assert_close(total, ref, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("m,n,k,chosen", [(2048, 4608, 200, 47), (2048, 9728, 264, 48), (2048, 5120, 264, 47), (512, 37888, 520, 48)])
def test_narrower_tiles_where_square_ones_leave_units_idle(ops_for, m, n, k, chosen):
    """Products whose 256 x 256 tiles would not go round the compute units take tiles of 160, 192 or
    320 features by themselves (the 7B query/key/value width, the 0.5B gate-up width, the 32B output
    width, the 7B gate-up at 512 tokens); the
    result is the float64 product, and the same bits as when that kernel is forced."""
    ops = ops_for(torch.bfloat16)
    assert ops.lib.mlr_gemm_bf16_kernel(m, n, k, 1) == chosen
    x = _rand((m, k), torch.bfloat16, 91)
    w = _rand((n, k), torch.bfloat16, 92, 0.05)
    b = _rand((n,), torch.float32, 93)
    got = ops.linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32)
    torch.testing.assert_close(got.cpu().double(), x.double() @ w.double().t() + b.double(), atol=2e-3, rtol=1e-4)
    assert torch.equal(got, ops.linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, mfma_kernel=chosen))


@pytest.mark.parametrize("m,n,k,slices,chosen", [
    (64, 37888, 512, 1, 65), (41, 37890, 512, 1, 65), (64, 27648, 512, 1, 64), (50, 16000, 1024, 1, 62), (64, 55296, 512, 1, 67),
    (20, 55296, 1024, 1, 67), (8, 37888, 1024, 1, 65), (8, 37888, 512, 1, 14), (48, 59136, 512, 1, 68), (64, 17920, 512, 1, 63),
    (33, 24000, 512, 1, 11), (64, 3584, 18944, 8, 64), (32, 5120, 5120, 8, 65), (40, 896, 4864, 8, 11),
])
@pytest.mark.parametrize("swiglu", [False, True])
def test_tiles_for_up_to_64_tokens_chosen_by_rounds(ops_for, m, n, k, slices, chosen, swiglu):
    """Products of up to 64 tokens through tiles choose the tile width (64 to 256 features, straight
    into LDS, or the register-staged tiles of 64) by how the tiles go round the compute units and
    what a unit takes in; these shapes reach every width, whole and cut along k, some with a last
    tile that is not whole."""
    if swiglu and slices > 1:
        pytest.skip("partial sums have no SwiGLU")
    ops = ops_for(torch.bfloat16)
    n = n - n % 4 if swiglu else n
    assert ops.lib.mlr_gemm_bf16_kernel(m, n, k, slices) == chosen
    x = _rand((m, k), torch.bfloat16, 71)
    w = (torch.randn((n, k), generator=torch.Generator(device="cuda").manual_seed(72), device="cuda") * 0.05).to(torch.bfloat16)
    ref = x.cuda().double() @ w.double().t()
    if swiglu:
        quads = ref.view(m, -1, 4)
        gate, up = quads[..., :2], quads[..., 2:]
        ref = (gate * torch.sigmoid(gate) * up).reshape(m, -1)
    got = ops.linear(x.cuda(), w, None, swiglu=swiglu, out_dtype=None if swiglu else torch.float32, partial_sums=slices > 1, slices=slices if slices > 1 else None)
    total = got.double().sum(0) if got.dim() == 3 else got.double()
    scale = float(ref.abs().max())
    torch.testing.assert_close(total, ref, atol=(2e-2 if swiglu else 2e-3) * max(1.0, scale), rtol=2e-2 if swiglu else 1e-4)


@pytest.mark.parametrize("m", [17, 31, 32, 33, 50, 64])
@pytest.mark.parametrize("slices", [1, 4])
@pytest.mark.parametrize("swiglu", [False, True])
def test_row_splitting_kernel_takes_up_to_64_tokens(ops_for, m, slices, swiglu):
    """The streaming kernel with two and four slabs of 16 tokens (chosen for small matrices, forced
    here at a width that is no multiple of its 16 rows), whole, cut along k, and with SwiGLU."""
    if swiglu and slices > 1:
        pytest.skip("partial sums have no SwiGLU")
    ops = ops_for(torch.bfloat16)
    n, k = 204, 904
    x = _rand((m, k), torch.bfloat16, 64)
    w = _rand((n, k), torch.bfloat16, 65, 0.05)
    b = None if swiglu else _rand((n,), torch.float32, 66)
    ref = x.double() @ w.double().t() + (0 if b is None else b.double())
    if swiglu:
        quads = ref.view(m, -1, 4)
        ref = (quads[..., :2] * torch.sigmoid(quads[..., :2]) * quads[..., 2:]).reshape(m, -1)
    got = ops.linear(x.cuda(), w.cuda(), None if b is None else b.cuda(), out_dtype=torch.float32, partial_sums=slices > 1,
                     mfma_kernel=16, slices=slices, swiglu=swiglu)
    total = got.cpu().double().sum(0) if slices > 1 else got.cpu().double()
    torch.testing.assert_close(total, ref, atol=2e-3, rtol=1e-4)
    # and by itself for a small matrix: the same values as when forced
    if not swiglu:
        chosen = ops.linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32)
        assert torch.equal(chosen, ops.linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, mfma_kernel=16))


# ---- rotary encoding and cache write ----------------------------------------------------------------
def test_rope_table(ops_for):
    ops = ops_for(torch.float32)
    pos = torch.tensor([0, 1, 2, 17, 4095, 32767, 131071], dtype=torch.int32)
    inv = 1.0 / (1e6 ** (torch.arange(0, 64, 2, dtype=torch.float64) / 64))
    cos, sin = ops.rope_table(pos.cuda(), inv.cuda())
    ang = pos.double()[:, None] * inv[None]
    torch.testing.assert_close(cos.cpu().double(), ang.cos(), atol=1e-7, rtol=0)
    torch.testing.assert_close(sin.cpu().double(), ang.sin(), atol=1e-7, rtol=0)
    assert torch.equal(cos[0].cpu(), torch.ones(32)) and torch.equal(sin[0].cpu(), torch.zeros(32))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,rotary", [(4, 2, 16, 16), (3, 1, 32, 32), (14, 2, 64, 64), (8, 8, 128, 64), (2, 1, 48, 48),
                                                         (28, 4, 128, 128), (5, 1, 80, 80), (3, 2, 20, 20)])
def test_rope_kv_write(ops_for, dtype, heads, kv_heads, head_dim, rotary):
    ops = ops_for(dtype)
    tokens, bs, pages = 11, 8, 9
    width = (heads + 2 * kv_heads) * head_dim
    qkv = _rand((tokens, width), dtype, 11)
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 8, 9, 100, 5], dtype=torch.int32)
    theta = 10000.0
    inv = 1.0 / (theta ** (torch.arange(0, rotary, 2, dtype=torch.float64) / rotary))
    cos, sin = ops.rope_table(positions.cuda(), inv.cuda())
    g = torch.Generator().manual_seed(12)
    slots = torch.randperm(pages * bs, generator=g)[:tokens].to(torch.int32)
    slots[4] = -1  # writes nothing
    kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=dtype).cuda()
    vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=dtype).cuda()
    dev = qkv.cuda().clone()
    ops.rope_kv_write(dev, (cos, sin, rotary), slots.cuda(), kp, vp, num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs)
    out = dev.cpu()

    def rot(x):  # [T, H, d] float64 -> rotated first `rotary` dims
        y = x.clone()
        part = x[..., :rotary].transpose(0, 1)  # [H, T, r]
        y[..., :rotary] = plain.apply_rope(part, positions, theta).transpose(0, 1)
        return y

    q_ref = rot(qkv[:, : heads * head_dim].double().view(tokens, heads, head_dim))
    k_ref = rot(qkv[:, heads * head_dim : (heads + kv_heads) * head_dim].double().view(tokens, kv_heads, head_dim))
    v_ref = qkv[:, (heads + kv_heads) * head_dim :].double().view(tokens, kv_heads, head_dim)
    tol = _tol(dtype)
    torch.testing.assert_close(out[:, : heads * head_dim].double().view(tokens, heads, head_dim), q_ref, **tol)
    kc, vc = kp.cpu().double(), vp.cpu().double().transpose(2, 3)  # values are transposed inside a page
    written = torch.zeros(pages, bs, dtype=torch.bool)
    for t in range(tokens):
        s = int(slots[t])
        if s < 0:
            continue
        page, off = divmod(s, bs)
        written[page, off] = True
        torch.testing.assert_close(kc[page, :, off], k_ref[t], **tol)
        torch.testing.assert_close(vc[page, :, off], v_ref[t], atol=0, rtol=0)
    untouched = ~written[:, None, :, None].expand_as(kc)
    assert torch.isnan(kc[untouched]).all() and torch.isnan(vc[untouched]).all()
    # position 0 is the identity (reference tests/test_manual_qwen_attention.py:35-42)
    assert torch.equal(out[0, : heads * head_dim], qkv[0, : heads * head_dim])


_QKV_CASES = [
    (14, 2, 64, 896, 8, True, True), (3, 1, 16, 40, 1, True, True), (6, 3, 48, 104, 16, True, True),
    (4, 4, 80, 72, 5, False, True), (5, 1, 128, 136, 13, True, False),
    (14, 2, 64, 896, 64, True, True), (3, 1, 32, 104, 17, True, True), (2, 2, 16, 40, 33, True, True),
    (14, 2, 64, 896, 300, True, True, 0), (14, 2, 64, 896, 130, True, True, 11), (14, 2, 64, 896, 130, True, True, 22),
    (14, 2, 64, 896, 300, True, True, 44), (3, 1, 48, 104, 70, True, True, 11), (3, 1, 48, 104, 70, True, True, 22),
    (5, 3, 16, 40, 200, True, True, 44), (7, 1, 80, 72, 99, True, True, 22), (2, 2, 96, 136, 65, True, False, 11),
    (4, 4, 80, 72, 77, False, True, 22), (5, 1, 256, 136, 40, True, True, 11), (3, 3, 128, 264, 150, True, True, 44),
    (14, 2, 64, 896, 8, True, True, 8), (3, 1, 16, 40, 1, True, True, 8), (4, 4, 80, 72, 5, False, True, 8),
    (5, 1, 128, 136, 7, True, False, 8), (6, 3, 48, 1208, 3, True, True, 8), (14, 2, 64, 896, 8, True, True, 16),
    (6, 3, 48, 104, 5, True, True, 16), (28, 4, 128, 3584, 8, True, True, 0), (28, 4, 128, 3584, 8, True, True, 16),
]


@pytest.mark.parametrize(
    "heads,kv_heads,head_dim,hidden,tokens,rotate,write,kernel", [c if len(c) == 8 else c + (0,) for c in _QKV_CASES]
)
def test_fused_qkv_rotation_cache_write_equals_the_three_kernels(ops_for, heads, kv_heads, head_dim, hidden, tokens, rotate, write, kernel):
    """Product, bias, rotation and cache write run as one kernel (row-splitting ones for few
    tokens, with 16 or 8 weight rows a workgroup, the tiled ones for many; each forced here); it has to leave the queries and the
    pages as the product followed by the rotation kernel does, and must not touch any slot but
    the tokens' own (a token without a slot writes nothing)."""
    ops = ops_for(torch.bfloat16)
    bs, pages = 8, max(9, tokens // 8 + 2)
    width = (heads + 2 * kv_heads) * head_dim
    x = _rand((tokens, hidden), torch.bfloat16, 71).cuda()
    w = _rand((width, hidden), torch.bfloat16, 72, 0.2).cuda()
    b = _rand((width,), torch.float32, 73).cuda()
    rotation = None
    if rotate:
        pos = torch.tensor(([3, 0, 911, 17, 40000] + list(range(5, tokens)))[:tokens], dtype=torch.int32).cuda()
        inv = (1.0 / (1e6 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))).cuda()
        cos, sin = ops.rope_table(pos, inv)
        rotation = (cos, sin, head_dim)
    g = torch.Generator().manual_seed(74)
    slots = torch.randperm(pages * bs, generator=g)[:tokens].to(torch.int32)
    if tokens > 2:
        slots[2] = -1
    slots = slots.cuda()
    out = {}
    for fused in (False, True):
        kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=torch.bfloat16).cuda()
        vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=torch.bfloat16).cuda()
        q = ops.qkv_rope_write(x, w, b, rotation, slots, kp, vp, num_heads=heads, num_kv_heads=kv_heads,
                               head_dim=head_dim, block_size=bs, write=write, fused=fused,
                               mfma_kernel=kernel if fused else 0)
        out[fused] = (q[:, : heads * head_dim].float().cpu(), kp.float().cpu(), vp.float().cpu())
    # each way against the float64 value of the operation, within one ulp per operand of the rotation
    reference = qkv_reference(x, w, b, rotation[0] if rotate else None, rotation[1] if rotate else None, heads, kv_heads, head_dim)
    for fused in (False, True):
        check_qkv("fused" if fused else "three kernels", *out[fused], slots, bs, reference, heads, kv_heads, head_dim, write=write)
    for name, a, c in zip(("queries", "key pages", "value pages"), out[False], out[True]):
        assert torch.equal(torch.isnan(a), torch.isnan(c)), f"{name}: other slots written"
        if tokens <= 16 and (kernel == 16 or (kernel == 0 and tokens > 8)):
            # both ways sum the product in the same order (up to 8 tokens the shape may choose the
            # kernel that sums two halves of k); the rotation's two products may be
            # contracted differently: a last-place difference at most
            tol = dict(atol=0, rtol=2 ** -7)
        else:
            # the unfused product comes from another kernel with another order of summation: sums may
            # round to neighbouring bfloat16 values, and the rotation subtracts
            tol = _tol(torch.bfloat16)
        torch.testing.assert_close(torch.nan_to_num(c), torch.nan_to_num(a), msg=lambda m: f"{name}: {m}", **tol)
    assert torch.isnan(out[True][1]).all() == (not write)


@pytest.mark.parametrize("heads,kv_heads,head_dim,hidden,tokens,rotate,write", [
    (14, 2, 64, 896, 64, True, True), (14, 2, 64, 896, 33, True, True), (3, 1, 16, 520, 1, True, True),
    (5, 1, 128, 1208, 8, True, True), (4, 4, 80, 640, 17, False, True), (6, 3, 48, 2056, 5, True, False),
    (28, 4, 128, 3584, 8, True, True), (28, 4, 128, 3584, 100, True, True), (6, 2, 64, 1032, 128, True, True),
])
def test_sliced_qkv_product_equals_the_three_kernels(ops_for, heads, kv_heads, head_dim, hidden, tokens, rotate, write):
    """The third way of the query/key/value product (cut along k through the tiled kernel, then one
    kernel that adds the slices, rotates and stores) against the product followed by the rotation
    kernel: same queries, same pages, no other slot touched; and the way is chosen by itself for
    a wide product."""
    ops = ops_for(torch.bfloat16)
    bs, pages = 8, max(9, tokens // 8 + 2)
    width = (heads + 2 * kv_heads) * head_dim
    x = _rand((tokens, hidden), torch.bfloat16, 171).cuda()
    w = _rand((width, hidden), torch.bfloat16, 172, 0.2).cuda()
    b = _rand((width,), torch.float32, 173).cuda()
    rotation = None
    if rotate:
        pos = torch.tensor(([3, 0, 911, 17, 40000] + list(range(5, tokens)))[:tokens], dtype=torch.int32).cuda()
        inv = (1.0 / (1e6 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))).cuda()
        cos, sin = ops.rope_table(pos, inv)
        rotation = (cos, sin, head_dim)
    g = torch.Generator().manual_seed(174)
    slots = torch.randperm(pages * bs, generator=g)[:tokens].to(torch.int32)
    if tokens > 2:
        slots[2] = -1
    slots = slots.cuda()
    out = {}
    for way in ("unfused", "sliced", "auto"):
        kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=torch.bfloat16).cuda()
        vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=torch.bfloat16).cuda()
        kw = dict(fused=False, sliced=False) if way == "unfused" else (dict(sliced=True) if way == "sliced" else {})
        q = ops.qkv_rope_write(x, w, b, rotation, slots, kp, vp, num_heads=heads, num_kv_heads=kv_heads,
                               head_dim=head_dim, block_size=bs, write=write, **kw)
        out[way] = (q[:, : heads * head_dim].float().cpu(), kp.float().cpu(), vp.float().cpu())
    reference = qkv_reference(x, w, b, rotation[0] if rotate else None, rotation[1] if rotate else None, heads, kv_heads, head_dim)
    for way in out:
        check_qkv(way, *out[way], slots, bs, reference, heads, kv_heads, head_dim, write=write)
    for name, a, c in zip(("queries", "key pages", "value pages"), out["unfused"], out["sliced"]):
        assert torch.equal(torch.isnan(a), torch.isnan(c)), f"{name}: other slots written"
        torch.testing.assert_close(torch.nan_to_num(c), torch.nan_to_num(a), msg=lambda m: f"{name}: {m}", **_tol(torch.bfloat16))
    assert torch.isnan(out["sliced"][1]).all() == (not write)
    if width * hidden * 2 >= 24 << 20 and tokens >= 4:
        for a, c in zip(out["sliced"], out["auto"]):
            assert torch.equal(torch.nan_to_num(a), torch.nan_to_num(c)), "the sliced way is chosen by itself here"


def _drawn_qkv_case(case):
    """The shape, positions and way that a seeded draw gives for `case`: head size, heads, width,
    tokens, rotation, cache write, way (chosen by shape, fused, sliced), page size, positions."""
    import random

    rng = random.Random(9000 + case)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256])
    kv_heads = rng.choice([1, 2, 3, 4, 8])
    heads = kv_heads * rng.choice([1, 2, 4, 7])
    hidden = 8 * rng.choice([rng.randint(2, 60), rng.randint(60, 300), rng.randint(300, 700)])
    tokens = rng.choice([1, 2, 3, rng.randint(4, 8), rng.randint(9, 16), rng.randint(17, 64), rng.randint(65, 400), rng.randint(400, 2100)])
    if (heads + 2 * kv_heads) * head_dim * hidden > 6e7:
        hidden = 8 * rng.randint(8, 100)
    rotate, write = rng.random() < 0.85, rng.random() < 0.85
    way = rng.choice(["auto", "fused", "sliced"])
    bs = rng.choice([8, 16, 32])
    positions = [rng.randint(0, 100000) for _ in range(tokens)] if rotate else None
    return head_dim, kv_heads, heads, hidden, tokens, rotate, write, way, bs, positions


@pytest.mark.parametrize("case", [23, 127, 182, 369, 5, 77])
def test_qkv_ways_where_two_roundings_meet_a_subtraction(ops_for, case):
    """Four drawn shapes (23, 127, 182, 369, of some 500) in which the fused or sliced way and the
    three kernels differ by more than a relative bound on the RESULT allows, in one or two elements
    each (|difference| 0.016 to 0.0625): the product of such an element lies at the middle between
    two bfloat16 values, the two ways sum it in different orders and round it to different
    neighbours, and the rotation then subtracts two products of nearly equal size, so one ulp of an
    operand is many ulps of the result.  Both ways are within one ulp per operand of the float64
    value, which is all that can be asked; two more draws stand for the ordinary case."""
    head_dim, kv_heads, heads, hidden, tokens, rotate, write, way, bs, positions = _drawn_qkv_case(case)
    ops = ops_for(torch.bfloat16)
    pages = max(9, tokens // bs + 3)
    width = (heads + 2 * kv_heads) * head_dim
    x = _rand((tokens, hidden), torch.bfloat16, 71 + case).cuda()
    w = _rand((width, hidden), torch.bfloat16, 72 + case, 0.2).cuda()
    b = _rand((width,), torch.float32, 73 + case).cuda()
    rotation = cos = sin = None
    if rotate:
        pos = torch.tensor(positions, dtype=torch.int32).cuda()
        inv = (1.0 / (1e6 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))).cuda()
        cos, sin = ops.rope_table(pos, inv)
        rotation = (cos, sin, head_dim)
    g = torch.Generator().manual_seed(74 + case)
    slots = torch.randperm(pages * bs, generator=g)[:tokens].to(torch.int32)
    if tokens > 2:
        slots[2] = -1
    slots = slots.cuda()
    reference = qkv_reference(x, w, b, cos, sin, heads, kv_heads, head_dim)
    ways = {"three kernels": dict(fused=False)}
    ways[way] = {} if way == "auto" else (dict(fused=True) if way == "fused" else dict(sliced=True))
    if way == "sliced" and (tokens > 64 or hidden < 512 or not rotate):
        ways[way] = {}
    for name, kw in ways.items():
        kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=torch.bfloat16).cuda()
        vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=torch.bfloat16).cuda()
        q = ops.qkv_rope_write(x, w, b, rotation, slots, kp, vp, num_heads=heads, num_kv_heads=kv_heads,
                               head_dim=head_dim, block_size=bs, write=write, **kw)
        check_qkv(name, q.float().cpu(), kp.float().cpu(), vp.float().cpu(), slots, bs, reference, heads, kv_heads,
                  head_dim, write=write)


# ---- attention ----------------------------------------------------------------------------------------
def _paged_case(entries, heads, kv_heads, head_dim, bs, dtype, seed, extra_pages=3, spike=False):
    """entries: list of (context_len, q_len).  Returns device inputs and the float64 expectation."""
    g = torch.Generator().manual_seed(seed)
    need = [-(-c // bs) for c, _ in entries]
    pages = sum(need) + extra_pages
    perm = torch.randperm(pages, generator=g).tolist()
    width = max(need)
    table = torch.full((len(entries), width), -1, dtype=torch.int32)
    kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=dtype)
    vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=dtype)  # transposed inside a page
    dense = []
    for r, (ctx_len, _) in enumerate(entries):
        ids = [perm.pop() for _ in range(need[r])]
        table[r, : need[r]] = torch.tensor(ids, dtype=torch.int32)
        k = torch.randn(ctx_len, kv_heads, head_dim, generator=g).to(dtype)
        v = torch.randn(ctx_len, kv_heads, head_dim, generator=g).to(dtype)
        if spike and ctx_len > 3:
            k[1] *= 6.0  # a far key that must dominate when the query points at it
        for p in range(ctx_len):
            kp[ids[p // bs], :, p % bs] = k[p]
            vp[ids[p // bs], :, :, p % bs] = v[p]
        dense.append((k.double(), v.double()))
    token_entry, positions = [], []
    for r, (ctx_len, q_len) in enumerate(entries):
        for i in range(q_len):
            token_entry.append(r)
            positions.append(ctx_len - q_len + i)
    tokens = len(positions)
    q = torch.randn(tokens, heads * head_dim + 24, generator=g).to(dtype)  # wider rows: a strided q
    if spike:
        for t, r in enumerate(token_entry):
            if entries[r][0] > 3:
                k1 = dense[r][0][1]  # [kv_heads, d]
                rep = k1.repeat_interleave(heads // kv_heads, dim=0).reshape(-1)
                q[t, : heads * head_dim] = (rep * 0.5).to(dtype)
    ctx = _plan(entries, token_entry, positions)
    return q, kp, vp, table, ctx, dense, token_entry, positions


def _plan(entries, token_entry, positions):
    """What the step function hands to the attention kernels about a batch."""
    from mini_llm_runtime_amd.kernels.ops import query_tiles

    q_lens = [ql for _, ql in entries]
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    import numpy as np

    from mini_llm_runtime_amd.kernels.plans import attention_plan
    from mini_llm_runtime_amd.parts.context import PlanInput

    q_starts = [c - ql for c, ql in entries]
    tiles = query_tiles(q_lens, q_starts)
    wide = query_tiles(q_lens, q_starts, tile=128)
    planned = attention_plan(PlanInput(np.asarray(q_lens, dtype=np.int32), np.asarray(q_starts, dtype=np.int32), max(c for c, _ in entries)))
    singles = [c for c, ql in entries if ql == 1]
    return SimpleNamespace(
        num_entries=len(entries),
        token_entry=torch.tensor(token_entry, dtype=torch.int32).cuda(),
        positions=torch.tensor(positions, dtype=torch.int32).cuda(),
        cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
        context_lens=torch.tensor([c for c, _ in entries], dtype=torch.int32).cuda(),
        max_context_len=max(c for c, _ in entries),
        max_q_len=max(q_lens),
        query_tiles=torch.from_numpy(tiles).cuda() if len(tiles) else None,
        num_query_tiles=len(tiles),
        wide_query_tiles=torch.from_numpy(wide).cuda() if len(wide) else None,
        num_wide_query_tiles=len(wide),
        long_prefix=planned.sizes["long_prefix"],
        num_decode_entries=len(singles),
        max_decode_context=max(singles, default=0),
    )


def _attention_reference(q, dense, token_entry, positions, heads, kv_heads, head_dim, scale, window):
    group = heads // kv_heads
    out = torch.zeros(len(positions), heads, head_dim, dtype=torch.float64)
    for t, (r, p) in enumerate(zip(token_entry, positions)):
        k, v = dense[r]
        first = 0 if not window else max(0, p - window + 1)
        kk = k[first : p + 1].repeat_interleave(group, dim=1)  # [n, H, d]
        vv = v[first : p + 1].repeat_interleave(group, dim=1)
        qq = q[t, : heads * head_dim].double().view(heads, head_dim)
        s = torch.einsum("hd,nhd->hn", qq, kk) * scale
        out[t] = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), vv)
    return out.reshape(len(positions), heads * head_dim)


ATTN_SHAPES = [(14, 2, 64), (4, 1, 32), (3, 3, 16), (8, 2, 128), (6, 2, 48), (5, 1, 80)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim", ATTN_SHAPES)
@pytest.mark.parametrize("bs", [8, 16])
def test_paged_attention_mixed_batch(ops_for, dtype, heads, kv_heads, head_dim, bs):
    ops = ops_for(dtype)
    # (context, new tokens): decode tokens, whole prompts, portions behind a cached prefix, page edges
    entries = [(1, 1), (bs, 1), (bs + 1, 1), (37, 37), (70, 5), (4 * bs + 1, 2), (130, 1), (2 * bs, bs)]
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, bs, dtype, 21)
    scale = head_dim**-0.5
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs, scale=scale, window=None,
    ).cpu()
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, None)
    assert torch.isfinite(got).all(), "a NaN page slot was read"
    torch.testing.assert_close(got.double(), ref, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 7, 16, 50])
def test_paged_attention_window(ops_for, dtype, window):
    ops = ops_for(dtype)
    heads, kv_heads, head_dim, bs = 4, 2, 32, 8
    entries = [(1, 1), (16, 16), (60, 3), (75, 1)]
    _check_window(ops, dtype, window, heads, kv_heads, head_dim, bs, entries)


@pytest.mark.parametrize("window", [1, 50, 128, 200])
@pytest.mark.parametrize("heads,kv_heads,head_dim,bs", [(4, 2, 32, 8), (6, 2, 128, 16), (7, 1, 64, 16)])
def test_wide_prefill_attention_window(window, heads, kv_heads, head_dim, bs):
    """Tiles of 128 queries under a window: whole prompts longer than two tiles, a portion behind a
    cached prefix whose early pages the window has passed, and decoded tokens beside them."""
    entries = [(1, 1), (300, 300), (260, 129), (75, 1), (131, 131)]
    _check_window(_wide_ops(), torch.bfloat16, window, heads, kv_heads, head_dim, bs, entries)


def _wide_ops():
    from mini_llm_runtime_amd.kernels.ops import HipOps
    from mini_llm_runtime_amd.kernels.tuning import KernelTuning

    return HipOps(torch.bfloat16, "cuda", tuning=KernelTuning(wide_attention_groups=1))


def _check_window(ops, dtype, window, heads, kv_heads, head_dim, bs, entries):
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, bs, dtype, 22)
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs, scale=0.2, window=window,
    ).cpu()
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, 0.2, window)
    torch.testing.assert_close(got.double(), ref, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_far_key_among_hundreds(ops_for, dtype):
    """Queries aligned with key 1 of a long context: that key's value must dominate."""
    ops = ops_for(dtype)
    heads, kv_heads, head_dim, bs = 4, 2, 64, 16
    entries = [(700, 1), (515, 3), (2049, 1)]
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, bs, dtype, 23, spike=True)
    scale = head_dim**-0.5
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs, scale=scale, window=None,
    ).cpu()
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, None)
    torch.testing.assert_close(got.double(), ref, **_tol(dtype))
    v1 = dense[0][1][1].repeat_interleave(heads // kv_heads, dim=0).reshape(-1)
    assert (got[0].double() - v1).abs().max() < 0.2, "the far key did not dominate"


def test_paged_attention_merge_needs_global_weights(ops_for):
    """Two keys with scores +-large and values 7 and -3: the answer is 7, not the mean 2
    (reference tests/test_split_kv_attention.py:62-73)."""
    ops = ops_for(torch.float32)
    bs = 4
    kp = torch.zeros(2, 1, bs, 16)
    vp = torch.zeros(2, 1, 16, bs)
    kp[0, 0, 0, 0] = 40.0
    kp[1, 0, 0, 0] = -40.0
    vp[0, 0, :, 0] = 7.0
    vp[1, 0, :, 0] = -3.0
    # context of 5 tokens: positions 0..3 in page 0 (1..3 neutral), position 4 in page 1
    q = torch.zeros(1, 16)
    q[0, 0] = 1.0
    ctx = _plan([(5, 1)], [0], [4])
    table = torch.tensor([[0, 1]], dtype=torch.int32)
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=1, num_kv_heads=1, head_dim=16, block_size=bs, scale=1.0, window=None,
    ).cpu()
    torch.testing.assert_close(got, torch.full((1, 16), 7.0), atol=1e-5, rtol=0)


def test_paged_attention_bad_page_poisons(ops_for):
    """A used table entry of -1 must never be read as a page (reference tests/test_paged_attention.py:158-171)."""
    ops = ops_for(torch.float32)
    entries = [(20, 1)]
    q, kp, vp, table, ctx, *_ = _paged_case(entries, 2, 1, 16, 8, torch.float32, 24)
    table[0, 1] = -1
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=2, num_kv_heads=1, head_dim=16, block_size=8, scale=0.25, window=None,
    ).cpu()
    assert torch.isnan(got).all()


def test_attention_matches_library_special_case(ops_for):
    """No rotation, whole prompt, MHA: equals torch's scaled_dot_product_attention(is_causal=True)."""
    ops = ops_for(torch.float32)
    heads, head_dim, bs, n = 3, 32, 8, 29
    q, kp, vp, table, ctx, dense, te, pos = _paged_case([(n, n)], heads, heads, head_dim, bs, torch.float32, 25)
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=heads, head_dim=head_dim, block_size=bs, scale=head_dim**-0.5, window=None,
    ).cpu()
    k, v = dense[0]
    qq = q[:, : heads * head_dim].double().view(n, heads, head_dim).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(qq, k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(got.double(), ref.transpose(0, 1).reshape(n, -1), atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("heads,kv_heads,head_dim", ATTN_SHAPES + [(40, 2, 64), (2, 2, 256)])
@pytest.mark.parametrize("partition", [64, 256, 4096])
def test_decode_attention_partitions(ops_for, heads, kv_heads, head_dim, partition):
    """The split-KV decode kernel with one, a few and many partitions, at context lengths around
    page and tile edges (reference tests/test_split_kv_attention.py:37-59: 1, 15, 16, 17, 65, 2048, 2049),
    against float64 and against the plain 32-bit kernel."""
    ops = ops_for(torch.bfloat16)
    old = ops.decode_partition
    ops.decode_partition = partition
    try:
        entries = [(n, 1) for n in (1, 15, 16, 17, 65, 300, 2048, 2049)]
        q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, 16, torch.bfloat16, 26)
        scale = head_dim**-0.5
        args = (q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx)
        kw = dict(num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=16, scale=scale, window=None)
        got = _attend(ops, *args, **kw).cpu()
        fma = _attend(ops, *args, kernel="fma", **kw).cpu()
    finally:
        ops.decode_partition = old
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, None)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), ref, **_tol(torch.bfloat16))
    torch.testing.assert_close(got.double(), fma.double(), **_tol(torch.bfloat16))


@pytest.mark.parametrize("heads,kv_heads,head_dim,bs,long", [
    (14, 2, 64, 16, 2048), (8, 2, 128, 16, 1100), (3, 1, 96, 8, 700), (2, 1, 256, 32, 600), (5, 5, 16, 64, 900),
])
@pytest.mark.parametrize("wide", [False, True])
def test_prefill_attention_long_prompt_and_portion(ops_for, heads, kv_heads, head_dim, bs, long, wide):
    """The tiled prefill kernel on a long prompt (many key tiles, both key groups, tiles handed out
    heavy first) and on a 300-token portion behind cached tokens, at several head and page sizes;
    with tiles of 64 queries and (forced: few tiles would not choose it) of 128."""
    ops = ops_for(torch.bfloat16) if not wide else _wide_ops()
    entries = [(long, long), (long - 250, 300), (77, 77)]
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, bs, torch.bfloat16, 27, spike=True)
    scale = head_dim**-0.5
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs, scale=scale, window=None,
    ).cpu()
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, None)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), ref, **_tol(torch.bfloat16))


@pytest.mark.parametrize("heads,kv_heads,head_dim,bs,wide", [(4, 2, 64, 16, False), (6, 2, 128, 16, False), (3, 1, 32, 8, True), (2, 2, 256, 32, False)])
def test_prompt_portions_behind_long_contexts_in_key_runs(ops_for, heads, kv_heads, head_dim, bs, wide):
    """Few query tiles behind thousands of cached tokens: the keys of every tile are cut into runs,
    a workgroup each, and merged; portions of 2 to 200 tokens, a whole short prompt beside them (its
    tiles have runs without keys), and a far key that carries the result."""
    ops = ops_for(torch.bfloat16) if not wide else _wide_ops()
    assert ops.tuning.key_run_groups > 9 * heads  # more than the tiles of this case: they are cut
    entries = [(9000, 200), (12000, 2), (70, 70), (8200, 65)]
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, bs, torch.bfloat16, 43, spike=True)
    assert ctx.long_prefix == 2
    scale = head_dim**-0.5
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs, scale=scale, window=None,
    ).cpu()
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, None)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), ref, **_tol(torch.bfloat16))


def test_attention_at_a_long_context(ops_for):
    """A decoded token and a 64-token portion behind some 20,000 cached positions: many partitions
    and key tiles, table rows of over a thousand pages, and a single far key (position 1) that
    carries the result, which an index or partition mistake would lose among the thousands."""
    ops = ops_for(torch.bfloat16)
    heads, kv_heads, head_dim, bs = 4, 2, 64, 16
    entries = [(20000, 1), (19000, 64), (33, 33)]
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, bs, torch.bfloat16, 41, spike=True)
    scale = head_dim**-0.5
    got = _attend(
        ops,
        q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx,
        num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=bs, scale=scale, window=None,
    ).cpu()
    ref = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, None)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), ref, **_tol(torch.bfloat16))
    # the far key really decides: the output is close to its value row
    v1 = dense[0][1][1]  # values at position 1 of the first entry, [kv_heads, d]
    want = v1.repeat_interleave(heads // kv_heads, dim=0).reshape(-1)
    assert torch.allclose(got[0].double(), want, atol=0.1), "the far key did not dominate"


# ---- sampling ---------------------------------------------------------------------------------------------
def test_sample_greedy_first_maximum(ops_for):
    ops = ops_for(torch.float32)
    logits = _rand((6, 1000), torch.float32, 30)
    logits[0, 17] = logits[0, 900] = 50.0  # tie: the first wins
    logits[1, 999] = 60.0
    logits[2, 0] = 60.0
    got = ops.sample(logits.cuda()).cpu()
    assert got.dtype == torch.int32
    assert got.tolist() == torch.argmax(logits, dim=-1).tolist()
    assert got[0] == 17
    big = _rand((3, 151936), torch.float32, 31)
    assert ops.sample(big.cuda()).cpu().tolist() == torch.argmax(big, -1).tolist()


def test_sample_temperature_inverse_cdf(ops_for):
    ops = ops_for(torch.float32)
    rows, vocab = 64, 517
    logits = _rand((rows, vocab), torch.float32, 32, 3.0)
    g = torch.Generator().manual_seed(33)
    u = torch.rand(rows, generator=g)
    u[0], u[1] = 0.0, 0.99999994
    temp = torch.full((rows,), 0.8)
    temp[2] = 0.0  # greedy row inside a sampled batch
    got = ops.sample(logits.cuda(), temp.cuda(), u.cuda()).cpu().long()
    assert got[2] == torch.argmax(logits[2])
    for i in range(rows):
        if temp[i] == 0:
            continue
        cdf = torch.cumsum(plain.temperature_probabilities(logits[i], float(temp[i])), 0)
        lo = 0.0 if got[i] == 0 else float(cdf[got[i] - 1])
        hi = float(cdf[got[i]])
        assert lo - 1e-5 <= float(u[i]) <= hi + 1e-5, (i, lo, float(u[i]), hi)
    # the same uniform number gives the same token whatever else is in the batch
    alone = ops.sample(logits[5:6].cuda(), temp[5:6].cuda(), u[5:6].cuda()).cpu()
    assert int(alone[0]) == int(got[5])
