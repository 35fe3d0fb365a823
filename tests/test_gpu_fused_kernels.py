"""The products of a few tokens that make their own activations (a norm, or the merge of the
decode attention's partitions, as the prologue of the matrix product), each alone against
float64 and against the kernels they replace, at sizes other than the engine's."""

from __future__ import annotations

import pytest
import torch

import plain_qwen2 as plain
from mini_llm_runtime_amd.kernels.pending import PendingMerge, PendingNorm
from mini_llm_runtime_amd.kernels.tuning import KernelTuning
from qkv_reference import check_qkv, qkv_reference
from test_gpu_kernels import _attend, _attention_reference, _paged_case, _rand, _tol

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(gpu_device):
    from mini_llm_runtime_amd.kernels.ops import HipOps

    return HipOps(torch.bfloat16, gpu_device)


def _delta(kind, m, k, seed):
    if kind == "none":
        return None
    if kind == "bf16":
        return _rand((m, k), torch.bfloat16, seed, 0.5)
    return _rand((int(kind), m, k), torch.float32, seed, 0.3)  # that many partial sums


@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (2, 130, 96), (4, 9728, 896), (3, 1152, 896), (4, 1000, 1000), (3, 320, 2048), (1, 20, 1536)])
@pytest.mark.parametrize("delta", ["none", "bf16", "1", "3", "8", "11"])
@pytest.mark.parametrize("weight_f32", [False, True])
def test_norm_as_the_prologue_of_a_product(ops, m, n, k, delta, weight_f32):
    """y = RMSNorm(x + delta) W^T + b in one kernel: the product, the updated stream and their
    agreement with the norm kernel followed by the product kernel."""
    x = _rand((m, k), torch.float32, 81, 2.0)
    d = _delta(delta, m, k, 82)
    nw = (1 + _rand((k,), torch.float32, 83, 0.1)).to(torch.float32 if weight_f32 else torch.bfloat16)
    w = _rand((n, k), torch.bfloat16, 84, 0.05)
    b = _rand((n,), torch.float32, 85)
    eps = 1e-5
    summed = x.double() + (0 if d is None else d.double().sum(0) if d.dim() == 3 else d.double())
    normed = plain.rms_norm(summed, nw.double(), eps)
    ref = normed.to(torch.bfloat16).double() @ w.double().t() + b.double()
    xd = x.cuda()
    before = xd.clone()
    pending = ops.defer_norm(xd, nw.cuda(), eps, None if d is None else d.cuda())
    assert isinstance(pending, PendingNorm)
    got = ops.linear(pending, w.cuda(), b.cuda())
    assert torch.equal(xd, before), "the stream that other workgroups read must stay as it was"
    assert got.shape == (m, n) and got.dtype == torch.bfloat16
    # the normed activations are rounded to bfloat16 before the product, as between two kernels;
    # a value that sits on a rounding edge may fall to the other side
    torch.testing.assert_close(got.cpu().double(), ref, atol=3e-2, rtol=2e-2)
    if d is None:
        assert pending.residual is xd
    else:
        assert pending.residual is not xd
        torch.testing.assert_close(pending.residual.cpu().double(), summed, atol=1e-5, rtol=1e-6)
    # against the two kernels it replaces
    xs = x.cuda()
    h = ops.rmsnorm(xs, nw.cuda(), eps, delta=None if d is None else d.cuda())
    two = ops.linear(h, w.cuda(), b.cuda())
    torch.testing.assert_close(got.float(), two.float(), atol=3e-2, rtol=2e-2)
    assert float((got.float() - two.float()).abs().mean()) < 2e-3
    if d is not None:
        torch.testing.assert_close(pending.residual, xs, atol=1e-6, rtol=1e-6)  # same sums in the same order
    again = ops.linear(ops.defer_norm(x.cuda(), nw.cuda(), eps, None if d is None else d.cuda()), w.cuda(), b.cuda())
    assert torch.equal(again, got)


@pytest.mark.parametrize("m,inter,k", [(1, 352, 96), (4, 4864, 896), (2, 130, 64), (3, 2432, 1536)])
def test_norm_prologue_with_swiglu_epilogue(ops, m, inter, k):
    x = _rand((m, k), torch.float32, 86, 1.5)
    d = _rand((2, m, k), torch.float32, 87, 0.3)
    nw = (1 + _rand((k,), torch.float32, 88, 0.1)).to(torch.bfloat16)
    gate = _rand((inter, k), torch.bfloat16, 89, 0.08)
    up = _rand((inter, k), torch.bfloat16, 90, 0.08)
    woven = torch.stack([gate.view(-1, 2, k), up.view(-1, 2, k)], dim=1).reshape(2 * inter, k).contiguous()
    h = plain.rms_norm(x.double() + d.double().sum(0), nw.double(), 1e-6).to(torch.bfloat16).double()
    g = h @ gate.double().t()
    ref = g * torch.sigmoid(g) * (h @ up.double().t())
    pending = ops.defer_norm(x.cuda(), nw.cuda(), 1e-6, d.cuda())
    got = ops.linear(pending, woven.cuda(), None, swiglu=True)
    assert got.shape == (m, inter)
    torch.testing.assert_close(got.cpu().double(), ref, atol=2e-2, rtol=3e-2)
    assert pending.residual is not None


@pytest.mark.parametrize("heads,kv_heads,head_dim,hidden,tokens", [(4, 2, 16, 64, 3), (14, 2, 64, 896, 4), (3, 1, 32, 96, 2), (6, 2, 48, 72, 1), (16, 2, 128, 2048, 4)])
@pytest.mark.parametrize("rotate", [True, False])
def test_norm_prologue_of_the_query_key_value_product(ops, heads, kv_heads, head_dim, hidden, tokens, rotate):
    """Norm, product, bias, rotation and cache write in one kernel leave the queries and the
    pages as the norm kernel followed by the fused product does; no other slot is touched."""
    bs, pages = 8, 9
    width = (heads + 2 * kv_heads) * head_dim
    x = _rand((tokens, hidden), torch.float32, 91, 2.0)
    d = _rand((4, tokens, hidden), torch.float32, 92, 0.3)
    nw = (1 + _rand((hidden,), torch.float32, 93, 0.1)).to(torch.bfloat16).cuda()
    w = _rand((width, hidden), torch.bfloat16, 94, 0.2).cuda()
    b = _rand((width,), torch.float32, 95).cuda()
    rotation = None
    if rotate:
        pos = torch.tensor(([3, 0, 911, 17, 40000] + list(range(5, 16)))[:tokens], dtype=torch.int32).cuda()
        inv = (1.0 / (1e6 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))).cuda()
        cos, sin = ops.rope_table(pos, inv)
        rotation = (cos, sin, head_dim)
    g = torch.Generator().manual_seed(96)
    slots = torch.randperm(pages * bs, generator=g)[:tokens].to(torch.int32)
    if tokens > 2:
        slots[2] = -1
    slots = slots.cuda()
    out = {}
    for fused in (False, True):
        kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=torch.bfloat16).cuda()
        vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=torch.bfloat16).cuda()
        xs = x.cuda()
        if fused:
            h = ops.defer_norm(xs, nw, 1e-6, d.cuda())
            assert isinstance(h, PendingNorm)
        else:
            h = ops.rmsnorm(xs, nw, 1e-6, delta=d.cuda())
        q = ops.qkv_rope_write(h, w, b, rotation, slots, kp, vp, num_heads=heads, num_kv_heads=kv_heads,
                               head_dim=head_dim, block_size=bs)
        stream = h.residual if fused else xs
        out[fused] = (q.float().cpu(), kp.float().cpu(), vp.float().cpu(), stream.cpu())
        if not fused:
            normed = h
    # both ways against the float64 value of product, rotation and rounding, from the normed rows of
    # the norm kernel.  The kernel that norms for itself may land a normed value on the neighbouring
    # bfloat16 value now and then: one such value moves a product by 2^-8 of its largest term.
    slack = float((normed.double().abs().max(dim=1).values[:, None] * w.double().abs().max(dim=1).values[None, :]).max()) * 2.0**-8
    reference = qkv_reference(normed, w, b, rotation[0] if rotate else None, rotation[1] if rotate else None, heads,
                              kv_heads, head_dim, p_slack=slack)
    for fused in (False, True):
        check_qkv("norm inside" if fused else "norm kernel first", *out[fused][:3], slots, bs, reference, heads, kv_heads,
                  head_dim, max_neighbours=0.03 if not fused else 0.1)
    for name, a, c in zip(("queries", "key pages", "value pages"), out[False], out[True]):
        assert torch.equal(torch.isnan(a), torch.isnan(c)), f"{name}: other slots written"
        torch.testing.assert_close(torch.nan_to_num(c), torch.nan_to_num(a), msg=lambda m: f"{name}: {m}", **_tol(torch.bfloat16))
    torch.testing.assert_close(out[True][3], out[False][3], atol=1e-6, rtol=1e-6)


def test_norm_prologue_is_refused_where_it_does_not_pay(ops, gpu_device):
    from mini_llm_runtime_amd.kernels.ops import HipOps

    nw = torch.ones(4096, dtype=torch.bfloat16).cuda()
    assert ops.defer_norm(torch.zeros(8, 4096).cuda(), nw, 1e-6, None) is None  # too wide
    assert ops.defer_norm(torch.zeros(5, 896).cuda(), nw[:896], 1e-6, None) is None  # more tokens than wavefronts
    small = HipOps(torch.bfloat16, gpu_device, tuning=KernelTuning(fuse_bytes=100_000))
    assert small.defer_norm(torch.zeros(4, 896).cuda(), nw[:896], 1e-6, torch.zeros(8, 4, 896).cuda()) is None  # too much to re-read
    assert small.defer_norm(torch.zeros(4, 896).cuda(), nw[:896], 1e-6, torch.zeros(2, 4, 896).cuda()) is not None
    assert HipOps(torch.float32, gpu_device).defer_norm(torch.zeros(2, 64).cuda(), torch.ones(64).cuda(), 1e-6, None) is None
    off = HipOps(torch.bfloat16, gpu_device, tuning=KernelTuning(fuse_norm=False, fuse_merge=False))
    assert off.defer_norm(torch.zeros(2, 64).cuda(), nw[:64], 1e-6, None) is None
    # a pending norm that meets a product which cannot fuse it is run on its own, with the same result
    x = _rand((4, 64), torch.float32, 97).cuda()
    w = _rand((24, 64), torch.bfloat16, 98).cuda()
    pending = ops.defer_norm(x.clone(), nw[:64], 1e-6, None)
    plainly = ops.linear(ops.rmsnorm(x.clone(), nw[:64], 1e-6), w, None, kernel="fma")
    assert torch.equal(ops.linear(pending, w, None, kernel="fma"), plainly) and pending.residual is not None
    # a weight beyond the limit streams faster through the tiled kernel: the norm runs on its own
    heavy = HipOps(torch.bfloat16, gpu_device, tuning=KernelTuning(fuse_weight_bytes=1000))
    pending = heavy.defer_norm(x.clone(), nw[:64], 1e-6, None)
    assert pending is not None
    assert torch.equal(heavy.linear(pending, w, None), ops.linear(ops.rmsnorm(x.clone(), nw[:64], 1e-6), w, None))


@pytest.mark.parametrize("heads,kv_heads,head_dim", [(14, 2, 64), (4, 1, 32), (8, 2, 128), (6, 2, 48), (5, 1, 80), (3, 3, 16)])
@pytest.mark.parametrize("partition", [64, 256])
@pytest.mark.parametrize("window", [None, 300])
@pytest.mark.parametrize("lengths", [(1, 15, 64, 65, 300, 700, 1023, 1100), (1100, 65), (700,)])
def test_merge_as_the_prologue_of_the_output_product(ops, heads, kv_heads, head_dim, partition, window, lengths):
    """The decode attention leaves its partitions unmerged and the output product merges them
    while it loads its operand: against float64 and against attention, merge and product as
    three kernels; entries of very different lengths (some use one partition, some all)."""
    from mini_llm_runtime_amd.kernels.ops import HipOps

    tuned = HipOps(torch.bfloat16, ops.device, tuning=KernelTuning(decode_partition=partition))
    entries = [(n, 1) for n in lengths]
    q, kp, vp, table, ctx, dense, te, pos = _paged_case(entries, heads, kv_heads, head_dim, 16, torch.bfloat16, 99)
    scale = head_dim**-0.5
    hidden = 136
    k = heads * head_dim
    wo = _rand((hidden, k), torch.bfloat16, 100, 0.1).cuda()
    bo = _rand((hidden,), torch.float32, 101).cuda()
    args = (q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx)
    kw = dict(num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_size=16, scale=scale, window=window)
    pending = _attend(tuned, *args, defer_merge=True, **kw)
    assert isinstance(pending, PendingMerge) and pending.splits > 1
    attended = _attend(tuned, *args, **kw)
    ref_att = _attention_reference(q, dense, te, pos, heads, kv_heads, head_dim, scale, window)
    torch.testing.assert_close(attended.cpu().double(), ref_att, **_tol(torch.bfloat16))
    assert torch.equal(tuned.settle(pending), attended), "the merge on its own gives what the attention call gives"
    calls = []
    original = tuned._call
    tuned._call = lambda name, *a, **kw: (calls.append(name), original(name, *a, **kw))[1]
    for sums in (False, True):
        fused = tuned.linear(pending, wo, bo, partial_sums=sums)
        three = tuned.linear(attended, wo, bo, partial_sums=sums)
        assert fused.shape == three.shape
        a = fused.float().sum(0) if fused.dim() == 3 else fused.float()
        c = three.float().sum(0) if three.dim() == 3 else three.float()
        ref = ref_att.to(torch.bfloat16).double() @ wo.cpu().double().t() + bo.cpu().double()
        torch.testing.assert_close(a.cpu().double(), ref, atol=3e-2, rtol=2e-2)
        torch.testing.assert_close(a, c, atol=2e-2, rtol=2e-2)
    if len(lengths) * k // 8 <= 256:
        assert calls.count("mlr_gemm_merge_fused_bf16") == 2, "few tokens: the product merges in its own kernel"
    sliced = tuned.linear(pending, wo, bo, partial_sums=True, slices=3)
    assert sliced.shape == (3, len(lengths), hidden)
    torch.testing.assert_close(sliced.sum(0).cpu().double(), ref, atol=3e-2, rtol=2e-2)


def test_merge_prologue_keeps_the_poison_of_a_missing_page(ops):
    entries = [(500, 1), (400, 1)]
    q, kp, vp, table, ctx, *_ = _paged_case(entries, 4, 2, 32, 16, torch.bfloat16, 102)
    table[1, 3] = -1
    wo = _rand((40, 128), torch.bfloat16, 103, 0.1).cuda()
    pending = _attend(ops, q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx, num_heads=4, num_kv_heads=2,
                                  head_dim=32, block_size=16, scale=0.2, window=None, defer_merge=True)
    assert isinstance(pending, PendingMerge)
    out = ops.linear(pending, wo, None).float().cpu()
    assert torch.isfinite(out[0]).all() and torch.isnan(out[1]).all()


def test_mixed_batches_and_single_partitions_do_not_defer(ops):
    """Only a batch of single tokens whose keys are cut into partitions defers its merge."""
    kw = dict(num_heads=4, num_kv_heads=2, head_dim=32, block_size=16, scale=0.2, window=None, defer_merge=True)
    q, kp, vp, table, ctx, *_ = _paged_case([(40, 1), (30, 1)], 4, 2, 32, 16, torch.bfloat16, 104)
    assert isinstance(_attend(ops, q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx, **kw), torch.Tensor)
    q, kp, vp, table, ctx, *_ = _paged_case([(600, 1), (500, 20)], 4, 2, 32, 16, torch.bfloat16, 105)
    assert isinstance(_attend(ops, q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx, **kw), torch.Tensor)


# ---- the product that finishes the residual stream, and the products that pay the norm it owes --------------
def _wide_open(gpu_device):
    """The kernels at every token count they take, not only where the engine chooses them."""
    from mini_llm_runtime_amd.kernels.ops import HipOps

    return HipOps(torch.bfloat16, gpu_device, tuning=KernelTuning(
        finish_min_tokens=1, finish_max_tokens=64, finish_weight_bytes=1 << 30, finish_activation_bytes=1 << 30))


_STREAM_SHAPES = [
    (1, 64, 64), (3, 896, 896), (4, 132, 200), (5, 100, 72), (8, 896, 4864), (9, 896, 896), (12, 132, 200), (16, 260, 1032),
    (17, 256, 512), (24, 100, 264), (32, 896, 896), (33, 64, 128), (50, 520, 264), (64, 896, 1024),
    (8, 3584, 264), (20, 4104, 136),  # more parts a row than a consumer holds in registers: its slower way
]


@pytest.mark.parametrize("m,n,k", _STREAM_SHAPES)
@pytest.mark.parametrize("bias,weight_f32", [(None, False), ("f32", True), ("bf16", False)])
def test_product_that_finishes_the_stream(gpu_device, m, n, k, bias, weight_f32):
    """stream += a W^T + b in the product's own kernel (4, 8 or 16 features a workgroup, one to four
    blocks of tokens), the next norm's activations short of their factor per row, and every row's sum
    of squares in parts: each against float64; then the products that pay the factor (plain, SwiGLU)
    against float64 and against the norm kernel followed by the same product."""
    from mini_llm_runtime_amd.kernels.pending import PendingLinear, PendingScale

    ops = _wide_open(gpu_device)
    a = _rand((m, k), torch.bfloat16, 201, 0.7)
    w = _rand((n, k), torch.bfloat16, 202, 0.1)
    b = None if bias is None else _rand((n,), torch.float32 if bias == "f32" else torch.bfloat16, 203)
    x = _rand((m, n), torch.float32, 204, 1.5)
    nw = (1 + _rand((n,), torch.float32, 205, 0.1)).to(torch.float32 if weight_f32 else torch.bfloat16)
    eps = 1e-5
    new_stream = x.double() + a.double() @ w.double().t() + (0 if b is None else b.double())
    pending = ops.linear(a.cuda(), w.cuda(), None if b is None else b.cuda(), for_stream=True)
    assert isinstance(pending, PendingLinear)
    xd = x.cuda()
    owed = ops.defer_norm(xd, nw.cuda(), eps, pending)
    assert isinstance(owed, PendingScale) and owed.residual is xd
    torch.testing.assert_close(xd.cpu().double(), new_stream, atol=2e-4 * k**0.5, rtol=1e-5)
    # h: the stream as the kernel left it times the weight, rounded once
    expect_h = (nw.double() * xd.cpu().double()).float().to(torch.bfloat16)
    torch.testing.assert_close(owed.h.cpu().float(), expect_h.float(), atol=0, rtol=2**-7)
    assert float((owed.h.cpu() != expect_h).double().mean()) < 0.01
    assert owed.sumsq.shape == (m, ops.lib.mlr_gemm_residual_parts(m, n))
    torch.testing.assert_close(owed.sumsq.double().sum(1).cpu(), xd.cpu().double().pow(2).sum(1), atol=0, rtol=1e-5)
    # the settled form is the plain norm of the stream
    normed = plain.rms_norm(xd.cpu().double(), nw.double(), eps)
    # consumers: y = normed W2^T + b2, the factor applied to the sums
    n2 = 4 * (37 + m)
    w2 = _rand((n2, n), torch.bfloat16, 206, 0.1)
    b2 = _rand((n2,), torch.float32, 207)
    scale = torch.rsqrt(xd.cpu().double().pow(2).mean(1, keepdim=True) + eps)
    exact = (owed.h.cpu().double() * scale) @ w2.double().t()  # from the very activations the kernel read
    got = ops.linear(owed, w2.cuda(), b2.cuda())
    if n % 8 == 0:  # (else there is no matrix-core product: the norm is settled by its own kernel)
        torch.testing.assert_close(got.cpu().double(), exact + b2.double(), atol=2e-2, rtol=1.6e-2)
    torch.testing.assert_close(got.cpu().double(), normed @ w2.double().t() + b2.double(), atol=6e-2, rtol=3e-2)
    wide = ops.linear(owed, w2.cuda(), b2.cuda(), out_dtype=torch.float32)
    if n % 8 == 0:
        torch.testing.assert_close(wide.cpu().double(), exact + b2.double(), atol=1e-3 * n**0.5, rtol=1e-4)
    else:  # no matrix-core product at this width: the norm is settled by its own kernel, then the plain product
        torch.testing.assert_close(wide.cpu().double(), normed @ w2.double().t() + b2.double(), atol=6e-2, rtol=3e-2)
    two = ops.linear(ops.rmsnorm(xd.clone(), nw.cuda(), eps), w2.cuda(), b2.cuda())
    torch.testing.assert_close(got.float(), two.float(), atol=6e-2, rtol=3e-2)
    # the two ways round differently (weight * stream rounded, then scaled; or normed, then rounded): on
    # average they stay within an ulp of bfloat16 (2^-7 of a value) of each other
    assert float((got.float() - two.float()).abs().mean()) < 2.0**-7 * float(two.float().abs().mean())
    glu = ops.linear(owed, w2.cuda(), None, swiglu=True)
    quads = exact.view(m, -1, 4)
    gate, up = quads[..., :2], quads[..., 2:]
    torch.testing.assert_close(glu.cpu().double(), (gate * torch.sigmoid(gate) * up).reshape(m, -1), atol=2e-2, rtol=3e-2)
    # every matrix-core kernel that takes these tokens pays the factor the same way
    for kernel in (16, 14, 11, 23, 45, 46, 47, 48, 62, 65, 68):
        if (kernel == 14 and m > 32) or n % 8:
            continue
        forced = ops.linear(owed, w2.cuda(), b2.cuda(), out_dtype=torch.float32, mfma_kernel=kernel)
        torch.testing.assert_close(forced.cpu().double(), exact + b2.double(), atol=1e-3 * n**0.5, rtol=1e-4, msg=lambda s: f"kernel {kernel}: {s}")
    # and cut along k, every slice scaled, the bias in the first
    if n % 8 == 0 and n >= 128:
        sliced = ops.linear(owed, w2.cuda(), b2.cuda(), partial_sums=True, slices=2)
        torch.testing.assert_close(sliced.sum(0).cpu().double(), exact + b2.double(), atol=1e-3 * n**0.5, rtol=1e-4)
    # settled, it is the norm kernel's own result
    assert torch.equal(ops.settle(owed), ops.rmsnorm(xd.clone(), nw.cuda(), eps))


@pytest.mark.parametrize("heads,kv_heads,head_dim,hidden,tokens", [
    (4, 2, 16, 64, 3), (14, 2, 64, 896, 8), (14, 2, 64, 896, 5), (3, 1, 32, 96, 13), (6, 2, 48, 72, 30), (14, 2, 64, 896, 64),
    (4, 1, 32, 128, 100), (14, 2, 64, 896, 300),
])
@pytest.mark.parametrize("rotate", [True, False])
def test_query_key_value_product_pays_the_owed_norm(gpu_device, heads, kv_heads, head_dim, hidden, tokens, rotate):
    """Every way of the query/key/value product (the row-splitting kernels with 8 and 16 rows, the tiled
    one, product then rotation kernel, cut along k) on activations that still owe their factor per
    row, against the float64 value computed from the very activations and sums of squares it read."""
    from mini_llm_runtime_amd.kernels.pending import PendingScale

    ops = _wide_open(gpu_device)
    bs, pages = 8, max(9, tokens // 8 + 2)
    width = (heads + 2 * kv_heads) * head_dim
    h = _rand((tokens, hidden), torch.bfloat16, 211, 2.0).cuda()
    parts = 7 if tokens % 2 else 70
    sumsq = (torch.rand(tokens, parts, generator=torch.Generator().manual_seed(212)) * hidden * 3 / parts).cuda()
    eps = 1e-6
    w = _rand((width, hidden), torch.bfloat16, 213, 0.2).cuda()
    b = _rand((width,), torch.float32, 214).cuda()
    rotation = None
    if rotate:
        pos = torch.tensor(([3, 0, 911, 17, 40000] + list(range(5, tokens)))[:tokens], dtype=torch.int32).cuda()
        inv = (1.0 / (1e6 ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))).cuda()
        cos, sin = ops.rope_table(pos, inv)
        rotation = (cos, sin, head_dim)
    g = torch.Generator().manual_seed(215)
    slots = torch.randperm(pages * bs, generator=g)[:tokens].to(torch.int32)
    if tokens > 2:
        slots[2] = -1
    slots = slots.cuda()
    factor = torch.rsqrt(sumsq.double().sum(1, keepdim=True).cpu() / hidden + eps)
    # the kernel multiplies float32 sums by a float32 factor: one more rounding of 2^-24, inside e_sum's allowance
    reference = qkv_reference(h.cpu().double() * factor, w, b, rotation[0] if rotate else None, rotation[1] if rotate else None,
                              heads, kv_heads, head_dim)
    ways = {"chosen": {}, "three kernels": dict(fused=False)}
    if tokens <= 8:
        ways["8 rows"] = dict(fused=True, mfma_kernel=8)
    if tokens <= 64:
        ways["16 rows"] = dict(fused=True, mfma_kernel=16)
    ways["tiled"] = dict(fused=True, mfma_kernel=11)
    if tokens <= 128 and hidden >= 512 and rotate:
        ways["cut along k"] = dict(sliced=True)
    for name, kw in ways.items():
        owed = PendingScale(h, sumsq, torch.ones(hidden, dtype=torch.bfloat16).cuda(), eps, torch.zeros(tokens, hidden).cuda())
        kp = torch.full((pages, kv_heads, bs, head_dim), float("nan"), dtype=torch.bfloat16).cuda()
        vp = torch.full((pages, kv_heads, head_dim, bs), float("nan"), dtype=torch.bfloat16).cuda()
        q = ops.qkv_rope_write(owed, w, b, rotation, slots, kp, vp, num_heads=heads, num_kv_heads=kv_heads,
                               head_dim=head_dim, block_size=bs, **kw)
        check_qkv(name, q.float().cpu(), kp.float().cpu(), vp.float().cpu(), slots, bs, reference, heads, kv_heads, head_dim)


def test_stream_finishing_product_is_used_where_it_pays(gpu_device):
    """By default only small matrices at 5 to 8 tokens go that way; everything else keeps the product
    cut along k and the norm kernel.  A product that is not taken that way, or that meets a norm which
    cannot run it, comes out as before."""
    from mini_llm_runtime_amd.kernels.ops import HipOps
    from mini_llm_runtime_amd.kernels.pending import PendingLinear

    ops = HipOps(torch.bfloat16, gpu_device)
    w_small = _rand((896, 896), torch.bfloat16, 221, 0.1).cuda()
    w_large = _rand((896, 4864), torch.bfloat16, 222, 0.1).cuda()
    for m, expect in ((1, False), (4, False), (5, True), (8, True), (9, False), (64, False)):
        out = ops.linear(_rand((m, 896), torch.bfloat16, 223).cuda(), w_small, None, for_stream=True)
        assert isinstance(out, PendingLinear) == expect, m
    assert not isinstance(ops.linear(_rand((8, 4864), torch.bfloat16, 224).cuda(), w_large, None, for_stream=True), PendingLinear)
    assert not isinstance(HipOps(torch.float32, gpu_device).linear(torch.zeros(8, 64).cuda(), torch.zeros(64, 64).cuda(), None, for_stream=True), PendingLinear)
    # a pending product that reaches the plain norm, an addition or a gather is run as a product of its own
    a = _rand((6, 896), torch.bfloat16, 225).cuda()
    pending = ops.linear(a, w_small, None, for_stream=True)
    assert isinstance(pending, PendingLinear)
    x = _rand((6, 896), torch.float32, 226).cuda()
    nw = torch.ones(896, dtype=torch.bfloat16).cuda()
    direct = ops.rmsnorm(x.clone(), nw, 1e-6, delta=ops.linear(a, w_small, None, partial_sums=True))
    assert torch.equal(ops.rmsnorm(x.clone(), nw, 1e-6, delta=pending), direct)
    rows = torch.tensor([4, 1], dtype=torch.int32).cuda()
    picked = ops.gather_rows(pending, rows)
    assert isinstance(picked, PendingLinear) and picked.shape == (2, 896)
    torch.testing.assert_close(ops.settle(picked).float().sum(0) if ops.settle(picked).dim() == 3 else ops.settle(picked).float(),
                               (a[rows.long()].float() @ w_small.float().t()), atol=3e-2, rtol=2e-2)
