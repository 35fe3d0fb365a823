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
from test_gpu_kernels import _attention_reference, _paged_case, _rand, _tol

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
    pending = tuned.paged_attention(*args, defer_merge=True, **kw)
    assert isinstance(pending, PendingMerge) and pending.splits > 1
    attended = tuned.paged_attention(*args, **kw)
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
    pending = ops.paged_attention(q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx, num_heads=4, num_kv_heads=2,
                                  head_dim=32, block_size=16, scale=0.2, window=None, defer_merge=True)
    assert isinstance(pending, PendingMerge)
    out = ops.linear(pending, wo, None).float().cpu()
    assert torch.isfinite(out[0]).all() and torch.isnan(out[1]).all()


def test_mixed_batches_and_single_partitions_do_not_defer(ops):
    """Only a batch of single tokens whose keys are cut into partitions defers its merge."""
    kw = dict(num_heads=4, num_kv_heads=2, head_dim=32, block_size=16, scale=0.2, window=None, defer_merge=True)
    q, kp, vp, table, ctx, *_ = _paged_case([(40, 1), (30, 1)], 4, 2, 32, 16, torch.bfloat16, 104)
    assert isinstance(ops.paged_attention(q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx, **kw), torch.Tensor)
    q, kp, vp, table, ctx, *_ = _paged_case([(600, 1), (500, 20)], 4, 2, 32, 16, torch.bfloat16, 105)
    assert isinstance(ops.paged_attention(q.cuda(), kp.cuda(), vp.cuda(), table.cuda(), ctx, **kw), torch.Tensor)
