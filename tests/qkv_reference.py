"""What the query/key/value kernels must produce, computed in float64 from their inputs, with a
bound that says how far a correct kernel may be from it.

Every way of that operation (product, then rotation kernel; one fused kernel with 16 or 8 weight
rows a workgroup, tiled, or with a norm in front; product cut along k and a finishing kernel)
computes, in the reference's order (src/mini_llm_runtime/qwen_model_runner.py:88-109):

    p    = x W^T + b            accumulated in float32, in an order that differs between kernels
    p^   = bfloat16(p)          the product as the model's dtype holds it
    out  = p^[j] cos - p^[j + d/2] sin      (low half; the high half adds), in float32
    out^ = bfloat16(out)

The float64 value of p is exact to 1e-16; a kernel's float32 sum differs from it by e_sum, up to
2^-23 of sum |x w| (a few float32 roundings at the size of the partial sums; measured: a sixth of
that).  For most values that matters only when p lies that close to the middle between two bfloat16
values: then p^ lands on the neighbour, ONE ulp(p) away (ulp: the spacing of bfloat16 at that
magnitude, 2^-7 of the value's power of two).  For a p that is itself as small as e_sum (thousands of
products that cancel) e_sum is the whole error.  Below, u(p) = ulp(p) + e_sum.  The rotation carries that on as ulp(p_a) |cos| + ulp(p_b) |sin|, and
where the two products nearly cancel (a subtraction of equal-sized operands) this is large against
the result, which is why a bound relative to the result cannot be tight.  The last rounding adds half
an ulp of the result, one where out sits near a middle itself.  So, with every ulp in bfloat16:

    |out^ - out_ref| <= u(p_a) |cos| + u(p_b) |sin| + ulp(out) + e32          (rotated heads)
    |p^   - p_ref^ | <= u(p)                                                    (values, no rotation)

(ulp(out) at the larger of the reference's and the kernel's value: where the products cancel the
reference may be next to zero while the kernel's value, an operand's ulp away, is not; e32: the
float32 rounding of the rotation's two products, 2^-22 of their sizes)

and neighbours are rare: all but a few per cent of the elements equal the reference's own rounding.
"""

from __future__ import annotations

import torch


def bf16_ulp(v: torch.Tensor) -> torch.Tensor:
    """Spacing of bfloat16 values at the magnitude of v (float64 in, float64 out)."""
    mag = v.abs().clamp_min(2.0**-126)
    return torch.exp2(torch.floor(torch.log2(mag)) - 7)


def to_bf16(v: torch.Tensor) -> torch.Tensor:
    return v.to(torch.float32).to(torch.bfloat16).double()


def qkv_reference(x, w, b, cos, sin, heads, kv_heads, head_dim, p_slack=0.0):
    """x [T, K], w [(heads + 2 kv) d, K], b [(heads + 2 kv) d] or None, cos/sin [T, d/2] (float32
    tables as the kernel gets them) or None.  Returns (reference [T, heads + 2 kv, d] float64 before
    the last rounding, bound [same] on |kernel output - reference| without the last rounding's own
    ulp, exact [same]: the reference's own rounding, rotated [same]: where a last rounding follows).
    p_slack: how far a kernel's p may be off for reasons of its input (a norm computed
    in the same kernel whose output lands on a neighbouring bfloat16 value now and then)."""
    x, w = x.double().cpu(), w.double().cpu()
    p = x @ w.t()
    e_sum = 2.0**-23 * (x.abs() @ w.abs().t())
    if b is not None:
        p = p + b.double().cpu()
        e_sum = e_sum + 2.0**-23 * b.double().cpu().abs()
    tokens = x.shape[0]
    p = p.view(tokens, heads + 2 * kv_heads, head_dim)
    p_hat = to_bf16(p)
    u = bf16_ulp(p) + e_sum.view_as(p) + p_slack
    ref = p_hat.clone()
    bound = u.clone()
    rotated = torch.zeros(ref.shape, dtype=torch.bool)
    if cos is not None:
        half = head_dim // 2
        c = cos.double().cpu()[:, None, :]
        s = sin.double().cpu()[:, None, :]
        rot = heads + kv_heads  # queries and keys are rotated, values are not
        lo, hi = p_hat[:, :rot, :half], p_hat[:, :rot, half:]
        ulo, uhi = u[:, :rot, :half], u[:, :rot, half:]
        ref[:, :rot, :half] = lo * c - hi * s
        ref[:, :rot, half:] = hi * c + lo * s
        e32 = 2.0**-22 * ((lo * c).abs() + (hi * s).abs() + (hi * c).abs() + (lo * s).abs())
        bound[:, :rot, :half] = ulo * c.abs() + uhi * s.abs() + e32
        bound[:, :rot, half:] = uhi * c.abs() + ulo * s.abs() + e32
        rotated[:, :rot] = True
    return ref, bound, to_bf16(ref), rotated


def check_qkv(name, q, key_pages, value_pages, slots, block_size, reference, heads, kv_heads, head_dim, write=True,
              max_neighbours=0.03):
    """Compare one way's outputs (queries [T, >= heads d]; pages on the CPU as float, NaN where
    nothing was written) with `qkv_reference`'s result."""
    ref, bound, exact, rotated = reference
    tokens = ref.shape[0]
    got = torch.full_like(ref, float("nan"))
    got[:, :heads] = q[:, : heads * head_dim].double().cpu().view(tokens, heads, head_dim)
    compare = torch.zeros(ref.shape, dtype=torch.bool)
    compare[:, :heads] = True
    if write:
        slot_list = slots.cpu().tolist()
        kp, vp = key_pages.double().cpu(), value_pages.double().cpu()
        for t, slot in enumerate(slot_list):
            if slot < 0:
                continue
            page, off = divmod(slot, block_size)
            got[t, heads : heads + kv_heads] = kp[page, :, off, :]
            got[t, heads + kv_heads :] = vp[page, :, :, off]
            compare[t, heads:] = True
    assert torch.isfinite(got[compare]).all(), f"{name}: a value that should have been written is missing"
    last_rounding = torch.where(rotated, bf16_ulp(torch.maximum(ref.abs(), torch.nan_to_num(got).abs())), 0.0)
    excess = ((got - ref).abs() - (bound + last_rounding) * (1 + 1e-6))[compare]
    worst = float(excess.max())
    if worst > 0:
        at = torch.nonzero(((got - ref).abs() - (bound + last_rounding) * (1 + 1e-6) > 0) & compare)[0].tolist()
        t, h, d = at
        raise AssertionError(
            f"{name}: {int((excess > 0).sum())} of {excess.numel()} values outside the bound of one ulp per operand, "
            f"worst by {worst:.3e}; first at token {t} head {h} dim {d}: got {float(got[t, h, d])!r}, reference "
            f"{float(ref[t, h, d])!r}, bound {float(bound[t, h, d])!r} + {float(last_rounding[t, h, d])!r}"
        )
    neighbours = float((got != exact)[compare].double().mean())
    assert neighbours <= max_neighbours, f"{name}: {neighbours:.1%} of the values are not the reference's own rounding"
