"""A stand-in for the HIP kernel library, written with torch tensor operations.

It exists so that everything above the kernels (cache manager, step function,
scheduler, engine, replay) can be exercised on a machine without a GPU, the way
the reference's tests swap its Python oracle in for its CUDA kernel
(tests/test_engine.py:82-101 of the reference).  It is test code: the product
never imports it and has no path that computes without the HIP library.

Each method has the signature and the contract of the method of the same name of
`mini_llm_runtime_amd.kernels.ops.HipOps`.
"""

from __future__ import annotations

from typing import Optional

import torch


class TorchOps:
    def __init__(self, dtype: torch.dtype = torch.float32, device: str = "cpu") -> None:
        self.dtype = dtype
        self.device = torch.device(device)
        self.calls: dict[str, int] = {}

    def _count(self, name: str) -> None:
        self.calls[name] = self.calls.get(name, 0) + 1

    # residual stream ------------------------------------------------------------------
    def embedding(self, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        self._count("embedding")
        return table[ids.long()].float()

    def rmsnorm(self, x, weight, eps, delta=None):
        self._count("rmsnorm")
        assert x.dtype == torch.float32
        if delta is not None:
            x += delta.float().sum(0) if delta.dim() == 3 else delta.float()
        variance = x.pow(2).mean(-1, keepdim=True)
        return (weight.float() * (x * torch.rsqrt(variance + eps))).to(self.dtype)

    def add_(self, x, delta):
        x += delta.float()

    def scale_softcap_(self, x, scale=1.0, cap=None):
        x *= scale
        if cap is not None:
            x.copy_(cap * torch.tanh(x / cap))

    def gather_rows(self, x, rows):
        return (x[:, rows.long()] if x.dim() == 3 else x[rows.long()]).contiguous()

    # matrix products ---------------------------------------------------------------------
    def linear(self, x, weight, bias=None, out_dtype=None, kernel="auto", swiglu=False, partial_sums=False, for_stream=False):
        self._count("linear")
        y = x.float() @ weight.float().t()
        if bias is not None:
            y = y + bias.float()
        if swiglu:  # rows of weight: gate 2j, gate 2j+1, up 2j, up 2j+1
            quads = y.view(y.shape[0], -1, 4)
            gate, up = quads[..., :2], quads[..., 2:]
            y = (gate * torch.sigmoid(gate) * up).reshape(y.shape[0], -1)
        return y.to(out_dtype or self.dtype)

    def silu_mul(self, gate_up):
        inter = gate_up.shape[1] // 2
        g = gate_up[:, :inter].float()
        u = gate_up[:, inter:].float()
        return (g * torch.sigmoid(g) * u).to(self.dtype)

    # positions and cache --------------------------------------------------------------------
    def rope_table(self, positions, inv_freq):
        ang = positions.double()[:, None] * inv_freq.double()[None, :]
        return ang.cos().float(), ang.sin().float()

    def rope_kv_write(
        self, qkv, rotation, slot_mapping, key_pages, value_pages, *, num_heads, num_kv_heads, head_dim, block_size, write=True
    ):
        self._count("rope_kv_write")
        tokens = qkv.shape[0]
        qs = num_heads * head_dim
        ks = num_kv_heads * head_dim
        q = qkv[:, :qs].view(tokens, num_heads, head_dim)
        k = qkv[:, qs : qs + ks].view(tokens, num_kv_heads, head_dim)
        v = qkv[:, qs + ks :].view(tokens, num_kv_heads, head_dim)
        if rotation is not None:
            cos, sin, r = rotation
            half = r // 2
            for t in (q, k):
                a = t[..., :half].float().clone()
                b = t[..., half:r].float().clone()
                c = cos[:, None, :]
                s = sin[:, None, :]
                t[..., :half] = (a * c - b * s).to(t.dtype)
                t[..., half:r] = (b * c + a * s).to(t.dtype)
        if write:
            slots = slot_mapping.long()
            ok = slots >= 0
            page = slots[ok] // block_size
            off = slots[ok] % block_size
            key_pages[page, :, off, :] = k[ok]
            value_pages[page, :, :, off] = v[ok]

    def qkv_rope_write(self, x, weight, bias, rotation, slot_mapping, key_pages, value_pages, **sizes):
        qkv = self.linear(x, weight, bias)
        self.rope_kv_write(qkv, rotation, slot_mapping, key_pages, value_pages, **sizes)
        return qkv

    def paged_attention(
        self, qkv, key_pages, value_pages, block_table, ctx, *, num_heads, num_kv_heads, head_dim, block_size, scale, window,
        defer_merge=False, plan=None,
    ):
        self._count("paged_attention")
        tokens = qkv.shape[0]
        group = num_heads // num_kv_heads
        q = qkv[:, : num_heads * head_dim].view(tokens, num_heads, head_dim).float()
        out = torch.zeros(tokens, num_heads, head_dim, dtype=torch.float32, device=qkv.device)
        table = block_table.long()
        for t in range(tokens):
            r = int(ctx.token_entry[t])
            p = int(ctx.positions[t])
            first = 0 if window is None else max(0, p - window + 1)
            idx = torch.arange(first, p + 1)
            page = table[r, idx // block_size]
            assert (page >= 0).all(), "attention would read a page that is not there"
            k = key_pages[page, :, idx % block_size, :].float()  # [n, Hkv, d]
            v = value_pages[page, :, :, idx % block_size].float()
            k = k.repeat_interleave(group, dim=1)
            v = v.repeat_interleave(group, dim=1)
            s = torch.einsum("hd,nhd->hn", q[t], k) * scale
            w = torch.softmax(s, dim=-1)
            out[t] = torch.einsum("hn,nhd->hd", w, v)
        return out.reshape(tokens, num_heads * head_dim).to(self.dtype)

    # sampling ----------------------------------------------------------------------------------
    def sample(self, logits, temperature: Optional[torch.Tensor], uniform: Optional[torch.Tensor]):
        self._count("sample")
        greedy = torch.argmax(logits, dim=-1).to(torch.int32)
        if temperature is None:
            return greedy
        out = greedy.clone()
        for i in range(logits.shape[0]):
            t = float(temperature[i])
            if t > 0:
                z = logits[i].float()
                e = torch.exp((z - z.max()) / t)
                c = torch.cumsum(e, dim=0)
                target = float(uniform[i]) * float(c[-1])
                out[i] = min(int(torch.searchsorted(c, torch.tensor(target), right=True)), logits.shape[1] - 1)
        return out
