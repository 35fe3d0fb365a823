"""The operations the parts compute with, bound to the HIP kernel library.

`HipOps` is the only implementation the product has: it loads the libraries that
`build.py` compiles for gfx950 and calls their extern "C" entry points through
ctypes with device pointers and the current HIP stream.  There is no CPU path;
constructing it without a GPU or without a working hipcc build raises.

Every method checks device, element type, layout and sizes of its tensors on the
host before a kernel is launched, so that a wrong call is an exception and never
a memory fault on the GPU.
"""

from __future__ import annotations

import ctypes
from typing import Any, Optional, Sequence, Union

import torch

from . import build
from .pending import PendingLinear, PendingMerge, PendingNorm, PendingScale
from .tuning import KernelTuning

_VP = ctypes.c_void_p
_I = ctypes.c_int
_I64 = ctypes.c_int64
_F = ctypes.c_float

_SIGNATURES = {
    "mlr_version": ([], _I),
    "mlr_embedding": ([_VP, _I, _VP, _VP, _I, _I, _I, _VP], _I),
    "mlr_rmsnorm": ([_VP, _VP, _VP, _I, _VP, _I, _VP, _I, _I, _I, _F, _VP], _I),
    "mlr_add": ([_VP, _VP, _I, _I64, _VP], _I),
    "mlr_scale_softcap": ([_VP, _F, _F, _I64, _VP], _I),
    "mlr_gather_rows": ([_VP, _VP, _VP, _I, _I64, _I, _I, _VP], _I),
    "mlr_silu_mul": ([_VP, _VP, _I, _I, _I, _VP], _I),
    "mlr_rope_table": ([_VP, _VP, _VP, _VP, _I, _I, _VP], _I),
    "mlr_rope_kv_write": ([_VP, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_qkv_finish": ([_VP, _I, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_gemm_simple": ([_VP, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_gemm_bf16": ([_VP, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _I, _I, _VP, _I, _F, _VP], _I),
    "mlr_gemm_residual_parts": ([_I, _I], _I),
    "mlr_gemm_residual_bf16": ([_VP, _VP, _VP, _I, _VP, _VP, _I, _VP, _VP, _I, _I, _I, _VP], _I),
    "mlr_gemm_bf16_slices": ([_I, _I, _I, _I], _I),
    "mlr_gemm_bf16_kernel": ([_I, _I, _I, _I], _I),
    "mlr_qkv_rope_write_bf16": (
        [_VP, _VP, _VP, _I, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _I, _VP, _I, _F, _VP],
        _I,
    ),
    "mlr_gemm_norm_fused_bf16": (
        [_VP, _VP, _VP, _VP, _I, _VP, _I, _F, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _I, _VP],
        _I,
    ),
    "mlr_qkv_norm_fused_bf16": (
        [_VP, _VP, _VP, _VP, _I, _VP, _I, _F, _VP, _VP, _I, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP],
        _I,
    ),
    "mlr_gemm_merge_fused_bf16": ([_VP, _VP, _I, _I, _I, _I, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _VP], _I),
    "mlr_paged_attention_simple": (
        [_VP, _I64, _VP, _VP, _VP, _I, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _VP],
        _I,
    ),
    "mlr_sample": ([_VP, _VP, _VP, _VP, _VP, _I, _I, _VP], _I),
    "mlr_sample_scratch": ([_I, _I], _I64),
    "mlr_attention_head_dim": ([], _I),
    "mlr_attention_key_tile": ([], _I),
    "mlr_attention_wide_tile": ([], _I),
    "mlr_attention_decode_scratch": ([_I, _I, _I], _I64),
    "mlr_attention_decode": (
        [_VP, _I64, _VP, _VP, _VP, _I, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _I, _I, _I, _VP],
        _I,
    ),
    "mlr_attention_decode_merge": ([_VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_attention_prefill_scratch": ([_I, _I, _I, _I], _I64),
    "mlr_attention_prefill": (
        [_VP, _I64, _VP, _VP, _VP, _I, _VP, _I, _I, _VP, _VP, _VP, _I, _I, _I, _I, _F, _I, _I, _VP, _VP],
        _I,
    ),
}

from .plans import PAGED_ATTENTION, QUERY_TILE, WIDE_QUERY_TILE, attention_plan, query_tiles  # noqa: F401


class KernelError(RuntimeError):
    """An entry point of the kernel library refused its arguments or failed to launch."""


def _dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise KernelError(f"the kernels take float32 or bfloat16, not {dtype}")


def load_library(module: build.Module = build.CORE) -> ctypes.CDLL:
    path = build.ensure_module(module)
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelError(f"cannot load the HIP kernel library {path}: {e}") from None
    lib.mlr_last_error.restype = ctypes.c_char_p
    lib.mlr_last_error.argtypes = []
    for name, (argtypes, restype) in _SIGNATURES.items():
        if hasattr(lib, name):
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
    return lib


class HipOps:
    def __init__(
        self,
        dtype: torch.dtype = torch.bfloat16,
        device: Union[str, torch.device] = "cuda",
        tuning: Optional[KernelTuning] = None,
    ) -> None:
        self.dtype = dtype
        self.tuning = tuning or KernelTuning()
        self.code = _dtype_code(dtype)
        device = torch.device(device)
        if device.type != "cuda":
            raise KernelError(
                f"the engine computes on an AMD GPU only (device {device} asked for); there is no CPU path"
            )
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible to this process; the engine has no CPU path")
        if device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self.device = device
        self.lib = load_library(build.CORE)
        if self.lib.mlr_version() != 1:
            raise KernelError("the built kernel library is of another version than this package")
        self._attention_libs: dict[int, ctypes.CDLL] = {}
        self.decode_partition = self.tuning.decode_partition
        self.max_k_slices = self.tuning.max_k_slices
        self.decode_max_groups = self.tuning.decode_max_groups

    def attention_library(self, head_dim: int) -> ctypes.CDLL:
        """The MFMA attention kernels of one head size, compiled on first use."""
        lib = self._attention_libs.get(head_dim)
        if lib is None:
            lib = load_library(build.attention_module(head_dim))
            if lib.mlr_attention_head_dim() != head_dim:
                raise KernelError(f"the attention library for head size {head_dim} was built for another size")
            self._attention_libs[head_dim] = lib
        return lib

    # ---- plans --------------------------------------------------------------------------------
    ATTENTION_PLAN = PAGED_ATTENTION

    @staticmethod
    def attention_plan(shape):
        """The plan `paged_attention` wants for a step of this shape (see kernels/plans.py)."""
        return attention_plan(shape)

    # ---- helpers --------------------------------------------------------------------------
    def _stream(self) -> _VP:
        """The HIP stream torch currently runs on for this device (a capture stream inside a
        graph capture); asked for at every launch, so by the cheapest route torch offers."""
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:
            return _VP(raw(self.device.index))
        return _VP(torch.cuda.current_stream(self.device).cuda_stream)

    def _call(self, name: str, *args: Any, lib: Optional[ctypes.CDLL] = None) -> None:
        lib = lib or self.lib
        status = getattr(lib, name)(*args)
        if status != 0:
            raise KernelError(lib.mlr_last_error().decode("utf-8", "replace"))

    def _check(
        self,
        t: torch.Tensor,
        name: str,
        dtype: Optional[Union[torch.dtype, Sequence[torch.dtype]]] = None,
        shape: Optional[Sequence[Optional[int]]] = None,
    ) -> torch.Tensor:
        # runs several times per kernel launch: the passing case takes the short way
        if not isinstance(t, torch.Tensor):
            raise KernelError(f"{name} must be a tensor")
        if t.device != self.device:
            raise KernelError(f"{name} is on {t.device}, the kernels run on {self.device}")
        if not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous")
        if dtype is not None and t.dtype is not dtype:
            allowed = (dtype,) if isinstance(dtype, torch.dtype) else tuple(dtype)
            if t.dtype not in allowed:
                raise KernelError(f"{name} has dtype {t.dtype}, expected {' or '.join(map(str, allowed))}")
        if shape is not None:
            actual = t.shape
            ok = len(actual) == len(shape)
            if ok:
                for want, have in zip(shape, actual):
                    if want is not None and want != have:
                        ok = False
                        break
            if not ok:
                raise KernelError(f"{name} has shape {tuple(actual)}, expected {tuple(shape)}")
        return t

    @staticmethod
    def _ptr(t: Optional[torch.Tensor]) -> _VP:
        return _VP(None if t is None else t.data_ptr())

    def _empty(self, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        return torch.empty(tuple(shape), dtype=dtype, device=self.device)

    # ---- residual stream --------------------------------------------------------------------
    def embedding(self, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        self._check(table, "embedding table", self.dtype, (None, None))
        self._check(ids, "token ids", torch.int32, (None,))
        vocab, hidden = table.shape
        out = self._empty((ids.shape[0], hidden), torch.float32)
        self._call(
            "mlr_embedding", self._ptr(table), self.code, self._ptr(ids), self._ptr(out),
            ids.shape[0], hidden, vocab, self._stream(),
        )
        return out

    def rmsnorm(
        self, x: torch.Tensor, weight: torch.Tensor, eps: float, delta: Optional[torch.Tensor] = None
    ) -> torch.Tensor:
        """x (float32 residual stream [rows, hidden]) += delta in place, then the RMSNorm of x
        in the engine's dtype.  delta: [rows, hidden] in the engine's dtype, or a float32 stack
        [S, rows, hidden] of partial sums (see `linear`), or None."""
        self._check(x, "residual stream", torch.float32, (None, None))
        rows, hidden = x.shape
        self._check(weight, "norm weight", (torch.float32, self.dtype), (hidden,))
        delta = self.settle(delta)
        plain = partial = None
        slices = 0
        if delta is not None and delta.dim() == 3:
            partial = self._check(delta, "partial sums", torch.float32, (None, rows, hidden))
            slices = delta.shape[0]
        elif delta is not None:
            plain = self._check(delta, "residual delta", self.dtype, (rows, hidden))
        out = self._empty((rows, hidden), self.dtype)
        self._call(
            "mlr_rmsnorm", self._ptr(x), self._ptr(plain), self._ptr(partial), slices, self._ptr(weight),
            int(weight.dtype == torch.float32), self._ptr(out), self.code, rows, hidden, float(eps), self._stream(),
        )
        return out

    def add_(self, x: torch.Tensor, delta: torch.Tensor) -> None:
        """x (float32) += delta (the engine's dtype, or float32), in place."""
        self._check(x, "residual stream", torch.float32)
        delta = self.settle(delta)
        self._check(delta, "residual delta", (self.dtype, torch.float32), tuple(x.shape))
        self._call("mlr_add", self._ptr(x), self._ptr(delta), _dtype_code(delta.dtype), x.numel(), self._stream())

    def scale_softcap_(self, x: torch.Tensor, scale: float = 1.0, cap: Optional[float] = None) -> None:
        """x (float32) = x * scale, then, with a cap, cap * tanh(x / cap); in place."""
        self._check(x, "values", torch.float32)
        if cap is not None and not cap > 0:
            raise KernelError("a soft cap must be > 0")
        self._call("mlr_scale_softcap", self._ptr(x), float(scale), float(cap or 0.0), x.numel(), self._stream())

    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """x[rows] for x [T, H], or x[:, rows] for a stack [S, T, H].  Of a product that has not run,
        the product of the chosen rows of its input, still not run: a row's values are then made by
        the same kernels whether it was chosen or all rows were taken."""
        if isinstance(x, PendingLinear):
            return PendingLinear(self.gather_rows(self.settle(x.x), rows), x.weight, x.bias)
        x = self.settle(x)
        self._check(x, "rows source", (torch.float32, torch.bfloat16))
        if x.dim() not in (2, 3):
            raise KernelError("gather_rows takes [T, H] or [S, T, H]")
        self._check(rows, "row indices", torch.int32, (None,))
        planes = x.shape[0] if x.dim() == 3 else 1
        src_rows, width = x.shape[-2], x.shape[-1]
        row_bytes = width * x.element_size()
        if row_bytes % 4:
            raise KernelError("gather_rows needs rows that are a multiple of 4 bytes wide")
        shape = (planes, rows.shape[0], width) if x.dim() == 3 else (rows.shape[0], width)
        out = self._empty(shape, x.dtype)
        self._call(
            "mlr_gather_rows", self._ptr(x), self._ptr(rows), self._ptr(out), rows.shape[0], row_bytes,
            src_rows, planes, self._stream(),
        )
        return out

    # ---- activations made inside the product that uses them ------------------------------------
    FUSED_TOKENS = 16  # the merge prologue takes up to this many tokens
    FUSED_NORM_TOKENS = 4  # the norm prologue up to this many (a wavefront per row)
    FUSED_NORM_WIDTH = 2048  # and rows up to this width
    FUSED_LDS_BYTES = 140 * 1024

    def defer_norm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, delta: Optional[torch.Tensor]):
        """The norm of `rmsnorm` as a `PendingNorm` when the product behind it could compute it
        in its own kernel (bfloat16, few tokens, a narrow model); else None."""
        if isinstance(delta, PendingLinear):
            return self._finish_stream(x, weight, float(eps), delta)  # None: the caller's norm kernel settles it
        if not (self.tuning.fuse_norm and self.dtype == torch.bfloat16 and x.dim() == 2):
            return None
        rows, hidden = x.shape
        if rows > self.FUSED_NORM_TOKENS or hidden > self.FUSED_NORM_WIDTH or hidden % 8:
            return None
        slices = delta.shape[0] if delta is not None and delta.dim() == 3 else 0
        if (1 + slices) * rows * hidden * 4 > self.tuning.fuse_bytes:  # every workgroup reads all of it
            return None
        return PendingNorm(x, delta, weight, float(eps))

    def settle(self, h):
        """The tensor behind a pending activation (run by a kernel of its own); tensors pass."""
        if isinstance(h, PendingNorm):
            if h.value is None:
                h.value = self.rmsnorm(h.x, h.weight, h.eps, delta=h.delta)
                h.residual = h.x
            return h.value
        if isinstance(h, PendingScale):
            if h.value is None:
                h.value = self.rmsnorm(h.residual, h.weight, h.eps)
            return h.value
        if isinstance(h, PendingLinear):
            return self.linear(h.x, h.weight, h.bias, partial_sums=True)
        if isinstance(h, PendingMerge):
            out = self._empty((h.tokens, h.heads * h.head_dim), self.dtype)
            self._call(
                "mlr_attention_decode_merge", self._ptr(h.partial), self._ptr(h.cu_q), self._ptr(h.context_lens),
                self._ptr(out), h.tokens, h.heads, h.window, h.part, h.splits, self._stream(), lib=h.library,
            )
            return out
        return h

    def _can_finish_stream(self, m: int, n: int, k: int) -> bool:
        """Whether the product [m, k] x [n, k]^T may run as the kernel that adds its result to the
        residual stream itself (`mlr_gemm_residual_bf16`): where the limits of the tuning say so."""
        t = self.tuning
        return (
            t.finish_stream and self.dtype == torch.bfloat16 and k % 8 == 0 and n % 4 == 0
            and max(1, t.finish_min_tokens) <= m <= min(64, t.finish_max_tokens)
            and n * k * 2 <= t.finish_weight_bytes and m * k * 2 <= t.finish_activation_bytes
        )

    def _finish_stream(self, x: torch.Tensor, weight: torch.Tensor, eps: float, pending: PendingLinear):
        """Run a pending product as the kernel that adds it to the stream `x` (in place) and leaves
        the norm's activations short of the factor per row: a `PendingScale`."""
        self._check(x, "residual stream", torch.float32, (None, None))
        rows, hidden = x.shape
        a = self.settle(pending.x)  # attention still in partitions is merged by its own kernel
        m, k = a.shape
        if m != rows or pending.weight.shape[0] != hidden or not self._can_finish_stream(m, hidden, k):
            return None
        self._check(a, "linear input", self.dtype, (m, k))
        self._check(pending.weight, "linear weight", self.dtype, (hidden, k))
        self._check(weight, "norm weight", (torch.float32, self.dtype), (hidden,))
        bias = pending.bias
        if bias is not None:
            self._check(bias, "linear bias", (torch.float32, self.dtype), (hidden,))
        parts = self.lib.mlr_gemm_residual_parts(m, hidden)
        h = self._empty((m, hidden), self.dtype)
        sumsq = self._empty((m, parts), torch.float32)
        self._call(
            "mlr_gemm_residual_bf16", self._ptr(a), self._ptr(pending.weight), self._ptr(bias),
            int(bias is not None and bias.dtype == torch.float32), self._ptr(x), self._ptr(weight),
            int(weight.dtype == torch.float32), self._ptr(h), self._ptr(sumsq), m, hidden, k, self._stream(),
        )
        return PendingScale(h, sumsq, weight, eps, x)

    @staticmethod
    def _no_scale() -> tuple:
        return (_VP(None), 0, 0.0)

    def _scale_arguments(self, h: PendingScale) -> tuple:
        return (self._ptr(h.sumsq), h.sumsq.shape[1], float(h.eps))

    def _norm_arguments(self, h: PendingNorm):
        """(checked tensors, ctypes arguments) of a norm prologue; allocates the updated stream."""
        x = self._check(h.x, "residual stream", torch.float32, (None, None))
        rows, hidden = x.shape
        self._check(h.weight, "norm weight", (torch.float32, self.dtype), (hidden,))
        plain = partial = None
        slices = 0
        if h.delta is not None and h.delta.dim() == 3:
            partial = self._check(h.delta, "partial sums", torch.float32, (None, rows, hidden))
            slices = partial.shape[0]
        elif h.delta is not None:
            plain = self._check(h.delta, "residual delta", self.dtype, (rows, hidden))
        x_out = self._empty((rows, hidden), torch.float32) if h.delta is not None else None
        args = (
            self._ptr(x), self._ptr(x_out), self._ptr(plain), self._ptr(partial), slices, self._ptr(h.weight),
            int(h.weight.dtype == torch.float32), float(h.eps),
        )
        return x_out if x_out is not None else x, args

    # ---- matrix products ----------------------------------------------------------------------
    def linear(
        self,
        x: torch.Tensor,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        out_dtype: Optional[torch.dtype] = None,
        kernel: str = "auto",
        swiglu: bool = False,
        partial_sums: bool = False,
        mfma_kernel: int = 0,
        slices: Optional[int] = None,
        for_stream: bool = False,
    ) -> torch.Tensor:
        """x [M, K] times weight [N, K] transposed, plus bias [N]; F.linear semantics.

        for_stream: the result is a part's output and goes nowhere but into the next norm as its
        delta (as with partial_sums); it may then come back unrun, as a `PendingLinear` that the norm
        runs together with the addition to the residual stream.

        bfloat16 products run on the matrix cores when k is a multiple of 8; float32
        products, and everything with kernel="fma", run as plain 32-bit FMA arithmetic.
        swiglu: the rows of `weight` are groups (gate 2j, gate 2j+1, up 2j, up 2j+1) and
        the result is silu(gate) * up, [M, N / 2].
        partial_sums: the caller hands the result to a norm as a not-yet-added delta and
        accepts, instead of [M, N], a float32 stack [S, M, N] of partial sums over slices
        of k (bias in slice 0).  Narrow products of a few tokens are cut that way so that
        all compute units stream the weight; the norm kernel adds the slices in order.
        mfma_kernel, slices: force one of the matrix-core kernels (16, 14, 11, 22, 23, 44 to 48, 62 to 68) and a number
        of k slices instead of letting the shape choose; for tests and tuning.
        """
        if kernel not in ("auto", "fma"):
            raise KernelError("kernel must be 'auto' or 'fma'")
        if for_stream:
            partial_sums = True
            m, k = x.shape
            if (
                kernel == "auto" and not swiglu and not mfma_kernel and slices is None and out_dtype in (None, self.dtype)
                and not isinstance(x, (PendingNorm, PendingScale)) and self._can_finish_stream(m, weight.shape[0], k)
            ):
                return PendingLinear(x, weight, bias)
        if isinstance(x, (PendingNorm, PendingMerge)):
            fused = self._linear_fused(x, weight, bias, out_dtype, kernel, swiglu, partial_sums, mfma_kernel, slices)
            if fused is not None:
                return fused
            x = self.settle(x)
        scale = self._no_scale()
        if isinstance(x, PendingScale):
            if x.value is None and kernel == "auto" and self.dtype == torch.bfloat16 and x.h.shape[1] % 8 == 0:
                scale, x = self._scale_arguments(x), x.h  # the product scales its sums row by row
            else:
                x = self.settle(x)
        self._check(x, "linear input", self.dtype, (None, None))
        m, k = x.shape
        self._check(weight, "linear weight", self.dtype, (None, k))
        n = weight.shape[0]
        if bias is not None:
            self._check(bias, "linear bias", (torch.float32, self.dtype), (n,))
        if swiglu and (n % 4 or bias is not None):
            raise KernelError("a SwiGLU product needs a multiple of 4 rows and no bias")
        out_dtype = out_dtype or self.dtype
        if out_dtype not in (torch.float32, self.dtype):
            raise KernelError(f"linear output must be float32 or {self.dtype}")
        bias_f32 = int(bias is not None and bias.dtype == torch.float32)
        if kernel == "auto" and self.dtype == torch.bfloat16 and k % 8 == 0:
            if slices is None:
                slices = 1
                if partial_sums and not swiglu:
                    slices = self.lib.mlr_gemm_bf16_slices(m, n, k, self.max_k_slices)
            elif slices < 1 or (slices > 1 and not (partial_sums and not swiglu)):
                raise KernelError("k slices need partial_sums and no SwiGLU")
            if slices > 1:
                y = self._empty((slices, m, n), torch.float32)
                out_f32 = 1
            else:
                y = self._empty((m, n // 2 if swiglu else n), out_dtype)
                out_f32 = int(out_dtype == torch.float32)
            self._call(
                "mlr_gemm_bf16", self._ptr(x), self._ptr(weight), self._ptr(bias), bias_f32, self._ptr(y), out_f32,
                int(swiglu), slices, int(mfma_kernel), m, n, k, *scale, self._stream(),
            )
            return y
        y = self._empty((m, n // 2 if swiglu else n), out_dtype)
        self._call(
            "mlr_gemm_simple", self._ptr(x), self._ptr(weight), self._ptr(bias), bias_f32, self._ptr(y),
            int(out_dtype == torch.float32), int(swiglu), self.code, m, n, k, self._stream(),
        )
        return y

    def _linear_fused(self, x, weight, bias, out_dtype, kernel, swiglu, partial_sums, mfma_kernel, slices):
        """`linear` on a pending activation in one kernel, or None when that cannot be."""
        m, k = x.shape
        if kernel != "auto" or mfma_kernel or self.dtype != torch.bfloat16 or k % 8 or m > self.FUSED_TOKENS:
            return None
        self._check(weight, "linear weight", self.dtype, (None, k))
        n = weight.shape[0]
        if bias is not None:
            self._check(bias, "linear bias", (torch.float32, self.dtype), (n,))
        if swiglu and (n % 4 or bias is not None):
            raise KernelError("a SwiGLU product needs a multiple of 4 rows and no bias")
        out_dtype = out_dtype or self.dtype
        bias_f32 = int(bias is not None and bias.dtype == torch.float32)
        if isinstance(x, PendingNorm):
            if x.value is not None or slices not in (None, 1) or m > self.FUSED_NORM_TOKENS:
                return None
            if n * k * 2 > min(self.tuning.fuse_weight_bytes, (1 << 32) - 1):  # 32-bit offsets into the weights
                return None
            # no K slices here: every workgroup needs whole rows for the norm's statistics
            residual, norm_args = self._norm_arguments(x)
            y = self._empty((m, n // 2 if swiglu else n), out_dtype)
            self._call(
                "mlr_gemm_norm_fused_bf16", *norm_args, self._ptr(weight), self._ptr(bias), bias_f32, self._ptr(y),
                int(out_dtype == torch.float32), int(swiglu), 0, m, n, k, self._stream(),
            )
            x.residual = residual
            return y
        if swiglu or not self.tuning.fuse_merge or n * k * 2 > min(self.tuning.fuse_weight_bytes, (1 << 32) - 1):
            return None
        if slices is None:
            slices = self.lib.mlr_gemm_bf16_slices(m, n, k, self.max_k_slices) if partial_sums else 1
        elif slices > 1 and not partial_sums:
            raise KernelError("k slices need partial_sums")
        per_slice = -(-(-(-k // 32)) // slices) * 32  # columns of a slice, in whole MFMA steps
        if m * (per_slice // 8) > 256 or m * (per_slice + 8) * 2 > self.FUSED_LDS_BYTES:
            return None  # a thread merges one chunk of 8 columns
        if m * per_slice * x.splits * 4 > self.tuning.fuse_bytes:  # what every workgroup reads to merge
            return None
        if slices > 1:
            y = self._empty((slices, m, n), torch.float32)
        else:
            y = self._empty((m, n), out_dtype)
        self._call(
            "mlr_gemm_merge_fused_bf16", self._ptr(x.partial), self._ptr(x.context_lens), x.heads, x.head_dim, x.window,
            x.part, x.splits, self._ptr(weight), self._ptr(bias), bias_f32, self._ptr(y),
            int(slices > 1 or out_dtype == torch.float32), slices, m, n, self._stream(),
        )
        return y

    def silu_mul(self, gate_up: torch.Tensor) -> torch.Tensor:
        self._check(gate_up, "gate_up", self.dtype, (None, None))
        rows, width = gate_up.shape
        if width % 2:
            raise KernelError("gate_up must have an even width")
        out = self._empty((rows, width // 2), self.dtype)
        self._call("mlr_silu_mul", self._ptr(gate_up), self._ptr(out), self.code, rows, width // 2, self._stream())
        return out

    # ---- positions and cache ---------------------------------------------------------------------
    def rope_table(self, positions: torch.Tensor, inv_freq: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        self._check(positions, "positions", torch.int32, (None,))
        self._check(inv_freq, "inverse frequencies", torch.float64, (None,))
        tokens, half = positions.shape[0], inv_freq.shape[0]
        cos = self._empty((tokens, half), torch.float32)
        sin = self._empty((tokens, half), torch.float32)
        self._call(
            "mlr_rope_table", self._ptr(positions), self._ptr(inv_freq), self._ptr(cos), self._ptr(sin),
            tokens, half, self._stream(),
        )
        return cos, sin

    def _check_pages(self, key_pages, value_pages, num_kv_heads, head_dim, block_size) -> int:
        """Pages as the attention kernels read them: values as wide as keys."""
        self._check(key_pages, "key pages", self.dtype, (None, num_kv_heads, block_size, head_dim))
        self._check(value_pages, "value pages", self.dtype, (key_pages.shape[0], num_kv_heads, head_dim, block_size))
        return key_pages.shape[0]

    def rope_kv_write(
        self,
        qkv: torch.Tensor,
        rotation: Optional[tuple[torch.Tensor, torch.Tensor, int]],
        slot_mapping: torch.Tensor,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        *,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        block_size: int,
        write: bool = True,
    ) -> None:
        width = (num_heads + 2 * num_kv_heads) * head_dim
        self._check(qkv, "qkv", self.dtype, (None, width))
        tokens = qkv.shape[0]
        cos = sin = None
        rotary_dim = 0
        if rotation is not None:
            cos, sin, rotary_dim = rotation
            if rotary_dim <= 0 or rotary_dim % 2 or rotary_dim > head_dim:
                raise KernelError("rotary_dim must be even and within head_dim")
            self._check(cos, "rotary cos", torch.float32, (tokens, rotary_dim // 2))
            self._check(sin, "rotary sin", torch.float32, (tokens, rotary_dim // 2))
        num_pages = 0
        if write:
            num_pages = self._check_pages(key_pages, value_pages, num_kv_heads, head_dim, block_size)
            self._check(slot_mapping, "slot mapping", torch.int32, (tokens,))
        self._call(
            "mlr_rope_kv_write", self._ptr(qkv), self.code, self._ptr(cos), self._ptr(sin),
            self._ptr(slot_mapping if write else None), self._ptr(key_pages if write else None),
            self._ptr(value_pages if write else None), tokens, num_heads, num_kv_heads, head_dim, rotary_dim,
            block_size, num_pages, int(write), self._stream(),
        )

    def qkv_rope_write(
        self,
        x: torch.Tensor,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor],
        rotation: Optional[tuple[torch.Tensor, torch.Tensor, int]],
        slot_mapping: torch.Tensor,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        *,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        block_size: int,
        write: bool = True,
        fused: Optional[bool] = None,
        mfma_kernel: int = 0,
        sliced: Optional[bool] = None,
    ) -> torch.Tensor:
        """Query/key/value product, rotation of queries and keys, keys and values into the cache.

        Returns a tensor whose leading num_heads * head_dim columns are the position-encoded
        queries, for `paged_attention`.  In bfloat16 with a full rotation this is ONE kernel
        that rotates the sums and stores them where they belong (a row-splitting kernel for up
        to 64 tokens, a tiled one beyond) unless the product is large; everything else is the
        product followed by `rope_kv_write`.  Up to 64 tokens of a wide product (tens of
        megabytes of weights), and 65 to 128 tokens from 8 MB on, go a third way: the product cut
        along k through the LDS-tiled kernel, which streams such weights twice as fast as the
        row-splitting one, and a small kernel that adds the slices up, rotates and stores.
        `fused` and `sliced` force a way, `mfma_kernel` the fused kernel (tests).
        """
        pending = x if isinstance(x, PendingNorm) and x.value is None else None
        if isinstance(x, PendingNorm) and pending is None:
            x = x.value
        scaled = None  # rows that still owe their normalisation: every way below ends in a product that pays it
        if isinstance(x, PendingScale):
            if x.value is None and self.dtype == torch.bfloat16 and x.h.shape[1] % 8 == 0:
                scaled = x
            else:
                x = self.settle(x)
        m, k = x.shape
        width = (num_heads + 2 * num_kv_heads) * head_dim
        can_fuse = (
            self.dtype == torch.bfloat16
            and k % 8 == 0
            and head_dim % 16 == 0
            and (rotation is None or rotation[2] == head_dim)
            and (m <= 16 or width * k * 2 < 1 << 31)
        )
        if sliced is None:
            # measured: the second kernel costs 3.5 to 5 us, which the tiled product wins back from
            # 24 MB of weights on (from 4 tokens; 64 MB: from one), or from 8 MB beyond 32 tokens
            weight_bytes = width * k * 2
            pays = (
                weight_bytes >= 64 << 20
                or (weight_bytes >= 24 << 20 and m >= 4)
                or (weight_bytes >= 8 << 20 and m > 32)
            )
            sliced = fused is None and can_fuse and pending is None and not mfma_kernel and m <= 64 and pays and k >= 512
            # 65 to 128 tokens: the fused tiled kernel reads the weights once per 64 tokens; cut along K
            # where the estimate of the plain product says so, the product and the finishing kernel
            # are 1.2 to 1.5 times faster from 8 MB of weights on (7B at 96 tokens: 33 us against 24)
            if (
                not sliced and fused is None and can_fuse and pending is None and not mfma_kernel
                and 64 < m <= 128 and weight_bytes >= 8 << 20
            ):
                mid_slices = self.lib.mlr_gemm_bf16_slices(m, width, k, 4)
                sliced = mid_slices > 1
        elif sliced and not (can_fuse and pending is None and m <= 128 and k >= 512):
            raise KernelError("the sliced query/key/value product takes up to 128 bfloat16 tokens and a full rotation")
        if sliced:
            slices = (8 if k >= 2048 else 4) if m <= 64 else max(2, self.lib.mlr_gemm_bf16_slices(m, width, k, 4))
            partial = self.linear(x, weight, bias, partial_sums=True, slices=slices)  # scales each slice, if owed
            cos = sin = None
            if rotation is not None:
                cos, sin, _ = rotation
                self._check(cos, "rotary cos", torch.float32, (m, head_dim // 2))
                self._check(sin, "rotary sin", torch.float32, (m, head_dim // 2))
            num_pages = 0
            if write:
                num_pages = self._check_pages(key_pages, value_pages, num_kv_heads, head_dim, block_size)
                self._check(slot_mapping, "slot mapping", torch.int32, (m,))
            q = self._empty((m, num_heads * head_dim), self.dtype)
            self._call(
                "mlr_qkv_finish", self._ptr(partial), slices, self._ptr(cos), self._ptr(sin),
                self._ptr(slot_mapping if write else None), self._ptr(key_pages if write else None),
                self._ptr(value_pages if write else None), self._ptr(q), m, num_heads, num_kv_heads, head_dim,
                block_size, num_pages, int(write), self._stream(),
            )
            return q
        if fused is None:
            # Measured at 2,048 tokens: the fused kernel wins while the product is small (0.5B to 3B
            # widths, and any width up to some 512 tokens); where the plain product would run in
            # 256 x 256 tiles (7B, 32B) it is 15 % faster followed by the rotation kernel.
            large = m > 64 and -(-m // 256) * -(-width // 256) >= 144
            fused = can_fuse and not large
        elif fused and not can_fuse:
            raise KernelError("the fused query/key/value kernel takes bfloat16 tokens and a full rotation")
        if pending is not None and not (
            fused and not mfma_kernel and m <= self.FUSED_NORM_TOKENS
            and width * k * 2 <= min(self.tuning.fuse_weight_bytes, (1 << 32) - 1)
        ):
            x, pending = self.settle(pending), None
        if not fused:
            qkv = self.linear(x, weight, bias)
            self.rope_kv_write(
                qkv, rotation, slot_mapping, key_pages, value_pages, num_heads=num_heads,
                num_kv_heads=num_kv_heads, head_dim=head_dim, block_size=block_size, write=write,
            )
            return qkv
        scale = self._no_scale()
        if scaled is not None:
            scale, x = self._scale_arguments(scaled), scaled.h
        if pending is None:
            self._check(x, "linear input", self.dtype, (None, None))
        self._check(weight, "qkv weight", self.dtype, (width, k))
        if bias is not None:
            self._check(bias, "qkv bias", (torch.float32, self.dtype), (width,))
        cos = sin = None
        if rotation is not None:
            cos, sin, _ = rotation
            self._check(cos, "rotary cos", torch.float32, (m, head_dim // 2))
            self._check(sin, "rotary sin", torch.float32, (m, head_dim // 2))
        num_pages = 0
        if write:
            num_pages = self._check_pages(key_pages, value_pages, num_kv_heads, head_dim, block_size)
            self._check(slot_mapping, "slot mapping", torch.int32, (m,))
        q = self._empty((m, num_heads * head_dim), self.dtype)
        if pending is not None:
            residual, norm_args = self._norm_arguments(pending)
            self._call(
                "mlr_qkv_norm_fused_bf16", *norm_args, self._ptr(weight), self._ptr(bias),
                int(bias is not None and bias.dtype == torch.float32), self._ptr(cos), self._ptr(sin),
                self._ptr(slot_mapping if write else None), self._ptr(key_pages if write else None),
                self._ptr(value_pages if write else None), self._ptr(q), m, k, num_heads, num_kv_heads, head_dim,
                block_size, num_pages, int(write), self._stream(),
            )
            pending.residual = residual
            return q
        self._call(
            "mlr_qkv_rope_write_bf16", self._ptr(x), self._ptr(weight), self._ptr(bias),
            int(bias is not None and bias.dtype == torch.float32), self._ptr(cos), self._ptr(sin),
            self._ptr(slot_mapping if write else None), self._ptr(key_pages if write else None),
            self._ptr(value_pages if write else None), self._ptr(q), m, k, num_heads, num_kv_heads, head_dim,
            block_size, num_pages, int(write), mfma_kernel, *scale, self._stream(),
        )
        return q

    def paged_attention(
        self,
        qkv: torch.Tensor,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        block_table: torch.Tensor,
        ctx: Any,
        *,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        block_size: int,
        scale: float,
        window: Optional[int],
        kernel: str = "auto",
        defer_merge: bool = False,
        plan: Any = None,
    ):
        """Causal attention of the step's tokens over their requests' pages.

        defer_merge: the caller hands the result to `linear` and nothing else; when every
        entry has one token and their keys are cut into partitions, it may then receive a
        `PendingMerge` (the partitions, for that product to merge) instead of a tensor.
        plan: what `attention_plan` made for this step (query tiles, single-token entries and
        the bound on their contexts); without one the matrix-core kernels are not used.

        qkv: [T, >= num_heads * head_dim], queries in the leading columns (already
        position-encoded); returns [T, num_heads * head_dim].  `ctx` describes the
        batch (StepContext).  bfloat16 with a head size in steps of 16 and a block
        size that is a multiple of 4 runs on the matrix cores: single-token entries
        through the split-KV decode kernel, the others through the tiled prefill
        kernel.  Everything else (float32, other sizes, kernel="fma") runs the plain
        32-bit kernel.
        """
        self._check(qkv, "queries", self.dtype, (None, None))
        tokens, stride = qkv.shape
        if stride < num_heads * head_dim:
            raise KernelError("the query rows are narrower than num_heads * head_dim")
        if num_heads % num_kv_heads:
            raise KernelError("query heads must be a multiple of KV heads")
        num_pages = self._check_pages(key_pages, value_pages, num_kv_heads, head_dim, block_size)
        entries = ctx.num_entries
        self._check(block_table, "block table", torch.int32, (entries, None))
        self._check(ctx.token_entry, "token entries", torch.int32, (tokens,))
        self._check(ctx.positions, "positions", torch.int32, (tokens,))
        if block_table.shape[1] * block_size < ctx.max_context_len:
            raise KernelError("the block table is narrower than the longest context")
        if kernel not in ("auto", "fma"):
            raise KernelError("kernel must be 'auto' or 'fma'")
        out = self._empty((tokens, num_heads * head_dim), self.dtype)
        width = block_table.shape[1]
        use_mfma = (
            kernel == "auto"
            and self.dtype == torch.bfloat16
            and head_dim % 16 == 0
            and 16 <= head_dim <= 256
            and block_size % 4 == 0
            and stride % 8 == 0
        )
        num_tiles = int(getattr(plan, "num_query_tiles", 0))
        num_decode = int(getattr(plan, "num_decode_entries", 0))
        if use_mfma and num_tiles + num_decode == 0:
            use_mfma = False  # a caller that planned nothing (kernel tests of the plain path)
        lib = None
        if use_mfma:
            lib = self.attention_library(head_dim)
            if num_tiles and (block_size & (block_size - 1) or not 8 <= block_size <= lib.mlr_attention_key_tile()):
                use_mfma = False  # the tiled prefill kernel takes power-of-two pages from 8 up to its key tile
        if not use_mfma:
            self._call(
                "mlr_paged_attention_simple", self._ptr(qkv), stride, self._ptr(key_pages), self._ptr(value_pages),
                self._ptr(block_table), width, self._ptr(ctx.token_entry), self._ptr(ctx.positions),
                self._ptr(out), self.code, tokens, entries, num_heads, num_kv_heads, head_dim, block_size,
                num_pages, float(scale), int(window or 0), self._stream(),
            )
            return out
        self._check(ctx.cu_q, "cu_q", torch.int32, (entries + 1,))
        self._check(ctx.context_lens, "context lengths", torch.int32, (entries,))
        if num_decode:
            span = int(plan.max_decode_context)
            if window:
                span = min(span, int(window) + 15)
            group_tiles = -(-(num_heads // num_kv_heads) // 16)
            base = num_decode * num_kv_heads * group_tiles
            part = max(64, self.decode_partition // 64 * 64)
            if part > 128 and base * -(-span // part) < 256:
                part = 128  # few entries: more, smaller partitions so that the compute units fill
            splits = max(1, min(-(-span // part), -(-self.decode_max_groups // base)))
            part = -(-(-(-span // splits)) // 64) * 64
            splits = -(-span // part)
            partial = None
            if splits > 1:
                partial = self._empty((lib.mlr_attention_decode_scratch(entries, num_heads, splits),), torch.float32)
            leave_unmerged = (
                defer_merge and self.tuning.fuse_merge and not num_tiles and num_decode == entries == tokens
                and 1 < splits <= 64 and tokens <= self.FUSED_TOKENS
            )
            self._call(
                "mlr_attention_decode", self._ptr(qkv), stride, self._ptr(key_pages), self._ptr(value_pages),
                self._ptr(block_table), width, self._ptr(ctx.cu_q), self._ptr(ctx.context_lens), self._ptr(out),
                self._ptr(partial), entries, num_heads, num_kv_heads, block_size, num_pages, float(scale),
                int(window or 0), part, splits, int(not leave_unmerged), self._stream(), lib=lib,
            )
            if leave_unmerged:
                return PendingMerge(
                    partial, ctx.cu_q, ctx.context_lens, tokens, num_heads, head_dim, int(window or 0), part, splits, lib
                )
        if num_tiles:
            # long prompts: tiles of 128 queries, whose key and value tiles in LDS serve twice the
            # products, once there are enough of them to keep every compute unit busy all the same
            tiles, wide = plan.query_tiles, 0
            num_wide = int(getattr(plan, "num_wide_query_tiles", 0))
            enough = self.tuning.wide_attention_groups
            behind = int(getattr(plan, "long_prefix", 0))  # 1: thousands of keys before every tile, 2: twice that
            if behind:
                enough = enough * 3 // 4  # heavy tiles everywhere: fewer of them keep the compute units busy
            if (
                num_wide * num_heads >= enough
                and getattr(plan, "wide_query_tiles", None) is not None
                and lib.mlr_attention_wide_tile() == WIDE_QUERY_TILE
            ):
                tiles, num_tiles, wide = plan.wide_query_tiles, num_wide, 1
            self._check(tiles, "query tiles", torch.int32, (num_tiles, 2))
            # few tiles behind long contexts: as many long chains on a few compute units; their keys
            # are cut into runs with a workgroup each, merged by a second kernel
            groups = num_tiles * num_heads
            key_runs = 1
            if behind == 2 and groups < self.tuning.key_run_groups:
                key_runs = min(8, -(-self.tuning.key_run_groups // groups))
            partial = None
            if key_runs > 1:
                partial = self._empty(
                    (lib.mlr_attention_prefill_scratch(num_tiles, num_heads, key_runs, wide),), torch.float32
                )
            self._call(
                "mlr_attention_prefill", self._ptr(qkv), stride, self._ptr(key_pages), self._ptr(value_pages),
                self._ptr(block_table), width, self._ptr(tiles), num_tiles, wide, self._ptr(ctx.cu_q),
                self._ptr(ctx.context_lens), self._ptr(out), num_heads, num_kv_heads, block_size, num_pages,
                float(scale), int(window or 0), key_runs, self._ptr(partial), self._stream(), lib=lib,
            )
        return out

    # ---- sampling -----------------------------------------------------------------------------------
    def sample(
        self,
        logits: torch.Tensor,
        temperature: Optional[torch.Tensor] = None,
        uniform: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """int32 [K]: argmax, or an inverse-CDF draw where temperature > 0."""
        self._check(logits, "logits", torch.float32, (None, None))
        rows, vocab = logits.shape
        if (temperature is None) != (uniform is None):
            raise KernelError("temperature and uniform numbers come together")
        if temperature is not None:
            self._check(temperature, "temperature", torch.float32, (rows,))
            self._check(uniform, "uniform numbers", torch.float32, (rows,))
        out = self._empty((rows,), torch.int32)
        scratch = self._empty((self.lib.mlr_sample_scratch(rows, vocab),), torch.float32)
        self._call(
            "mlr_sample", self._ptr(logits), self._ptr(temperature), self._ptr(uniform), self._ptr(out),
            self._ptr(scratch), rows, vocab, self._stream(),
        )
        return out
