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
from .pending import NormedDelta, PendingLinear, PendingMerge, PendingNorm, PendingScale
from .tuning import KernelTuning

_VP = ctypes.c_void_p
_I = ctypes.c_int
_I64 = ctypes.c_int64
_F = ctypes.c_float

_SIGNATURES = {
    "mlr_version": ([], _I),
    "mlr_embedding": ([_VP, _I, _VP, _VP, _I, _I, _I, _I, _VP], _I),
    "mlr_add_normed": ([_VP, _VP, _I, _I, _VP, _I, _F, _VP, _I, _F, _I, _VP, _I, _I, _I, _VP], _I),
    "mlr_glu_clamped": ([_VP, _I, _VP, _I, _I, _I, _F, _F, _VP], _I),
    "mlr_latent_prepare": (
        [_VP, _I, _VP, _VP, _VP, _VP, _VP, _I, _VP, _I, _F, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _VP,
         _I, _VP],
        _I,
    ),
    "mlr_streams_fill": ([_VP, _VP, _I, _I, _I, _VP], _I),
    "mlr_streams_step": ([_VP, _I, _I, _I, _VP, _I, _VP, _I, _I, _VP, _VP, _VP, _VP, _I, _F, _VP, _VP, _I, _VP], _I),
    "mlr_head_norm_rope_write": (
        [_VP, _I, _VP, _VP, _VP, _VP, _I, _F, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _I, _VP], _I,
    ),
    "mlr_matrix_memory_scan": (
        [_VP, _I, _I, _I, _I, _I, _I, _VP, _I, _VP, _VP, _VP, _VP, _F, _F, _VP, _I, _I, _I, _I, _I, _VP, _VP, _VP], _I,
    ),
    "mlr_matrix_memory_runs": ([_I, _I], _I),
    "mlr_moe_identity": ([_VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_heads_linear": ([_VP, _I64, _I, _VP, _VP, _I64, _I, _VP, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_retention_scan": (
        [_VP, _I, _VP, _I, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _I, _F, _VP, _I, _I, _I, _I, _I, _I, _VP, _I64, _VP], _I,
    ),
    "mlr_retention_scratch": ([_I, _I, _I, _I, _I], _I64),
    "mlr_retention_gate": ([_VP, _VP, _I, _I, _VP, _I, _I, _I, _I, _F, _VP, _I, _F, _I64, _I, _I, _VP], _I),
    "mlr_short_conv": ([_VP, _VP, _I, _VP, _I, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_qk_norm_rope_write": (
        [_VP, _I, _VP, _VP, _I, _F, _VP, _VP, _VP, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _VP],
        _I,
    ),
    "mlr_pool_kv_write": ([_VP, _VP, _VP, _I, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_pooled_share": ([_VP, _I64, _VP, _VP, _VP, _I, _I, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _I, _VP], _I),
    "mlr_scale_heads": ([_VP, _VP, _VP, _I64, _I, _I, _I, _I, _I, _F, _VP], _I),
    "mlr_gla_scan": (
        [_VP, _I, _I, _I, _VP, _VP, _I, _I, _F, _VP, _VP, _I, _VP, _VP, _VP, _VP, _F, _VP, _I, _I, _I, _I, _I, _VP, _VP, _VP], _I,
    ),
    "mlr_gla_runs": ([_I, _I], _I),
    "mlr_rmsnorm": ([_VP, _VP, _VP, _I, _VP, _I, _VP, _I, _I, _I, _F, _VP], _I),
    "mlr_add": ([_VP, _VP, _I, _I64, _VP], _I),
    "mlr_add_slices": ([_VP, _VP, _I, _I64, _VP], _I),
    "mlr_scale_softcap": ([_VP, _F, _F, _I64, _VP], _I),
    "mlr_gather_rows": ([_VP, _VP, _VP, _I, _I64, _I, _I, _VP], _I),
    "mlr_silu_mul": ([_VP, _VP, _I, _I, _I, _VP], _I),
    "mlr_rope_table": ([_VP, _VP, _VP, _VP, _I, _I, _F, _VP], _I),
    "mlr_rope_kv_write": ([_VP, _I, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_qkv_finish": ([_VP, _I, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _VP], _I),
    "mlr_gemm_simple": ([_VP, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _I, _VP, _VP, _F, _F, _VP], _I),
    "mlr_gemm_bf16": ([_VP, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _I, _I, _VP, _I, _F, _VP, _VP, _F, _F, _VP], _I),
    "mlr_moe_route": ([_VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _I, _VP], _I),
    "mlr_moe_tile_rows": ([_I], _I),
    "mlr_moe_max_tiles": ([_I, _I, _I], _I),
    "mlr_moe_align": ([_VP, _I, _I, _I, _I, _VP, _VP, _VP, _VP], _I),
    "mlr_moe_gemm": ([_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _I, _VP], _I),
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
        [_VP, _I64, _VP, _VP, _VP, _I, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _VP, _VP, _VP, _VP,
         _I, _I, _I, _VP, _VP],
        _I,
    ),
    "mlr_sample": ([_VP, _VP, _VP, _VP, _VP, _I, _I, _VP], _I),
    "mlr_sample_scratch": ([_I, _I], _I64),
    "mlr_attention_head_dim": ([], _I),
    "mlr_attention_key_tile": ([], _I),
    "mlr_attention_wide_tile": ([], _I),
    "mlr_attention_decode_scratch": ([_I, _I, _I], _I64),
    "mlr_attention_decode": (
        [_VP, _I64, _VP, _VP, _VP, _I, _VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _F, _I, _I, _I, _I, _I, _VP, _VP, _VP, _VP],
        _I,
    ),
    "mlr_attention_decode_merge": ([_VP, _VP, _VP, _VP, _I, _I, _I, _I, _I, _I, _VP, _VP], _I),
    "mlr_attention_prefill_scratch": ([_I, _I, _I, _I], _I64),
    "mlr_attention_prefill": (
        [_VP, _I64, _VP, _VP, _VP, _I, _VP, _I, _I, _VP, _VP, _VP, _I, _I, _I, _I, _F, _I, _I, _I, _VP, _VP, _VP, _VP, _VP],
        _I,
    ),
}

# what `linear` may do to its sums before it stores them (the entry points' `swiglu` argument)
_EPILOGUES = {None: 0, "swiglu": 1, "relu2": 2, "sigmoid": 3, "gelu_tanh": 4, "clamped_glu": 5}

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
    def embedding(self, table: torch.Tensor, ids: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """table[ids] as float32 (the residual stream), or in `out_dtype` = the engine's dtype."""
        self._check(table, "embedding table", self.dtype, (None, None))
        self._check(ids, "token ids", torch.int32, (None,))
        out_dtype = out_dtype or torch.float32
        if out_dtype not in (torch.float32, self.dtype):
            raise KernelError(f"embedding output must be float32 or {self.dtype}")
        vocab, hidden = table.shape
        out = self._empty((ids.shape[0], hidden), out_dtype)
        self._call(
            "mlr_embedding", self._ptr(table), self.code, self._ptr(ids), self._ptr(out), int(out_dtype == torch.float32),
            ids.shape[0], hidden, vocab, self._stream(),
        )
        return out

    def rmsnorm(
        self, x: torch.Tensor, weight: torch.Tensor, eps: float, delta: Optional[torch.Tensor] = None
    ) -> torch.Tensor:
        """x (float32 residual stream [rows, hidden]) += delta in place, then the RMSNorm of x
        in the engine's dtype.  delta: [rows, hidden] in the engine's dtype, or a float32 stack
        [S, rows, hidden] of partial sums (see `linear`), or None."""
        if isinstance(delta, NormedDelta):  # one kernel: the normed addition and this norm
            return self.add_normed(x, delta.y, delta.weight, delta.eps, next_weight=weight, next_eps=eps)
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

    def add_normed(
        self,
        x: torch.Tensor,
        y,
        weight: torch.Tensor,
        eps: float,
        next_weight: Optional[torch.Tensor] = None,
        next_eps: float = 0.0,
        cast: bool = False,
    ) -> Optional[torch.Tensor]:
        """x (float32 residual stream [rows, hidden], in place) += weight * y * rsqrt(mean(y^2) + eps): a part's
        output that enters the stream through a norm of its own.  y: [rows, hidden] in the engine's dtype or
        float32, a float32 stack [S, rows, hidden] whose sum it is, or a product that has not run.  The same
        kernel then makes what reads the stream next: with `next_weight` the RMSNorm of the new x (weight,
        `next_eps`), with `cast` x itself, both in the engine's dtype; else nothing is returned."""
        self._check(x, "residual stream", torch.float32, (None, None))
        rows, hidden = x.shape
        y = self.settle(y)
        slices = 0
        if y.dim() == 3:
            self._check(y, "partial sums", torch.float32, (None, rows, hidden))
            slices = y.shape[0]
        else:
            self._check(y, "sublayer output", (torch.float32, self.dtype), (rows, hidden))
        self._check(weight, "norm weight", (torch.float32, self.dtype), (hidden,))
        mode = 0
        out = None
        if next_weight is not None:
            self._check(next_weight, "next norm weight", (torch.float32, self.dtype), (hidden,))
            mode = 1
        elif cast:
            mode = 2
        if mode:
            out = self._empty((rows, hidden), self.dtype)
        self._call(
            "mlr_add_normed", self._ptr(x), self._ptr(y), int(y.dtype == torch.float32), slices, self._ptr(weight),
            int(weight.dtype == torch.float32), float(eps), self._ptr(next_weight),
            int(next_weight is not None and next_weight.dtype == torch.float32), float(next_eps), mode, self._ptr(out),
            self.code, rows, hidden, self._stream(),
        )
        return out

    def add_(self, x: torch.Tensor, delta: torch.Tensor) -> None:
        """x (float32) += delta (the engine's dtype, or float32; or a float32 stack [S, ...] of partial sums, or a
        product that has not run), in place."""
        self._check(x, "residual stream", torch.float32)
        delta = self.settle(delta)
        if delta.dim() == x.dim() + 1:  # partial sums: one after the other, in order, in one kernel
            self._check(delta, "partial sums", torch.float32, (None, *x.shape))
            self._call("mlr_add_slices", self._ptr(x), self._ptr(delta), delta.shape[0], x.numel(), self._stream())
            return
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
        if isinstance(x, NormedDelta):  # the norm is per row: it commutes with the choice of rows
            return NormedDelta(self.gather_rows(x.y, rows), x.weight, x.eps)
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
        if isinstance(delta, NormedDelta):
            return None  # the norm kernel that adds a normed delta makes the activations itself
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
        if isinstance(h, NormedDelta):  # what it adds to the stream, float32
            y = self.settle(h.y)
            added = torch.zeros(y.shape[-2:], dtype=torch.float32, device=self.device)
            self.add_normed(added, y, h.weight, h.eps)
            return added
        if isinstance(h, PendingMerge):
            out = self._empty((h.tokens, h.heads * h.head_dim), self.dtype)
            self._call(
                "mlr_attention_decode_merge", self._ptr(h.partial), self._ptr(h.cu_q), self._ptr(h.context_lens),
                self._ptr(out), h.tokens, h.heads, h.window, 0, h.part, h.splits, _VP(None), self._stream(), lib=h.library,
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
        activation: Optional[str] = None,
        multiply: Optional[torch.Tensor] = None,
        clamped_glu: Optional[tuple[float, float]] = None,
        multiply_rows: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """x [M, K] times weight [N, K] transposed, plus bias [N]; F.linear semantics.

        clamped_glu: (limit, alpha).  The rows of `weight` (and the bias with them) are woven as for `swiglu`
        (gate 2j, gate 2j+1, up 2j, up 2j+1) and the result is g * sigmoid(alpha g) * (u + 1), [M, N / 2], with
        g = min(gate, limit) and u = clamp(up, -limit, limit): the pairing's other gating, with a bias.

        activation: "relu2" (max(v, 0)^2) or "sigmoid", applied to the sums (after the bias) in the
        product's epilogue, in 32-bit, before the one rounding to the output's dtype.
        multiply: [M, N] in the engine's dtype; the (activated) sums are multiplied with it element
        by element before they are stored: a gate, sigmoid(x Wg^T) * other, in one kernel.
        multiply_rows: int32 [M]; `multiply` is then a table [rows, N] of which result row i takes row
        multiply_rows[i] (gathered inside the epilogue, e.g. by token id; the indices must lie inside the table).

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
        if activation not in _EPILOGUES or activation in ("swiglu", "clamped_glu"):
            raise KernelError(f"unknown activation {activation!r}")
        glu_limit = glu_alpha = 0.0
        if clamped_glu is not None:
            if swiglu or activation is not None or multiply is not None or partial_sums or for_stream or slices not in (None, 1):
                raise KernelError("the clamped gating goes with whole sums and nothing else")
            glu_limit, glu_alpha = float(clamped_glu[0]), float(clamped_glu[1])
            if not glu_limit > 0:
                raise KernelError("the clamped gating needs a limit > 0")
            x = self.settle(x)  # no fused prologue knows this pairing
        if (activation is not None or multiply is not None) and (swiglu or partial_sums or for_stream or slices not in (None, 1)):
            raise KernelError("an activation or a multiplier goes with whole sums: no SwiGLU pairing, no slices of k")
        epilogue = 1 if swiglu else _EPILOGUES[activation]
        if clamped_glu is not None:
            epilogue = _EPILOGUES["clamped_glu"]
            swiglu = True  # for the shape of the result; the bias check below is the pairing-without-bias one
        if for_stream:
            partial_sums = True
            m, k = x.shape
            if (
                kernel == "auto" and not swiglu and not mfma_kernel and slices is None and out_dtype in (None, self.dtype)
                and not isinstance(x, (PendingNorm, PendingScale)) and self._can_finish_stream(m, weight.shape[0], k)
            ):
                return PendingLinear(x, weight, bias)
        if isinstance(x, (PendingNorm, PendingMerge)):
            fused = None
            if multiply is None:
                fused = self._linear_fused(x, weight, bias, out_dtype, kernel, epilogue, partial_sums, mfma_kernel, slices)
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
        if swiglu and (n % 4 or (bias is not None and clamped_glu is None)):
            raise KernelError("a SwiGLU product needs a multiple of 4 rows and no bias")
        out_dtype = out_dtype or self.dtype
        if out_dtype not in (torch.float32, self.dtype):
            raise KernelError(f"linear output must be float32 or {self.dtype}")
        bias_f32 = int(bias is not None and bias.dtype == torch.float32)
        if multiply_rows is not None:
            if multiply is None:
                raise KernelError("row indices come with a multiplier")
            self._check(multiply_rows, "multiplier rows", torch.int32, (m,))
            self._check(multiply, "multiplier table", self.dtype, (None, n))
        elif multiply is not None:
            self._check(multiply, "multiplier", self.dtype, (m, n))
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
                epilogue, slices, int(mfma_kernel), m, n, k, *scale, self._ptr(multiply), self._ptr(multiply_rows),
                glu_limit, glu_alpha, self._stream(),
            )
            return y
        y = self._empty((m, n // 2 if swiglu else n), out_dtype)
        self._call(
            "mlr_gemm_simple", self._ptr(x), self._ptr(weight), self._ptr(bias), bias_f32, self._ptr(y),
            int(out_dtype == torch.float32), epilogue, self.code, m, n, k, self._ptr(multiply),
            self._ptr(multiply_rows), glu_limit, glu_alpha, self._stream(),
        )
        return y

    def _linear_fused(self, x, weight, bias, out_dtype, kernel, epilogue, partial_sums, mfma_kernel, slices):
        """`linear` on a pending activation in one kernel, or None when that cannot be.  `epilogue`:
        the code of what happens to the sums (0 nothing, 1 the SwiGLU pairing, 2 and 3 activations)."""
        swiglu = epilogue == 1
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
                int(out_dtype == torch.float32), epilogue, 0, m, n, k, self._stream(),
            )
            x.residual = residual
            return y
        if epilogue or not self.tuning.fuse_merge or n * k * 2 > min(self.tuning.fuse_weight_bytes, (1 << 32) - 1):
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
    def rope_table(
        self, positions: torch.Tensor, inv_freq: torch.Tensor, amplitude: float = 1.0
    ) -> tuple[torch.Tensor, torch.Tensor]:
        self._check(positions, "positions", torch.int32, (None,))
        self._check(inv_freq, "inverse frequencies", torch.float64, (None,))
        tokens, half = positions.shape[0], inv_freq.shape[0]
        cos = self._empty((tokens, half), torch.float32)
        sin = self._empty((tokens, half), torch.float32)
        self._call(
            "mlr_rope_table", self._ptr(positions), self._ptr(inv_freq), self._ptr(cos), self._ptr(sin),
            tokens, half, float(amplitude), self._stream(),
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
        chunk: Optional[int] = None,
        sinks: Optional[torch.Tensor] = None,
        pooled: Optional[tuple] = None,
        score_bias: Optional[torch.Tensor] = None,
    ):
        """Causal attention of the step's tokens over their requests' pages.

        score_bias: float32 [num_heads]; no softmax then: a visible key weighs sigmoid(score * scale +
        score_bias[head]) whatever the other keys are, and the weights are not normalised.

        pooled: (key pages, value pages, block table, pool) of a second set of pages that holds ONE key and
        value for every run of `pool` positions (see `pool_kv_write`); with a window, a query at position p
        then also sees the entries of the runs that end at or before p - window, in the same softmax.

        sinks: float32 [num_heads]; the softmax's denominator of head h then also holds exp(sinks[h]), a
        term with no key and no value (not scaled).

        window / chunk: which of the keys 0..p a query at position p sees: with a window the last
        `window` of them, with a chunked mask those from floor(p / chunk) * chunk on; at most one of
        the two.

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
        if chunk is not None and (chunk <= 0 or window):
            raise KernelError("a chunked mask has a size > 0 and no window beside it")
        chunk = int(chunk or 0)
        if sinks is not None:
            self._check(sinks, "sinks", torch.float32, (num_heads,))
        if score_bias is not None:
            self._check(score_bias, "score bias", torch.float32, (num_heads,))
            if sinks is not None or pooled is not None:
                raise KernelError("keys weighed one by one have no sink and no pooled entries")
        out = self._empty((tokens, num_heads * head_dim), self.dtype)
        width = block_table.shape[1]
        pooled_keys = pooled_values = pooled_table = None
        pooled_width = pooled_pages = pool = 0
        if pooled is not None:
            pooled_keys, pooled_values, pooled_table, pool = pooled
            pool = int(pool)
            if pool <= 0 or not window:
                raise KernelError("pooled entries have a run length > 0 and come with a window")
            pooled_pages = self._check_pages(pooled_keys, pooled_values, num_kv_heads, head_dim, block_size)
            self._check(pooled_table, "pooled block table", torch.int32, (entries, None))
            pooled_width = pooled_table.shape[1]
            if pooled_width * block_size * pool < ctx.max_context_len - int(window) - pool + 1:
                raise KernelError("the pooled block table is narrower than the runs before the longest context's window")
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
                num_pages, float(scale), int(window or 0), chunk, self._ptr(sinks), self._ptr(pooled_keys),
                self._ptr(pooled_values), self._ptr(pooled_table), pooled_width, pooled_pages, pool,
                self._ptr(score_bias), self._stream(),
            )
            return out
        self._check(ctx.cu_q, "cu_q", torch.int32, (entries + 1,))
        self._check(ctx.context_lens, "context lengths", torch.int32, (entries,))
        share = None
        if pooled is not None:
            # the pooled entries' share of every token's softmax (few keys: a plain kernel); the matrix-core
            # kernels take the window's tokens and their merge takes this share in, before the sink
            share = self._empty((tokens, num_heads, head_dim + 2), torch.float32)
            self._call(
                "mlr_pooled_share", self._ptr(qkv), stride, self._ptr(pooled_keys), self._ptr(pooled_values),
                self._ptr(pooled_table), pooled_width, pooled_pages, self._ptr(ctx.token_entry), self._ptr(ctx.positions),
                self._ptr(share), tokens, num_heads, num_kv_heads, head_dim, block_size, float(scale), int(window),
                pool, self._stream(),
            )
        if num_decode:
            span = int(plan.max_decode_context)
            if window:
                span = min(span, int(window) + 15)
            if chunk:
                span = min(span, chunk + 15)  # a partition starts at a multiple of 16 at or before the first key
            group_tiles = -(-(num_heads // num_kv_heads) // 16)
            base = num_decode * num_kv_heads * group_tiles
            part = max(64, self.decode_partition // 64 * 64)
            if part > 128 and base * -(-span // part) < 256:
                part = 128  # few entries: more, smaller partitions so that the compute units fill
            splits = max(1, min(-(-span // part), -(-self.decode_max_groups // base)))
            part = -(-(-(-span // splits)) // 64) * 64
            splits = -(-span // part)
            partial = None
            if splits > 1 or share is not None:
                partial = self._empty((lib.mlr_attention_decode_scratch(entries, num_heads, splits),), torch.float32)
            leave_unmerged = (
                defer_merge and self.tuning.fuse_merge and not num_tiles and num_decode == entries == tokens
                and 1 < splits <= 64 and tokens <= self.FUSED_TOKENS and not chunk and sinks is None and share is None
                and score_bias is None
            )
            self._call(
                "mlr_attention_decode", self._ptr(qkv), stride, self._ptr(key_pages), self._ptr(value_pages),
                self._ptr(block_table), width, self._ptr(ctx.cu_q), self._ptr(ctx.context_lens), self._ptr(out),
                self._ptr(partial), entries, num_heads, num_kv_heads, block_size, num_pages, float(scale),
                int(window or 0), chunk, part, splits, int(not leave_unmerged), self._ptr(sinks), self._ptr(share),
                self._ptr(score_bias), self._stream(), lib=lib,
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
            if key_runs > 1 or share is not None:
                partial = self._empty(
                    (lib.mlr_attention_prefill_scratch(num_tiles, num_heads, key_runs, wide),), torch.float32
                )
            self._call(
                "mlr_attention_prefill", self._ptr(qkv), stride, self._ptr(key_pages), self._ptr(value_pages),
                self._ptr(block_table), width, self._ptr(tiles), num_tiles, wide, self._ptr(ctx.cu_q),
                self._ptr(ctx.context_lens), self._ptr(out), num_heads, num_kv_heads, block_size, num_pages,
                float(scale), int(window or 0), chunk, key_runs, self._ptr(partial), self._ptr(sinks), self._ptr(share),
                self._ptr(score_bias), self._stream(), lib=lib,
            )
        return out

    # ---- other mixers and feed-forwards ----------------------------------------------------------------
    def glu_clamped(self, sums: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
        """sums [rows, 2 * inter] (gate sums, then up sums; float32 or the engine's dtype) ->
        g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit), [rows, inter]."""
        self._check(sums, "gate and up sums", (torch.float32, self.dtype), (None, None))
        rows, width = sums.shape
        if width % 2:
            raise KernelError("gate and up sums must have an even width")
        out = self._empty((rows, width // 2), self.dtype)
        self._call(
            "mlr_glu_clamped", self._ptr(sums), int(sums.dtype == torch.float32), self._ptr(out), self.code, rows,
            width // 2, float(limit), float(alpha), self._stream(),
        )
        return out

    def latent_prepare(
        self,
        projected: torch.Tensor,
        *,
        heads: int,
        head_dim: int,
        rot_dim: int,
        kv_rank: int,
        own_cache: bool,
        gated: bool,
        norm_weight: Optional[torch.Tensor],
        eps: float,
        rotation: Optional[tuple[torch.Tensor, torch.Tensor, int]],
        slot_mapping: torch.Tensor,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        block_size: int,
        kernel_dim: int,
        queries: Optional[torch.Tensor] = None,
    ):
        """From a latent-attention layer's input sums (float32 [T, heads * (head_dim + rot_dim) (+ kv_rank +
        rot_dim) (+ heads)]: queries, own latent and shared key part, gate logits) to what its kernels take:
        (unrotated query parts [T, heads * head_dim]; latent queries [T, heads * kernel_dim] whose columns
        kv_rank .. kv_rank + rot_dim hold the rotated query parts and whose first kv_rank are left to
        `heads_linear`; gates sigmoid(logit), float32 [T, heads], or None).  With `own_cache` the normed latent
        and the rotated key part go into the pages: key rows [latent ; key part ; 0], values [latent ; 0].
        queries: float32 [T, heads * (head_dim + rot_dim)] when the query sums come from a product of their own;
        `projected` then starts with the latent."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        if queries is not None:
            self._check(queries, "query sums", torch.float32, (tokens, None))
        cos = sin = None
        rotary = 0
        if rotation is not None:
            cos, sin, rotary = rotation
            self._check(cos, "rotary cos", torch.float32, (tokens, rotary // 2))
            self._check(sin, "rotary sin", torch.float32, (tokens, rotary // 2))
        num_pages = 0
        if own_cache:
            num_pages = self._check_pages(key_pages, value_pages, 1, kernel_dim, block_size)
            self._check(slot_mapping, "slot mapping", torch.int32, (tokens,))
            self._check(norm_weight, "latent norm weight", (torch.float32, self.dtype), (kv_rank,))
        q_plain = self._empty((tokens, heads * head_dim), self.dtype)
        q_latent = self._empty((tokens, heads * kernel_dim), self.dtype)
        gate = self._empty((tokens, heads), torch.float32) if gated else None
        self._call(
            "mlr_latent_prepare", self._ptr(projected), width, self._ptr(q_plain), self._ptr(q_latent), self._ptr(gate),
            self._ptr(cos), self._ptr(sin), int(rotary), self._ptr(norm_weight if own_cache else None),
            int(own_cache and norm_weight.dtype == torch.float32), float(eps),
            self._ptr(slot_mapping if own_cache else None), self._ptr(key_pages if own_cache else None),
            self._ptr(value_pages if own_cache else None), self.code, tokens, heads, head_dim, rot_dim, kv_rank,
            kernel_dim, block_size, num_pages, int(own_cache), int(gated), self._ptr(queries),
            int(queries.shape[1]) if queries is not None else 0, self._stream(),
        )
        return q_plain, q_latent, gate

    def heads_linear(
        self,
        x: torch.Tensor,
        weight: torch.Tensor,
        *,
        in_stride: int,
        out: Optional[torch.Tensor] = None,
        out_stride: Optional[int] = None,
        row_scale: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """One small matrix per head: y[t, h, :] = weight[h] x[t, h, :k] for weight [heads, n, k] and x [T, heads
        * in_stride] (head h's input starts at column h * in_stride), times row_scale[t, h] (float32) if given.
        Returns [T, heads * n], or writes head h's result to columns h * out_stride .. + n of `out`."""
        self._check(weight, "per-head weights", self.dtype, (None, None, None))
        heads, n, k = weight.shape
        self._check(x, "per-head input", self.dtype, (None, None))
        tokens = x.shape[0]
        if in_stride < k or x.shape[1] < heads * in_stride:
            raise KernelError("the input rows do not hold every head's values")
        if out is None:
            out_stride = n
            out = self._empty((tokens, heads * n), self.dtype)
        else:
            self._check(out, "per-head output", self.dtype, (tokens, None))
            if out_stride is None or out_stride < n or out.shape[1] < heads * out_stride:
                raise KernelError("the output rows do not hold every head's values")
        if row_scale is not None:
            self._check(row_scale, "row scale", torch.float32, (tokens, heads))
        self._call(
            "mlr_heads_linear", self._ptr(x), x.shape[1], int(in_stride), self._ptr(weight), self._ptr(out), out.shape[1],
            int(out_stride), self._ptr(row_scale), self.code, tokens, heads, n, k, self._stream(),
        )
        return out

    RETENTION_CHUNK_FROM = 4  # mean tokens an entry from which retention runs in chunks

    def retention_scan(
        self,
        projected: torch.Tensor,
        state: torch.Tensor,
        read_rows: torch.Tensor,
        write_rows: torch.Tensor,
        ctx: Any,
        *,
        heads: int,
        head_dim: int,
        value_dim: int,
        decay: torch.Tensor,
        key_scale: float,
        rotation: Optional[tuple[torch.Tensor, torch.Tensor, int]],
        chunked: Optional[bool] = None,
    ) -> torch.Tensor:
        """Retention of the step's tokens, every entry's in order: S = decay_h S + k v^T, o = S^T q per head,
        from the state in row read_rows[entry] of `state` [rows, heads, head_dim, value_dim] (zeros where the
        entry starts its request) to row write_rows[entry].  `projected` (float32 [T, >= 2 * heads * head_dim +
        heads * value_dim]) holds q, k and v; q and k are rotated and k scaled by `key_scale` here, in 32-bit
        (the chunked way does that in place: `projected` is the caller's scratch).
        Returns o, float32 [T, heads * value_dim].  Steps of single tokens (and of a few) run the recurrence
        token by token with the state in registers; steps with longer entries run it 64 tokens at a time
        on the matrix cores, in true 32-bit both ways (`chunked` forces one of them)."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        entries = ctx.num_entries
        if chunked is None:
            chunked = tokens > self.RETENTION_CHUNK_FROM * entries  # more than a few tokens an entry
        self._check(state, "retention state", torch.float32, (None, heads, head_dim, value_dim))
        self._check(read_rows, "state rows to read", torch.int32, (entries,))
        self._check(write_rows, "state rows to write", torch.int32, (entries,))
        self._check(ctx.cu_q, "cu_q", torch.int32, (entries + 1,))
        self._check(ctx.q_starts, "q_starts", torch.int32, (entries,))
        self._check(decay, "decays", torch.float32, (heads,))
        cos = sin = None
        rotary = 0
        if rotation is not None:
            cos, sin, rotary = rotation
            self._check(cos, "rotary cos", torch.float32, (tokens, rotary // 2))
            self._check(sin, "rotary sin", torch.float32, (tokens, rotary // 2))
        out = self._empty((tokens, heads * value_dim), torch.float32)
        scratch, floats = None, 0
        if chunked:
            floats = int(self.lib.mlr_retention_scratch(tokens, entries, heads, head_dim, value_dim))
            if floats:
                scratch = self._empty((floats,), torch.float32)
        self._call(
            "mlr_retention_scan", self._ptr(projected), width, self._ptr(state), state.shape[0], self._ptr(read_rows),
            self._ptr(write_rows), self._ptr(ctx.cu_q), self._ptr(ctx.q_starts), self._ptr(decay), self._ptr(cos),
            self._ptr(sin), int(rotary), float(key_scale), self._ptr(out), entries, heads, head_dim, value_dim,
            int(bool(chunked)), tokens, self._ptr(scratch), floats, self._stream(),
        )
        return out

    def retention_gate(
        self,
        retained: torch.Tensor,
        projected: torch.Tensor,
        *,
        heads: int,
        value_dim: int,
        gate_offset: int,
        eps: float,
        norm_weight: Optional[torch.Tensor] = None,
        scale: float = 1.0,
        out: Optional[torch.Tensor] = None,
        column: int = 0,
        gate: str = "silu",
    ) -> torch.Tensor:
        """Every head's retained[t, h, :] divided by its root mean square (eps inside the root), times
        `norm_weight` [value_dim] (one weight for all heads) or [heads * value_dim] (None: none), times `gate`
        ("silu" or "sigmoid") of the gate sums in columns
        gate_offset .. of `projected`, times `scale`; [T, heads * value_dim] in the engine's dtype, or written
        into columns column .. of the wider `out` [T, K]."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        self._check(retained, "retained", torch.float32, (tokens, heads * value_dim))
        if gate_offset < 0 or gate_offset + heads * value_dim > width:
            raise KernelError("the projected rows do not hold the gate")
        if gate not in ("silu", "sigmoid"):
            raise KernelError("the gate is 'silu' or 'sigmoid'")
        per_head = norm_weight is not None and heads > 1 and norm_weight.numel() == heads * value_dim
        if norm_weight is not None:
            self._check(norm_weight, "head norm weight", (torch.float32, self.dtype), (heads * value_dim if per_head else value_dim,))
        out, view, row = self._columns(out, column, tokens, heads * value_dim)
        self._call(
            "mlr_retention_gate", self._ptr(retained), self._ptr(projected), width, int(gate_offset), view,
            self.code, tokens, heads, value_dim, float(eps), self._ptr(norm_weight),
            int(norm_weight is not None and norm_weight.dtype == torch.float32), float(scale), row, int(per_head),
            int(gate == "sigmoid"), self._stream(),
        )
        return out

    def _columns(self, out: Optional[torch.Tensor], column: int, tokens: int, width: int):
        """Where a kernel writes [tokens, width] activations: a tensor of its own, or columns column ..
        column + width of a wider `out`; returns (tensor, pointer to the first element, row length)."""
        if out is None:
            out = self._empty((tokens, width), self.dtype)
            return out, self._ptr(out), width
        self._check(out, "activations of several parts", self.dtype, (tokens, None))
        row = out.shape[1]
        if column < 0 or column + width > row:
            raise KernelError("the columns lie outside the rows they are written into")
        return out, _VP(out.data_ptr() + column * out.element_size()), row

    # ---- parts that run side by side ---------------------------------------------------------------------
    def short_conv(
        self,
        h: torch.Tensor,
        weight: torch.Tensor,
        state: Optional[torch.Tensor],
        read_rows: Optional[torch.Tensor],
        write_rows: Optional[torch.Tensor],
        ctx: Any,
        *,
        add_input: bool = True,
    ) -> torch.Tensor:
        """h [T, W] (+ when `add_input`) its causal convolution over time, per channel and entry: out_t = sum_j
        weight[:, j] * h_(t - taps + 1 + j), weight [W, taps].  The taps - 1 inputs before a step's first token
        come from row read_rows[entry] of `state` [rows, taps - 1, W] float32 (zeros where the entry starts its
        request); the newest taps - 1 inputs are left in row write_rows[entry]."""
        self._check(h, "convolution input", self.dtype, (None, None))
        tokens, width = h.shape
        self._check(weight, "convolution taps", (torch.float32, self.dtype), (width, None))
        taps = weight.shape[1]
        entries = ctx.num_entries
        rows = 0
        if taps > 1:
            self._check(state, "carried inputs", torch.float32, (None, taps - 1, width))
            rows = state.shape[0]
        else:
            state = None
            read_rows, write_rows = ctx.q_starts, ctx.q_starts  # never read
        self._check(read_rows, "state rows to read", torch.int32, (entries,))
        self._check(write_rows, "state rows to write", torch.int32, (entries,))
        self._check(ctx.token_entry, "token entries", torch.int32, (tokens,))
        self._check(ctx.cu_q, "cu_q", torch.int32, (entries + 1,))
        self._check(ctx.q_starts, "q_starts", torch.int32, (entries,))
        out = self._empty((tokens, width), self.dtype)
        self._call(
            "mlr_short_conv", self._ptr(h), self._ptr(weight), int(weight.dtype == torch.float32), self._ptr(state), rows,
            self._ptr(read_rows), self._ptr(write_rows), self._ptr(ctx.token_entry), self._ptr(ctx.cu_q),
            self._ptr(ctx.q_starts), self._ptr(out), self.code, tokens, width, taps, int(bool(add_input)), self._stream(),
        )
        return out

    def qk_norm_rope_write(
        self,
        projected: torch.Tensor,
        q_norm: Optional[torch.Tensor],
        k_norm: Optional[torch.Tensor],
        eps: float,
        head_scale: Optional[torch.Tensor],
        rotation: Optional[tuple[torch.Tensor, torch.Tensor, int]],
        slot_mapping: torch.Tensor,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        *,
        num_heads: int,
        num_kv_heads: int,
        dim: int,
        value_dim: int,
        head_dim: int,
        block_size: int,
        gated: bool = False,
        projected_column: int = 0,
    ) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        """From the float32 sums `projected` [T, q | k | v | gate logits] (from column `projected_column` on, when
        the rows also hold other parts' sums): q and k each divided by the root mean
        square of their WHOLE projection and multiplied by q_norm [heads * dim] / k_norm [kv_heads * dim] (None:
        no norm), rotated (the first r dims of a head in two halves), q times head_scale[head] (float32 [heads]
        or None); k and v stored in the pages at `slot_mapping` (negative: not stored).  All in 32-bit, one
        rounding.  Returns q [T, heads * head_dim] in the engine's dtype (heads padded with zeros to the pages'
        head size) and, if `gated`, sigmoid(gate logits) float32 [T, heads]."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        if projected_column < 0 or width - projected_column < num_heads * dim + num_kv_heads * (dim + value_dim) + (num_heads if gated else 0):
            raise KernelError("the projected rows are too narrow")
        weight_f32 = 0
        for w, n, name in ((q_norm, num_heads * dim, "query norm weight"), (k_norm, num_kv_heads * dim, "key norm weight")):
            if w is not None:
                self._check(w, name, (torch.float32, self.dtype), (n,))
                weight_f32 = int(w.dtype == torch.float32)
        if q_norm is not None and k_norm is not None and q_norm.dtype != k_norm.dtype:
            raise KernelError("the two norm weights must have one dtype")
        if head_scale is not None:
            self._check(head_scale, "head scale", torch.float32, (num_heads,))
        cos = sin = None
        rotary = 0
        if rotation is not None:
            cos, sin, rotary = rotation
            if rotary <= 0 or rotary % 2 or rotary > dim:
                raise KernelError("rotary_dim must be even and within dim")
            self._check(cos, "rotary cos", torch.float32, (tokens, rotary // 2))
            self._check(sin, "rotary sin", torch.float32, (tokens, rotary // 2))
        num_pages = self._check_pages(key_pages, value_pages, num_kv_heads, head_dim, block_size)
        self._check(slot_mapping, "slot mapping", torch.int32, (tokens,))
        q = self._empty((tokens, num_heads * head_dim), self.dtype)
        gate = self._empty((tokens, num_heads), torch.float32) if gated else None
        self._call(
            "mlr_qk_norm_rope_write", _VP(projected.data_ptr() + 4 * int(projected_column)), width, self._ptr(q_norm), self._ptr(k_norm), weight_f32,
            float(eps), self._ptr(head_scale), self._ptr(cos), self._ptr(sin), int(rotary), self._ptr(slot_mapping),
            self._ptr(key_pages), self._ptr(value_pages), self._ptr(q), self._ptr(gate), self.code, tokens, num_heads,
            num_kv_heads, dim, value_dim, head_dim, block_size, num_pages, int(bool(gated)), self._stream(),
        )
        return q, gate

    def pool_kv_write(
        self,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        block_table: torch.Tensor,
        pooled_slots: torch.Tensor,
        pooled_keys: torch.Tensor,
        pooled_values: torch.Tensor,
        ctx: Any,
        *,
        num_kv_heads: int,
        head_dim: int,
        block_size: int,
        pool: int,
    ) -> None:
        """Every token of the step that completes a run of `pool` positions (pooled_slots[t] >= 0) stores the means
        of the run's keys and of its values, as the token pages hold them, at that slot of the pooled pages."""
        num_pages = self._check_pages(key_pages, value_pages, num_kv_heads, head_dim, block_size)
        pooled_pages = self._check_pages(pooled_keys, pooled_values, num_kv_heads, head_dim, block_size)
        tokens = pooled_slots.shape[0]
        self._check(pooled_slots, "pooled slot mapping", torch.int32, (tokens,))
        self._check(block_table, "block table", torch.int32, (ctx.num_entries, None))
        self._check(ctx.token_entry, "token entries", torch.int32, (tokens,))
        self._check(ctx.positions, "positions", torch.int32, (tokens,))
        if pool <= 0:
            raise KernelError("a run has at least one position")
        self._call(
            "mlr_pool_kv_write", self._ptr(key_pages), self._ptr(value_pages), self._ptr(block_table), block_table.shape[1],
            num_pages, self._ptr(ctx.token_entry), self._ptr(ctx.positions), self._ptr(pooled_slots), self._ptr(pooled_keys),
            self._ptr(pooled_values), pooled_pages, self.code, tokens, num_kv_heads, head_dim, block_size, int(pool),
            self._stream(),
        )

    def scale_heads(
        self,
        attended: torch.Tensor,
        gate: Optional[torch.Tensor],
        *,
        heads: int,
        head_dim: int,
        out_dim: int,
        scale: float = 1.0,
        out: Optional[torch.Tensor] = None,
        column: int = 0,
    ) -> torch.Tensor:
        """The first `out_dim` dims of every head of attended [T, heads * head_dim], times gate[t, head] (float32 [T,
        heads] or None) and `scale`: [T, heads * out_dim], or columns column .. of the wider `out`."""
        self._check(attended, "attended heads", self.dtype, (None, heads * head_dim))
        tokens = attended.shape[0]
        if gate is not None:
            self._check(gate, "head gates", torch.float32, (tokens, heads))
        if not 0 < out_dim <= head_dim:
            raise KernelError("out_dim must lie within head_dim")
        out, view, row = self._columns(out, column, tokens, heads * out_dim)
        self._call(
            "mlr_scale_heads", self._ptr(attended), self._ptr(gate), view, row, self.code, tokens, heads, head_dim,
            out_dim, float(scale), self._stream(),
        )
        return out

    def gla_scan(
        self,
        projected: torch.Tensor,
        state: torch.Tensor,
        read_rows: torch.Tensor,
        write_rows: torch.Tensor,
        ctx: Any,
        *,
        heads: int,
        head_dim: int,
        value_dim: int,
        decay_weight: torch.Tensor,
        decay_bias: Optional[torch.Tensor],
        low_offset: int,
        tau: float,
        q_scale: float,
        by_runs: Optional[bool] = None,
        projected_column: int = 0,
    ) -> torch.Tensor:
        """Linear attention with a decay per key channel and token, every entry's tokens in order: S = diag(a_t) S +
        k_t v_t^T, o_t = S^T (q_t * q_scale) per head, a_t = sigmoid(W2 low_t + bias)^(1 / tau) with low_t the columns
        low_offset .. low_offset + rank of `projected` (float32 [T, q | k | v | ...]) and W2 = decay_weight [heads *
        head_dim, rank].  State rows as for `retention_scan`.  Everything in 32-bit.  Returns o, float32 [T, heads *
        value_dim].  `by_runs`: entries are cut into runs of 64 tokens that are walked in parallel, twice, with a carry
        of the state between the walks (None: when the step has 128 tokens more than entries); else a wavefront walks
        a whole entry token by token.  The two differ by the order of 32-bit sums only."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        entries = ctx.num_entries
        self._check(decay_weight, "decay weight", (torch.float32, self.dtype), (heads * head_dim, None))
        rank = decay_weight.shape[1]
        if decay_bias is not None:
            self._check(decay_bias, "decay bias", (torch.float32, self.dtype), (heads * head_dim,))
        own = width - int(projected_column)  # the rows may hold other parts' sums before this part's
        if projected_column < 0 or low_offset < 0 or low_offset + rank > own or 2 * heads * head_dim + heads * value_dim > own:
            raise KernelError("the projected rows do not hold q, k, v and the decay's inputs")
        self._check(state, "recurrent state", torch.float32, (None, heads, head_dim, value_dim))
        self._check(read_rows, "state rows to read", torch.int32, (entries,))
        self._check(write_rows, "state rows to write", torch.int32, (entries,))
        self._check(ctx.cu_q, "cu_q", torch.int32, (entries + 1,))
        self._check(ctx.q_starts, "q_starts", torch.int32, (entries,))
        out = self._empty((tokens, heads * value_dim), torch.float32)
        if by_runs is None:
            by_runs = tokens - entries >= 128
        decay = runs = run_decay = None
        if by_runs:
            decay = self._empty((tokens, heads * head_dim), torch.float32)
            most = int(self.lib.mlr_gla_runs(tokens, entries))
            runs = self._empty((most, heads, head_dim, value_dim), torch.float32)
            run_decay = self._empty((most, heads, head_dim), torch.float32)
        self._call(
            "mlr_gla_scan", _VP(projected.data_ptr() + 4 * int(projected_column)), width, int(low_offset), rank, self._ptr(decay_weight),
            self._ptr(decay_bias), int(decay_weight.dtype == torch.float32),
            int(decay_bias is not None and decay_bias.dtype == torch.float32), float(tau), self._ptr(decay),
            self._ptr(state), state.shape[0], self._ptr(read_rows), self._ptr(write_rows), self._ptr(ctx.cu_q),
            self._ptr(ctx.q_starts), float(q_scale), self._ptr(out), entries, heads, head_dim, value_dim, tokens,
            self._ptr(runs), self._ptr(run_decay), self._stream(),
        )
        return out

    # ---- several residual streams ---------------------------------------------------------------------------
    def streams_fill(self, x: torch.Tensor, streams: int) -> torch.Tensor:
        """`streams` copies of x (float32 [T, hidden]) as one tensor [streams, T, hidden]."""
        self._check(x, "residual stream", torch.float32, (None, None))
        tokens, hidden = x.shape
        out = self._empty((int(streams), tokens, hidden), torch.float32)
        self._call("mlr_streams_fill", self._ptr(x), self._ptr(out), tokens, hidden, int(streams), self._stream())
        return out

    def streams_step(
        self,
        x: torch.Tensor,
        *,
        update=None,
        read_weights: Optional[torch.Tensor] = None,
        norm_weight: Optional[torch.Tensor] = None,
        eps: float = 0.0,
        rows: Optional[torch.Tensor] = None,
        want_sum: bool = False,
    ):
        """One kernel for what happens to residual streams x (float32 [S, T, hidden]) between two sublayers.
        update = (y, mix [S, S], write [S]): all streams at once from the old ones, x_t = sum_s mix[s, t] x_s +
        write[t] * y, with y a sublayer's output ([T, hidden] in the engine's dtype or float32, a float32 stack
        whose sum it is, or a product that has not run).  Then u = sum_s read_weights[s] x_s (None: the plain
        sum) and, with `norm_weight`, h = u * rsqrt(mean(u^2) + eps) * norm_weight in the engine's dtype.
        rows: int32 [K] tokens to do this for; the streams themselves are then left as they are.
        Returns (h or None, u as float32 if `want_sum` else None)."""
        self._check(x, "residual streams", torch.float32, (None, None, None))
        streams, tokens, hidden = x.shape
        y = mix = write = None
        slices = 0
        if update is not None:
            y, mix, write = update
            y = self.settle(y)
            if y.dim() == 3:
                self._check(y, "partial sums", torch.float32, (None, tokens, hidden))
                slices = y.shape[0]
            else:
                self._check(y, "sublayer output", (torch.float32, self.dtype), (tokens, hidden))
            self._check(mix, "stream mixing matrix", torch.float32, (streams, streams))
            self._check(write, "stream output weights", torch.float32, (streams,))
        if read_weights is not None:
            self._check(read_weights, "stream input weights", torch.float32, (streams,))
        out_rows = tokens
        if rows is not None:
            self._check(rows, "row indices", torch.int32, (None,))
            out_rows = rows.shape[0]
        h = total = None
        if norm_weight is not None:
            self._check(norm_weight, "norm weight", (torch.float32, self.dtype), (hidden,))
            h = self._empty((out_rows, hidden), self.dtype)
        if want_sum:
            total = self._empty((out_rows, hidden), torch.float32)
        self._call(
            "mlr_streams_step", self._ptr(x), streams, tokens, hidden, self._ptr(rows), out_rows, self._ptr(y),
            int(y is not None and y.dtype == torch.float32), slices, self._ptr(mix), self._ptr(write),
            self._ptr(read_weights), self._ptr(norm_weight),
            int(norm_weight is not None and norm_weight.dtype == torch.float32), float(eps), self._ptr(h),
            self._ptr(total), self.code, self._stream(),
        )
        return h, total

    # ---- attention whose heads are normed one by one ---------------------------------------------------------
    def head_norm_rope_write(
        self,
        projected: torch.Tensor,
        *,
        heads: int,
        kv_heads: int,
        head_dim: int,
        value_dim: int,
        kernel_dim: int,
        eps: float,
        rotation: Optional[tuple[torch.Tensor, torch.Tensor, int]],
        slot_mapping: torch.Tensor,
        key_pages: torch.Tensor,
        value_pages: torch.Tensor,
        block_size: int,
        gated: bool = False,
        keep_values: bool = False,
        first_values: Optional[torch.Tensor] = None,
        mix_weight: Optional[torch.Tensor] = None,
    ):
        """From the float32 sums of an attention layer's input product ([T, heads * head_dim + kv_heads * head_dim +
        kv_heads * value_dim (+ heads)]: queries, keys, values, gate logits) to what the attention kernels take.
        Queries and keys are rotated (the first r dims of a head in two halves) and then every head is divided
        by its root mean square over head_dim; every value head by its own over value_dim (eps inside the roots,
        no weights).  With `first_values` (float32 [T, kv_heads * value_dim]) and `mix_weight` (float32 [1]) the
        values become (1 - w) v + w first_values.  Queries go to [T, heads * kernel_dim], keys and values into
        the pages at `slot_mapping`, all zero beyond their own widths.  Returns (queries, sigmoid of the gate
        logits as float32 [T, heads] or None, the normed values before mixing as float32 if `keep_values`)."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        cos = sin = None
        rotary = 0
        if rotation is not None:
            cos, sin, rotary = rotation
            self._check(cos, "rotary cos", torch.float32, (tokens, rotary // 2))
            self._check(sin, "rotary sin", torch.float32, (tokens, rotary // 2))
        num_pages = self._check_pages(key_pages, value_pages, kv_heads, kernel_dim, block_size)
        self._check(slot_mapping, "slot mapping", torch.int32, (tokens,))
        if width < (heads + kv_heads) * head_dim + kv_heads * value_dim + (heads if gated else 0):
            raise KernelError("the projected rows are too narrow")
        if first_values is not None:
            self._check(first_values, "first values", torch.float32, (tokens, kv_heads * value_dim))
            self._check(mix_weight, "value mixing weight", torch.float32, (1,))
        q = self._empty((tokens, heads * kernel_dim), self.dtype)
        gate = self._empty((tokens, heads), torch.float32) if gated else None
        kept = self._empty((tokens, kv_heads * value_dim), torch.float32) if keep_values else None
        self._call(
            "mlr_head_norm_rope_write", self._ptr(projected), width, self._ptr(q), self._ptr(gate), self._ptr(cos),
            self._ptr(sin), int(rotary), float(eps), self._ptr(slot_mapping), self._ptr(key_pages),
            self._ptr(value_pages), self._ptr(kept), self._ptr(first_values),
            self._ptr(mix_weight if first_values is not None else None), self.code, tokens, heads, kv_heads, head_dim,
            value_dim, kernel_dim, block_size, num_pages, self._stream(),
        )
        return q, gate, kept

    # ---- matrix memory with exponential gates -----------------------------------------------------------------
    MEMORY_RUNS_FROM = 128  # tokens more than entries from which the memory's scan walks runs instead of whole entries

    def matrix_memory_scan(
        self,
        projected: torch.Tensor,
        state: torch.Tensor,
        read_rows: torch.Tensor,
        write_rows: torch.Tensor,
        ctx: Any,
        *,
        heads: int,
        head_dim: int,
        value_dim: int,
        offsets: Sequence[int],
        cap: float,
        q_scale: float,
        in_runs: Optional[bool] = None,
    ) -> torch.Tensor:
        """The step's tokens, every entry's in order, through a matrix memory per head: with i = cap tanh(a / cap), f
        = logsigmoid(cap tanh(b / cap)) (a, b the gates' sums), m' = max(f + m, i), C' = exp(f + m - m') C + exp(i
        - m') k v^T, n' likewise with k alone, o = C'^T q / (max(|n' . q|, exp(-m')) + 1e-6).  `projected` (float32
        [T, width]) holds q, k, v and the two gates' sums at the columns `offsets` = (q, k, v, input gate, forget
        gate); q is scaled by `q_scale`.  state [rows, heads, head_dim * value_dim + head_dim + 1] float32 holds C,
        n and m of row read_rows[entry] (zeros, m included, where the entry starts its request) and receives them
        in row write_rows[entry].  Returns o, float32 [T, heads * value_dim].  Steps of few tokens an entry walk
        every entry whole; steps with `MEMORY_RUNS_FROM` tokens more than entries cut them into runs of 64 tokens
        that are all walked at once, twice, with the state carried between the walks (`in_runs` forces one way):
        that reorders 32-bit sums only."""
        self._check(projected, "projected input", torch.float32, (None, None))
        tokens, width = projected.shape
        entries = ctx.num_entries
        self._check(state, "memory state", torch.float32, (None, heads, head_dim * value_dim + head_dim + 1))
        self._check(read_rows, "state rows to read", torch.int32, (entries,))
        self._check(write_rows, "state rows to write", torch.int32, (entries,))
        self._check(ctx.cu_q, "cu_q", torch.int32, (entries + 1,))
        self._check(ctx.q_starts, "q_starts", torch.int32, (entries,))
        q_off, k_off, v_off, i_off, f_off = (int(o) for o in offsets)
        out = self._empty((tokens, heads * value_dim), torch.float32)
        if in_runs is None:
            in_runs = tokens >= entries + self.MEMORY_RUNS_FROM
        runs = gates = None
        if in_runs:
            most = int(self.lib.mlr_matrix_memory_runs(tokens, entries))
            runs = self._empty((most, heads, head_dim * value_dim + head_dim + 1), torch.float32)
            gates = self._empty((most, heads, 2), torch.float32)
        self._call(
            "mlr_matrix_memory_scan", self._ptr(projected), width, q_off, k_off, v_off, i_off, f_off, self._ptr(state),
            state.shape[0], self._ptr(read_rows), self._ptr(write_rows), self._ptr(ctx.cu_q), self._ptr(ctx.q_starts),
            float(cap), float(q_scale), self._ptr(out), entries, heads, head_dim, value_dim, tokens, self._ptr(runs),
            self._ptr(gates), self._stream(),
        )
        return out

    # ---- routed experts --------------------------------------------------------------------------------
    def route_experts(
        self, logits: torch.Tensor, correction: Optional[torch.Tensor], *, top: int, groups: int, keep_groups: int,
        scale: float, scores: str = "sigmoid", normalise: bool = False,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """Which experts every token uses (int32 [T, top]) and with what weight (float32 [T, top]),
        from the router's float32 logits z [T, experts]: s = sigmoid(z), c = s + correction; the expert
        axis is cut into `groups` contiguous blocks, a block scores the top-2 sum of its c, and ids are
        the arg-top-`top` of c over the experts of the `keep_groups` highest blocks; weights = s[ids] *
        `scale` (c only decides).  scores="softmax": s = softmax(z) over all experts instead.  normalise: the
        chosen weights are divided by their sum (+ 1e-20) before the scale."""
        if scores not in ("sigmoid", "softmax"):
            raise KernelError("router scores are 'sigmoid' or 'softmax'")
        self._check(logits, "router logits", torch.float32, (None, None))
        tokens, experts = logits.shape
        if correction is not None:
            self._check(correction, "router correction", torch.float32, (experts,))
        ids = self._empty((tokens, top), torch.int32)
        weights = self._empty((tokens, top), torch.float32)
        self._call(
            "mlr_moe_route", self._ptr(logits), self._ptr(correction), self._ptr(ids), self._ptr(weights), tokens,
            experts, int(top), int(groups), int(keep_groups), float(scale), int(scores == "softmax"), int(bool(normalise)),
            self._stream(),
        )
        return ids, weights

    def expert_products(
        self,
        h: torch.Tensor,
        up_weight: torch.Tensor,
        down_weight: torch.Tensor,
        ids: torch.Tensor,
        weights: torch.Tensor,
        *,
        experts: int,
        activation: str,
        kernel: str = "auto",
        pass_through: int = 0,
    ) -> torch.Tensor:
        """The chosen experts' outputs, weighted: float32 [top, T, hidden] with [j, t] = weights[t, j]
        * down_e(act(up_e(h[t]))), e = ids[t, j]; the sum over j is the mixture's output, which a norm
        adds to the stream in that order.  activation "swiglu": a gated expert, up_weight holds every
        expert's gate rows and then its up rows ([experts * 2 * inner, hidden]) and act is silu(gate) * up, made
        by a kernel of its own between the two products.  pass_through: ids experts .. experts + pass_through
        - 1 name experts without matrices whose output is their input: [j, t] = weights[t, j] * h[t].  up_weight [experts * inner, hidden], down_weight [experts *
        hidden, inner].  Three launches: the pairs sorted by expert into tiles of rows, and a grouped
        product over the tiles for each of the two matrices (bfloat16 with hidden and inner multiples
        of 8 on the matrix cores, everything else, and kernel="fma", as plain 32-bit arithmetic)."""
        if kernel not in ("auto", "fma"):
            raise KernelError("kernel must be 'auto' or 'fma'")
        if activation not in ("relu2", "sigmoid", "swiglu"):
            raise KernelError(f"unknown activation {activation!r}")
        gated = activation == "swiglu"
        self._check(h, "expert input", self.dtype, (None, None))
        tokens, hidden = h.shape
        self._check(ids, "expert ids", torch.int32, (tokens, None))
        top = ids.shape[1]
        self._check(weights, "expert weights", torch.float32, (tokens, top))
        if experts <= 0 or up_weight.shape[0] % experts:
            raise KernelError("the stacked expert matrices do not divide by the number of experts")
        wide = up_weight.shape[0] // experts  # rows of an expert's first matrix
        if gated and wide % 2:
            raise KernelError("a gated expert's first matrix holds gate rows and as many up rows")
        inner = wide // 2 if gated else wide
        self._check(up_weight, "expert up weights", self.dtype, (experts * wide, hidden))
        self._check(down_weight, "expert down weights", self.dtype, (experts * hidden, inner))
        pairs = tokens * top
        mfma = int(kernel == "auto" and self.dtype == torch.bfloat16 and hidden % 8 == 0 and inner % 8 == 0)
        # many rows an expert (on average: the host does not know the routing): tiles of 64 rows through
        # LDS; few: tiles of 16 rows that stream the expert's weights
        big = int(bool(mfma) and pairs >= self.tuning.moe_tiled_rows * experts)
        if big and pairs >= self.tuning.moe_wide_tiled_rows * experts:
            big = 2  # tiles of 128 rows
        if big:
            mfma = 1 + big
        max_tiles = self.lib.mlr_moe_max_tiles(pairs, experts, big)
        index = self._empty((pairs + experts + 1 + 2 * max_tiles,), torch.int32)
        order, offsets, tiles = index[:pairs], index[pairs : pairs + experts + 1], index[pairs + experts + 1 :]
        self._call(
            "mlr_moe_align", self._ptr(ids), pairs, experts, big, max_tiles, self._ptr(order), self._ptr(offsets),
            self._ptr(tiles), self._stream(),
        )
        act = self._empty((pairs, wide), self.dtype)
        out = self._empty((top, tokens, hidden), torch.float32)
        common = (self._ptr(order), self._ptr(offsets), self._ptr(tiles))
        self._call(
            "mlr_moe_gemm", self._ptr(h), self._ptr(up_weight), *common, _VP(None), self._ptr(act), 1, self.code, mfma,
            max_tiles, tokens, top, wide, hidden, 0 if gated else _EPILOGUES[activation], self._stream(),
        )
        if gated:
            act = self.silu_mul(act)  # rows that no pair owns hold whatever memory held: nothing reads them
        if pass_through:
            self._call(
                "mlr_moe_identity", self._ptr(h), self._ptr(ids), self._ptr(weights), self._ptr(out), self.code, tokens,
                top, hidden, experts, self._stream(),
            )
        self._call(
            "mlr_moe_gemm", self._ptr(act), self._ptr(down_weight), *common, self._ptr(weights), self._ptr(out), 0,
            self.code, mfma, max_tiles, tokens, top, hidden, inner, 0, self._stream(),
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
