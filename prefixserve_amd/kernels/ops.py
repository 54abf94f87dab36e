"""Python face of the kernel library: checks shapes on the host, then launches the
hand-written HIP kernels on torch's current stream with raw pointers.

There is no other implementation behind these calls: without a GPU or without the
compiled library, constructing ``HipOps`` raises. The only library routine on the path is
the matrix product ``torch.matmul`` (hipBLASLt) for bfloat16 products with more than 64
rows, where the reference's engine also calls a library (prefixserve/model/llama.py:113-126);
every 32-bit product and every product with at most 64 rows is a kernel of this package.
"""

from __future__ import annotations

import contextlib
import ctypes
import logging
import os
from typing import Any, Sequence

import torch

from prefixserve_amd.build import ensure_kernels
from prefixserve_amd.parts.base import NormedRows

_F32, _BF16 = 0, 1
_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"kernels take float32 or bfloat16, got {dtype}")


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


logger = logging.getLogger(__name__)

_SIGNATURES = {
    "psamd_embed": [_vp, _vp, _vp, _i32, _vp, _i64, _i32, _i32],
    "psamd_add_rmsnorm": [_vp, _vp, _vp, _i32, _i32, _i64, _vp, _vp, _i32, _f32, _vp, _i32, _i64, _i32],
    "psamd_swiglu": [_vp, _vp, _vp, _i32, _i64, _i32, _i32],
    "psamd_rope_kv_append": [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "psamd_linear": [_vp, _vp, _i32, _vp, _i32, _vp, _i32, _i64, _i32, _i32],
    "psamd_gemm_lt": [_vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32],
    "psamd_linear_skinny": [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32],
    "psamd_linear_skinny_ksplit": [_i32, _i32, _i32],
    "psamd_qkv_rope_append": [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "psamd_normed_supports": [_i32, _i32],
    "psamd_linear_skinny_add": [_vp, _vp, _vp, _vp, _i32, _i32, _i32],
    "psamd_linear_normed": [_vp, _vp, _vp, _vp, _i32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32],
    "psamd_qkv_rope_append_normed": [_vp, _vp, _vp, _i32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "psamd_attention_generic": [_vp, _vp, _i32, _vp, _vp, _i32, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32,
                                _vp, _vp, _i32],
    "psamd_attention_mfma_supports": [_i32, _i32, _i32],
    "psamd_attention_prefill_nsplit": [_i32, _i32, _i32, _i32, _i32],
    "psamd_attention_prefill_part_rows": [_i32, _i32, _i32],
    "psamd_attention_decode_skewed": [_i32, _i32, _i64],
    "psamd_attention_decode_plan": [_i32, _i32, _i32, _i32, _i32, _vp, _vp],
    "psamd_attention_decode_max_parts": [_i32],
    "psamd_attention_prefill": [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                _f32, _i32, _vp, _vp, _i32, _i32],
    "psamd_attention_decode": [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                               _i32, _f32, _i32, _i32, _i32],
    "psamd_attention_prefill_extras": [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                       _f32, _i32, _vp, _vp, _i32, _i32, _vp, _vp, _i32],
    "psamd_attention_decode_extras": [_vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                      _i32, _f32, _i32, _i32, _i32, _vp, _vp, _i32],
    "psamd_sample": [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32],
    "psamd_scaled_add_rmsnorm": [_vp, _vp, _f32, _vp, _i32, _i32, _i64, _vp, _i32, _f32, _vp, _i32, _i64, _i32],
    "psamd_to_activation": [_vp, _vp, _vp, _i32, _i64],
    "psamd_rope_norm_kv_append": [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _i32, _f32, _vp, _vp],
    "psamd_qk_prepare_kv_append": [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _i32, _f32, _vp, _vp, _vp, _i32, _vp, _vp, _i32],
    "psamd_residual_add": [_vp, _vp, _vp, _i32, _i32, _i64, _i64, _i32],
    "psamd_stream_affine": [_vp, _vp, _i64, _i32, _f32, _vp],
    "psamd_concat_to_activation": [_vp, _vp, _vp, _vp, _i32, _i64, _i32],
    "psamd_heads_linear": [_vp, _vp, _i32, _i64, _i32, _vp, _i32, _vp, _i32, _i64, _i32, _i64, _i32, _i32, _i32],
    "psamd_latent_kv_append": [_vp, _vp, _i64, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _f32, _vp, _vp],
    "psamd_causal_conv": [_vp, _vp, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _i32, _i32],
    "psamd_gated_scan": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _i32,
                         _vp, _i32, _i32, _vp, _i32, _vp, _i32, _i32, _i32],
    "psamd_moe_route": [_vp, _vp, _i32, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _vp, _i32],
    "psamd_moe_topk": [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _i32],
    "psamd_moe_grouped_max_tiles": [_i64, _i32],
    "psamd_moe_experts_grouped": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _f32, _i32, _i32],
    "psamd_moe_topk_group": [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp, _i32],
    "psamd_moe_experts_rows": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _f32, _i32],
    "psamd_row_gate": [_vp, _vp, _vp, _i32, _vp, _i64, _i32, _i32],
    "psamd_layernorm_step": [_vp, _vp, _vp, _vp, _i32, _i32, _i64, _vp, _vp, _f32, _vp, _vp, _f32, _vp, _i32, _i64, _i32],
    "psamd_add_sinusoid": [_vp, _vp, _vp, _vp, _i64, _i32],
    "psamd_short_conv": [_vp, _vp, _i32, _i64, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32],
    "psamd_gated_delta_prepare": [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _i32, _f32, _f32],
    "psamd_general_delta_prepare": [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _i32, _i32,
                                    _i32, _f32, _f32],
    "psamd_delta_scan": [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64,
                         _vp, _vp, _i32, _i32, _i32, _i32, _i32],
    "psamd_heads_norm_gate": [_vp, _vp, _i64, _i32, _i32, _vp, _i32, _f32, _vp, _i32, _i64, _i32, _vp],
    "psamd_short_conv_to": [_vp, _vp, _i32, _i64, _vp, _vp, _vp, _i32, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32],
    "psamd_stream_rms_norm": [_vp, _vp, _vp, _f32, _i64, _i32],
    "psamd_hyper_read": [_vp, _vp, _i32, _vp, _vp, _f32, _vp, _vp, _i32, _i64, _i32],
    "psamd_hyper_write": [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i64, _f32, _vp, _i32, _i32, _i64, _f32, _i64, _i32],
    "psamd_weighted_sum": [_vp, _vp, _i32, _i32, _i64, _f32, _vp, _i32, _i32, _i64, _f32, _vp, _i64],
    "psamd_activation": [_vp, _vp, _i32, _i64, _i32],
    "psamd_gated_group_norm": [_vp, _vp, _vp, _i64, _vp, _i32, _vp, _i32, _i64, _vp, _i32, _f32, _vp, _i64, _i32],
    "psamd_state_space_prepare": [_vp, _vp, _vp, _vp, _vp, _i64, _i32],
    "psamd_matrix_memory_gates": [_vp, _vp, _vp, _f32, _vp, _vp, _i64, _vp, _vp, _i32, _i32],
    "psamd_matrix_memory_operands": [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _vp, _vp, _i64],
    "psamd_memory_read_norm_gate": [_vp, _vp, _vp, _i64, _i32, _i32, _f32, _vp, _f32, _vp, _i32, _i64, _vp, _i64],
    "psamd_pool_kv_append": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32],
    "psamd_attention_masked_mfma": [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                    _f32, _i32, _i32, _vp, _vp, _vp, _i32, _vp, _i32],
    "psamd_attention_masked": [_vp, _vp, _i32, _vp, _vp, _i32, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32, _i32,
                               _vp, _vp, _vp, _i32, _vp],
}

ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu": 3}


GATE_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2}


class HipOps:
    PREFILL_TILE_Q = 32    # queries per workgroup of the prefill attention kernel (its 4 waves split the keys)
    SKINNY_MAX_ROWS = 64
    FUSED_SWIGLU_MAX_ROWS = 32      # above it (to SKINNY_MAX_ROWS) gate/up goes to the library, where there is one
    LIBRARY_ADD_MIN_ROWS = 1024     # from here on a product that feeds the residual stream adds into it in the library
    MOE_ROUTE_FUSED_MAX_TOKENS = 0   # up to here one kernel computes router logits and choice; above, product + choice
    MOE_PAIRWISE_MAX_TOKENS = 2     # up to here a bfloat16 step's experts run pair by pair; above, grouped by expert
    MFMA_ATTENTION_EXTRAS = True    # whether the matrix-core attention takes a sink and a bias by distance
    name = "hip"

    def __init__(self, device: torch.device | str, workspace: Any = None) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("prefixserve_amd runs on a GPU only: no device kernels can run on "
                              f"{self.device} and there is no CPU implementation to fall back to")
        self.lib = ensure_kernels()
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(self.lib, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        self.lib.psamd_last_error.restype = ctypes.c_char_p
        self.lib.psamd_sample_scratch_floats.argtypes = [ctypes.c_int]
        self.lib.psamd_sample_scratch_floats.restype = ctypes.c_int64
        self.ws = workspace
        self._sample_scratch: torch.Tensor | None = None
        self._step_stream: int | None = None
        self._plans: dict[tuple, tuple[int, int]] = {}
        self._bounds: dict[Any, int] = {}                # sizes of the attention's partial-result buffers, from the library
        self._fuses: dict[tuple[int, int], bool] = {}
        self._slice_views: dict[tuple, tuple] = {}      # (name, slices, rows) -> (buffer, its [slices, rows, N] view)
        # The library for large bfloat16 products, called directly if it can be (it sets itself up
        # here, outside any capture); through torch.mm otherwise.
        self.lib.psamd_gemm_lt_available.argtypes = []
        with torch.cuda.device(self.device):
            self._direct_library = bool(self.lib.psamd_gemm_lt_available())
        # Set while a step is run for, or under, graph capture: the key length that grids and
        # LDS tables are sized by instead of the step's own, and no product with a workspace.
        self.fixed_kv_len: int | None = None
        self.fixed_skew = False      # with fixed_kv_len: whether the step's context lengths count as skewed

    # ---------------------------------------------------------------- helpers

    def _stream(self) -> int:
        if self._step_stream is not None:
            return self._step_stream
        return torch.cuda.current_stream(self.device).cuda_stream

    @contextlib.contextmanager
    def step_scope(self):
        """All calls inside go to the stream that is current now: a step runs on one stream,
        and asking torch for it costs as much as launching a small kernel."""
        outer = self._step_stream
        self._step_stream = torch.cuda.current_stream(self.device).cuda_stream
        try:
            yield
        finally:
            self._step_stream = outer

    def _ok(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.psamd_last_error().decode())

    # ------------------------------------------------- kernels a part brings itself

    def load_extension(self, path: "str | os.PathLike[str]", signatures: dict[str, list]) -> ctypes.CDLL:
        """Loads a library of device kernels built with ``build.build_extension`` and declares
        its entry points (``name -> ctypes argument types``; each returns 0 or an error code):
        how a part with a kernel of its own gets at it without a change to this file. The part
        calls ``lib.entry(ops.stream_pointer(), tensor.data_ptr(), ...)`` and hands the result to
        ``ops.check``; the stream is the step's, so the call may be captured like any other."""
        try:
            lib = ctypes.CDLL(os.fspath(path))
        except OSError as e:
            raise KernelError(f"cannot load the kernel library {path}: {e}") from None
        for name, argtypes in signatures.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                raise KernelError(f"{path} has no entry point {name}") from None
            fn.argtypes = list(argtypes)
            fn.restype = ctypes.c_int
        return lib

    def stream_pointer(self) -> int:
        """The stream this step's kernels are launched on, as a kernel library takes it."""
        return self._stream()

    @staticmethod
    def check(rc: int, what: str) -> None:
        """Raises if an entry point of an extension returned an error code."""
        if rc != 0:
            raise KernelError(f"{what} failed with code {rc}")

    @staticmethod
    def _need(cond: bool, msg: str) -> None:
        if not cond:
            raise KernelError(msg)

    def fuses_norm(self, count: int, width: int, dtype: torch.dtype) -> bool:
        """Whether a bfloat16 step of ``count`` tokens of this width runs without norm kernels:
        the products that read the normalized residual stream normalize its rows themselves
        (``NormedRows`` for x), and ``linear_to_residual`` adds into the stream."""
        if dtype != torch.bfloat16:
            return False
        key = (int(count), int(width))
        ok = self._fuses.get(key)
        if ok is None:
            ok = self._fuses[key] = bool(self.lib.psamd_normed_supports(*key))
        return ok

    def normed(self, x: "torch.Tensor | NormedRows", name: str = "normed.x") -> torch.Tensor:
        """x as a tensor: rows handed over with their norm still to be applied go through the
        norm kernel now (for a consumer whose kernel does not normalize its tokens itself)."""
        if not isinstance(x, NormedRows):
            return x
        out = self.ws.get(name, x.shape, x.dtype)
        if x.rows is None:
            self.add_rmsnorm(x.residual, None, x.weight, x.eps, out)
        else:
            self.add_rmsnorm_rows(x.residual, None, x.rows, x.weight, x.eps, out)
        return out

    def _normed_args(self, x: NormedRows, k: int) -> tuple:
        self._need(x.residual.dtype == torch.float32 and x.residual.is_contiguous() and x.residual.shape[1] == k,
                   "rows to normalize must be float32 [T, K]")
        self._need(x.weight.numel() == k and x.weight.is_contiguous(), "the norm's weight must be [K]")
        if x.rows is not None:
            self._need(x.rows.dtype == torch.int32 and x.rows.is_contiguous(), "rows must be int32")
        return x.residual.data_ptr(), _ptr(x.rows), x.weight.data_ptr(), _code(x.weight.dtype), float(x.eps)

    def prepare_matrix(self, w: torch.Tensor, rt: Any) -> torch.Tensor:
        """A weight matrix on the device in the activation dtype (bfloat16 values widen to
        float32 exactly on the 32-bit path)."""
        return w.to(device=rt.device, dtype=rt.dtype).contiguous()

    # ------------------------------------------------------------ elementwise

    def embed(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> None:
        t, h = out.shape
        self._need(ids.dtype == torch.int32 and ids.numel() == t, "embed: ids must be int32 [T]")
        self._need(table.shape[1] == h and out.dtype == torch.float32 and out.is_contiguous(), "embed: bad output")
        self._ok(self.lib.psamd_embed(self._stream(), ids.data_ptr(), table.data_ptr(), _code(table.dtype),
                                      out.data_ptr(), t, h, table.shape[0]))

    def _delta_args(self, delta, t: int, h: int, out_dtype: torch.dtype) -> tuple:
        """(pointer, dtype code, slices, stride) of a delta: [T, H] in the activation dtype, or
        [S, T, H] float32 partial sums of a K-split product."""
        if delta is None:
            return None, _F32, 0, 0
        self._need(delta.is_contiguous(), "delta must be contiguous")
        if delta.dim() == 3:
            self._need(delta.dtype == torch.float32 and delta.shape[1:] == (t, h), "partial sums must be float32 [S, T, H]")
            return delta.data_ptr(), _F32, delta.shape[0], t * h
        self._need(delta.shape == (t, h) and delta.dtype == out_dtype, "delta must match the output")
        return delta.data_ptr(), _code(delta.dtype), 1, 0

    def add_rmsnorm(self, residual, delta, weight, eps: float, out) -> None:
        t, h = residual.shape
        self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "add_rmsnorm: residual must be float32")
        self._need(out.shape == (t, h) and out.is_contiguous(), "add_rmsnorm: bad output shape")
        self._need(weight.numel() == h, "add_rmsnorm: weight size")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, out.dtype)
        self._ok(self.lib.psamd_add_rmsnorm(self._stream(), residual.data_ptr(), dptr, dcode, slices, stride, None,
                                            weight.data_ptr(), _code(weight.dtype), eps, out.data_ptr(),
                                            _code(out.dtype), t, h))

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps: float, out) -> None:
        t, h = residual.shape
        s = rows.numel()
        self._need(residual.dtype == torch.float32 and rows.dtype == torch.int32, "add_rmsnorm_rows: dtypes")
        self._need(out.shape == (s, h) and out.is_contiguous(), "add_rmsnorm_rows: bad output shape")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, out.dtype)
        self._ok(self.lib.psamd_add_rmsnorm(self._stream(), residual.data_ptr(), dptr, dcode, slices, stride,
                                            rows.data_ptr(), weight.data_ptr(), _code(weight.dtype), eps,
                                            out.data_ptr(), _code(out.dtype), s, h))

    def scaled_add_rmsnorm(self, residual, delta, alpha: float, weight, eps: float, out) -> None:
        """The norm behind the sum: residual <- weight * rmsnorm(alpha * residual + delta), in 32-bit and
        in place; ``out`` (or None) receives the same rows in the activation dtype."""
        t, h = residual.shape
        self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "scaled_add_rmsnorm: residual must be float32")
        self._need(weight.numel() == h and weight.is_contiguous(), "scaled_add_rmsnorm: weight size")
        if out is not None:
            self._need(out.shape == (t, h) and out.is_contiguous(), "scaled_add_rmsnorm: bad output shape")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, out.dtype if out is not None else torch.float32)
        self._ok(self.lib.psamd_scaled_add_rmsnorm(self._stream(), residual.data_ptr(), float(alpha), dptr, dcode, slices,
                                                   stride, weight.data_ptr(), _code(weight.dtype), float(eps), _ptr(out),
                                                   _code(out.dtype) if out is not None else _F32, t, h))

    def to_activation(self, src, out) -> None:
        """out = src (float32) in out's dtype."""
        self._need(src.dtype == torch.float32 and src.is_contiguous() and out.is_contiguous() and src.shape == out.shape,
                   "to_activation: a float32 tensor and an output of its shape")
        self._ok(self.lib.psamd_to_activation(self._stream(), src.data_ptr(), out.data_ptr(), _code(out.dtype), src.numel()))

    def swiglu(self, gate_up, out, activation: str = "silu") -> None:
        """out = act(gate) * up for [gate | up] rows; ``activation`` is the gate's: "silu", "relu" or "gelu_tanh"."""
        t, inter = out.shape
        self._need(gate_up.shape == (t, 2 * inter) and gate_up.dtype == out.dtype, "swiglu: shapes")
        self._ok(self.lib.psamd_swiglu(self._stream(), gate_up.data_ptr(), out.data_ptr(), _code(out.dtype), t, inter,
                                       GATE_ACTIVATIONS[activation]))

    def residual_add(self, residual, delta) -> None:
        """residual (float32 [T, H]) += delta: [T, H] in any kernel dtype, or [S, T, H] float32 slices
        (added in ascending order). For an arrangement that adds a sub-layer's output without a
        norm behind the sum."""
        t, h = residual.shape
        self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "residual_add: the stream is float32")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, delta.dtype)
        self._ok(self.lib.psamd_residual_add(self._stream(), residual.data_ptr(), dptr, dcode, slices, stride, t, h))

    def stream_affine(self, x, factor: float = 1.0, row=None) -> None:
        """x (float32 [T, H]) <- x * factor + row (float32 [H] or None), in place."""
        t, h = x.shape
        self._need(x.dtype == torch.float32 and x.is_contiguous(), "stream_affine: a float32 tensor")
        if row is not None:
            self._need(row.dtype == torch.float32 and row.numel() == h and row.is_contiguous(), "stream_affine: the row is float32 [H]")
        self._ok(self.lib.psamd_stream_affine(self._stream(), x.data_ptr(), t, h, float(factor), _ptr(row)))

    def concat_to_activation(self, a, b, out) -> None:
        """out[t] = [a[t], b[t]] in out's dtype; a and b float32 [T, H]."""
        t, h = a.shape
        self._need(a.dtype == torch.float32 and b.dtype == torch.float32 and a.shape == b.shape and a.is_contiguous()
                   and b.is_contiguous() and out.shape == (t, 2 * h) and out.is_contiguous(), "concat_to_activation: shapes")
        self._ok(self.lib.psamd_concat_to_activation(self._stream(), a.data_ptr(), b.data_ptr(), out.data_ptr(),
                                                     _code(out.dtype), t, h))

    def heads_linear(self, x, x_offset: int, x_head: int, w, out, out_offset: int, out_head: int) -> None:
        """One small product per head: out[t, out_offset + h * out_head + n] = sum_k x[t, x_offset + h * x_head + k]
        * w[h, n, k] for w [H, N, K]; x and out are 2-d and contiguous, their heads lie inside their
        rows. One dtype for x, w and out; float accumulation."""
        heads, n, k = w.shape
        m = x.shape[0]
        self._need(x.dim() == 2 and out.dim() == 2 and x.is_contiguous() and out.is_contiguous() and w.is_contiguous()
                   and out.shape[0] == m, "heads_linear: operands")
        self._need(x.dtype == w.dtype == out.dtype, "heads_linear: one dtype")
        self._need(x_offset >= 0 and x_offset + (heads - 1) * x_head + k <= x.shape[1]
                   and out_offset >= 0 and out_offset + (heads - 1) * out_head + n <= out.shape[1], "heads_linear: heads outside their rows")
        size = x.element_size()
        self._ok(self.lib.psamd_heads_linear(
            self._stream(), x.data_ptr() + x_offset * size, _code(x.dtype), x.shape[1], x_head, w.data_ptr(), _code(w.dtype),
            out.data_ptr() + out_offset * size, _code(out.dtype), out.shape[1], out_head, m, heads, n, k))

    def latent_kv_append(self, rows, q_lat, hq: int, dim: int, rot: int, rank: int, slots: int, positions, table,
                         norm_weight, eps: float, kv, write_slot) -> None:
        """Latent attention between its input product and the attention: ``rows`` [T, hq (dim + rot) + rank + rot]
        holds the heads' queries and the token's compressed vector with the shared key part. The
        compressed vector is normalized (weight, eps), the key part and every head's last ``rot``
        query dimensions are rotated pair by pair (neighbours; ``table`` [pos, rot/2, 2]); the page
        receives key and value, ``q_lat`` [T, hq * slots] every head's rotated part at [rank, rank + rot)
        and zeros behind it."""
        t = rows.shape[0]
        self._need(rows.is_contiguous() and q_lat.is_contiguous() and q_lat.dtype == rows.dtype
                   and rows.shape[1] >= hq * (dim + rot) + rank + rot and q_lat.shape == (t, hq * slots), "latent_kv_append: shapes")
        self._need(positions.dtype == torch.int32 and positions.numel() == t, "latent_kv_append: positions")
        self._need(norm_weight.dtype == torch.float32 and norm_weight.numel() == rank and norm_weight.is_contiguous(),
                   "latent_kv_append: the norm's weight is float32 [rank]")
        if rot:
            self._need(table is not None and table.dtype == torch.float32 and table.shape[1:] == (rot // 2, 2)
                       and table.is_contiguous() and table.shape[0] >= 1, "latent_kv_append: table must be float32 [positions, rot/2, 2]")
        if kv is not None:
            self._need(kv.dtype == rows.dtype and kv.shape[1:] == (2, 1, 16 * slots) and kv.is_contiguous(),
                       "latent_kv_append: cache must be [blocks, 2, 1, 16 * slots] in the activation dtype")
            self._need(write_slot.dtype == torch.int32 and write_slot.numel() == t, "latent_kv_append: write slots")
        self._ok(self.lib.psamd_latent_kv_append(self._stream(), rows.data_ptr(), rows.shape[1], q_lat.data_ptr(), _code(rows.dtype),
                                                 t, hq, dim, rot, rank, slots, positions.data_ptr(), _ptr(table),
                                                 norm_weight.data_ptr(), float(eps), _ptr(kv),
                                                 None if kv is None else write_slot.data_ptr()))

    def _state_args(self, state, ctx, width: int, taps: int) -> tuple:
        self._need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
                   and state.shape[1] >= taps * width, "recurrence: the state is float32 [slots, taps * width]")
        # Slot numbers are checked by the step packer against the number of slots the runner made.
        return state.data_ptr(), state.shape[1]

    def causal_conv(self, rows, col: int, bias, conv_w, conv_b, u, state, ctx) -> None:
        """u[t, c] = conv_b[c] + sum_j conv_w[c, j] v(t - (taps - 1) + j, c), v = rows[:, col + c] + bias[c] over
        each item's tokens, continued in front of the item's first token from the inputs its state
        slot saved (``state`` [slots, taps * width]: taps - 1 saved inputs, oldest first, then the
        recurrence's own row). ``u`` is float32 [T, width]. The state is only read."""
        t, width = u.shape
        taps = conv_w.shape[1]
        self._need(rows.is_contiguous() and 0 <= col and col + width <= rows.shape[1] and rows.shape[0] == t, "causal_conv: rows")
        self._need(u.dtype == torch.float32 and u.is_contiguous(), "causal_conv: u is float32")
        for v, shape in ((bias, (width,)), (conv_w, (width, taps)), (conv_b, (width,))):
            self._need(v.dtype == torch.float32 and tuple(v.shape) == shape and v.is_contiguous(), "causal_conv: float32 parameters")
        self._need(t == ctx.num_tokens, "causal_conv: token count differs from the step batch")
        sptr, srow = self._state_args(state, ctx, width, taps)
        self._ok(self.lib.psamd_causal_conv(self._stream(), rows.data_ptr() + col * rows.element_size(), _code(rows.dtype),
                                            rows.shape[1], bias.data_ptr(), conv_w.data_ptr(), conv_b.data_ptr(), u.data_ptr(),
                                            sptr, srow, ctx.tok_item.data_ptr(), ctx.item_start.data_ptr(),
                                            ctx.slots.data_ptr(), t, width, taps))

    def gated_scan(self, gates, gate_bias, u, decay, rows, y_col: int, x_col: int, y_bias, x_bias, out, state, ctx,
                   blocks: int, taps: int) -> None:
        """The gated linear recurrence over each item's tokens from its state slot (see ``causal_conv`` for
        the slot's layout): r, i = sigmoid(gates[t, b, :bw] + ., gates[t, b, bw:] + .), log a = decay * r,
        S <- a S + sqrt(1 - a^2) i u; out = S * gelu_tanh(rows[:, y_col + c] + y_bias). Leaves S and the
        item's last taps - 1 inputs (rows[:, x_col + c] + x_bias) in the slot."""
        t, width = u.shape
        self._need(gates.dtype == torch.float32 and gates.shape == (t, 2 * width) and gates.is_contiguous()
                   and u.dtype == torch.float32 and u.is_contiguous(), "gated_scan: gates and u are float32")
        self._need(width % blocks == 0 and out.shape == (t, width) and out.is_contiguous() and out.dtype == rows.dtype
                   and rows.is_contiguous() and max(y_col, x_col) + width <= rows.shape[1] and rows.shape[0] == t, "gated_scan: shapes")
        for v, n in ((gate_bias, 2 * width), (decay, width), (y_bias, width), (x_bias, width)):
            self._need(v.dtype == torch.float32 and v.numel() == n and v.is_contiguous(), "gated_scan: float32 parameters")
        self._need(t == ctx.num_tokens, "gated_scan: token count differs from the step batch")
        sptr, srow = self._state_args(state, ctx, width, taps)
        size = rows.element_size()
        # Items of more than one token are cut into the step's tiles of queries: summed up tile by tile,
        # then run side by side. Room for the carries of the most tiles any step of this many tokens has.
        n_tiles, n_single = int(ctx.num_prefill_tiles), int(ctx.num_decode)
        self._need(ctx.pf_tiles.dtype == torch.int32 and ctx.dec_items.dtype == torch.int32, "gated_scan: the step's lists")
        carry = None
        if n_tiles:
            carry = self.ws.get("recurrent.carry", (3 * n_tiles * width,), torch.float32)
        self._ok(self.lib.psamd_gated_scan(self._stream(), gates.data_ptr(), gate_bias.data_ptr(), u.data_ptr(), decay.data_ptr(),
                                           rows.data_ptr() + y_col * size, rows.data_ptr() + x_col * size, _code(rows.dtype),
                                           rows.shape[1], y_bias.data_ptr(), x_bias.data_ptr(), out.data_ptr(), sptr, srow,
                                           ctx.item_start.data_ptr(), ctx.slots.data_ptr(), ctx.num_items,
                                           ctx.pf_tiles.data_ptr(), n_tiles, self.PREFILL_TILE_Q, ctx.dec_items.data_ptr(),
                                           n_single, _ptr(carry), width, blocks, taps))

    def rope_kv_append(self, qkv, hq: int, hkv: int, d: int, positions, table, kv, write_slot) -> None:
        t = qkv.shape[0]
        self._need(qkv.shape[1] == (hq + 2 * hkv) * d and qkv.is_contiguous(), "rope_kv_append: qkv shape")
        self._need(positions.dtype == torch.int32 and positions.numel() == t, "rope_kv_append: positions")
        if table is not None:
            self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                       "rope_kv_append: table must be float32 [positions, D/2, 2]")
        if kv is not None:
            self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                       "rope_kv_append: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
            self._need(write_slot.dtype == torch.int32 and write_slot.numel() == t, "rope_kv_append: write slots")
        self._ok(self.lib.psamd_rope_kv_append(self._stream(), qkv.data_ptr(), _code(qkv.dtype), t, hq, hkv, d,
                                               positions.data_ptr(), _ptr(table), _ptr(kv),
                                               None if kv is None else write_slot.data_ptr()))

    def rope_norm_kv_append(self, qkv, hq: int, hkv: int, d: int, positions, table, kv, write_slot, norm_dim: int,
                            norm_eps: float, bias=None, q_weight=None, k_weight=None, values_from_keys: bool = False,
                            q_weight_per_head: bool = False) -> None:
        """``rope_kv_append`` with every q and k head divided, behind the rotation, by the root mean
        square over its ``norm_dim`` own dimensions (0: no norm; the head's other slots hold zeros).
        ``hkv`` may be 0: rows of queries alone, nothing written to pages. ``bias`` (float32
        [(hq + hkv) * d]) is added to the q and k heads first; ``q_weight`` / ``k_weight`` (float32 [d])
        multiply the normalized heads; ``values_from_keys``: the rows are [q | k] only and the value
        written to the pages is the key as projected (with its bias, before rotation and norm).
        ``q_weight_per_head``: ``q_weight`` is float32 [hq * d], a factor of its own for every query head."""
        t = qkv.shape[0]
        general = bias is not None or q_weight is not None or k_weight is not None or values_from_keys
        if general:
            row_heads = hq + (hkv if values_from_keys else 2 * hkv)
            self._need(qkv.shape[1] == row_heads * d and qkv.is_contiguous(), "rope_norm_kv_append: qkv shape")
            self._need(positions.dtype == torch.int32 and positions.numel() == t, "rope_norm_kv_append: positions")
            self._need(0 <= norm_dim <= d and d % 2 == 0 and d <= 256, "rope_norm_kv_append: head sizes")
            for v, n in ((bias, (hq + hkv) * d), (q_weight, hq * d if q_weight_per_head else d), (k_weight, d)):
                if v is not None:
                    self._need(v.dtype == torch.float32 and v.numel() == n and v.is_contiguous(),
                               "rope_norm_kv_append: bias and norm weights are float32")
            if table is not None:
                self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous()
                           and table.shape[0] >= 1, "rope_norm_kv_append: table must be float32 [positions, D/2, 2]")
            if kv is not None:
                self._need(hkv > 0 and kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                           "rope_norm_kv_append: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
                self._need(write_slot.dtype == torch.int32 and write_slot.numel() == t, "rope_norm_kv_append: write slots")
            self._ok(self.lib.psamd_qk_prepare_kv_append(
                self._stream(), qkv.data_ptr(), _code(qkv.dtype), t, hq, hkv, d, positions.data_ptr(), _ptr(table),
                int(norm_dim), float(norm_eps), _ptr(bias), _ptr(q_weight), _ptr(k_weight), int(values_from_keys), _ptr(kv),
                None if kv is None else write_slot.data_ptr(), int(q_weight_per_head)))
            return
        self._need(qkv.shape[1] == (hq + 2 * hkv) * d and qkv.is_contiguous(), "rope_norm_kv_append: qkv shape")
        self._need(positions.dtype == torch.int32 and positions.numel() == t, "rope_norm_kv_append: positions")
        self._need(0 <= norm_dim <= d and d % 2 == 0 and d <= 256, "rope_norm_kv_append: head sizes")
        if table is not None:
            self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                       "rope_norm_kv_append: table must be float32 [positions, D/2, 2]")
            self._need(table.shape[0] >= 1, "rope_norm_kv_append: empty table")
        if kv is not None:
            self._need(hkv > 0 and kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                       "rope_norm_kv_append: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
            self._need(write_slot.dtype == torch.int32 and write_slot.numel() == t, "rope_norm_kv_append: write slots")
        self._ok(self.lib.psamd_rope_norm_kv_append(self._stream(), qkv.data_ptr(), _code(qkv.dtype), t, hq, hkv, d,
                                                    positions.data_ptr(), _ptr(table), int(norm_dim), float(norm_eps),
                                                    _ptr(kv), None if kv is None else write_slot.data_ptr()))

    def qkv_rope_append(self, x, w_qkv, qkv, hq: int, hkv: int, d: int, positions, table, kv, write_slot) -> None:
        """qkv = x @ w_qkv^T, q and k rotated, k and v written to their pages. One kernel for a
        bfloat16 step of at most 64 tokens; otherwise the product followed by ``rope_kv_append``."""
        m, k = x.shape
        if isinstance(x, NormedRows):
            if (x.rows is None and d % 16 == 0 and qkv.dtype == torch.bfloat16 and self.fuses_norm(m, k, x.dtype)):
                resid, _rows, nw, nw_code, eps = self._normed_args(x, k)
                self._need(w_qkv.shape == ((hq + 2 * hkv) * d, k) and qkv.shape == (m, (hq + 2 * hkv) * d), "qkv: shapes")
                self._need(w_qkv.is_contiguous() and qkv.is_contiguous() and w_qkv.dtype == torch.bfloat16, "qkv: operands")
                self._need(positions.dtype == torch.int32 and positions.numel() == m, "qkv: positions")
                if table is not None:
                    self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                               "qkv: table must be float32 [positions, D/2, 2]")
                if kv is not None:
                    self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                               "qkv: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
                    self._need(write_slot.dtype == torch.int32 and write_slot.numel() == m, "qkv: write slots")
                self._ok(self.lib.psamd_qkv_rope_append_normed(
                    self._stream(), resid, nw, nw_code, eps, w_qkv.data_ptr(), qkv.data_ptr(), m, k, hq, hkv, d,
                    positions.data_ptr(), _ptr(table), _ptr(kv), None if kv is None else write_slot.data_ptr()))
                return
            x = self.normed(x)
        if (x.dtype == torch.bfloat16 and 0 < m <= self.SKINNY_MAX_ROWS and k % 8 == 0 and d % 16 == 0):
            self._need(w_qkv.shape == ((hq + 2 * hkv) * d, k) and qkv.shape == (m, (hq + 2 * hkv) * d), "qkv: shapes")
            self._need(x.is_contiguous() and w_qkv.is_contiguous() and qkv.is_contiguous(), "qkv: contiguous operands")
            self._need(positions.dtype == torch.int32 and positions.numel() == m, "qkv: positions")
            if table is not None:
                self._need(table.dtype == torch.float32 and table.shape[1:] == (d // 2, 2) and table.is_contiguous(),
                           "qkv: table must be float32 [positions, D/2, 2]")
            if kv is not None:
                self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                           "qkv: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
                self._need(write_slot.dtype == torch.int32 and write_slot.numel() == m, "qkv: write slots")
            self._ok(self.lib.psamd_qkv_rope_append(self._stream(), x.data_ptr(), w_qkv.data_ptr(), qkv.data_ptr(), m, k,
                                                    hq, hkv, d, positions.data_ptr(), _ptr(table), _ptr(kv),
                                                    None if kv is None else write_slot.data_ptr()))
            return
        self.linear(x, w_qkv, qkv)
        self.rope_kv_append(qkv, hq, hkv, d, positions, table, kv, write_slot)

    # ---------------------------------------------------------------- products

    def linear(self, x, w, out) -> None:
        m, k = x.shape
        n = w.shape[0]
        if isinstance(x, NormedRows):
            if m > 0 and w.dtype == torch.bfloat16 and self.fuses_norm(m, k, x.dtype):
                resid, rows, nw, nw_code, eps = self._normed_args(x, k)
                self._need(w.shape[1] == k and out.shape == (m, n) and w.is_contiguous() and out.is_contiguous(), "linear: operands")
                self._ok(self.lib.psamd_linear_normed(self._stream(), resid, rows, nw, nw_code, eps, w.data_ptr(), out.data_ptr(),
                                                      _code(out.dtype), m, n, k, 0))
                return
            x = self.normed(x)
        self._need(w.shape[1] == k and out.shape == (m, n), f"linear: shapes {tuple(x.shape)} x {tuple(w.shape)}")
        self._need(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear: contiguous operands")
        self._need(x.dtype == w.dtype, "linear: x and w must have one dtype")
        if m == 0:
            return
        if x.dtype == torch.bfloat16 and k % 8 == 0:
            if m > self.SKINNY_MAX_ROWS and self._direct_library:
                # Library product, as in the reference (float32 output for more than 64 rows of logits).
                rc = self.lib.psamd_gemm_lt(self._stream(), x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out.dtype),
                                            m, n, k, 0 if self.fixed_kv_len else 1, 0)
                if rc != 2:                      # 2: no algorithm for this shape (without a workspace): the paths below
                    self._ok(rc)
                    return
            if m <= self.SKINNY_MAX_ROWS or out.dtype == torch.float32:
                for r0 in range(0, m, self.SKINNY_MAX_ROWS):
                    r1 = min(m, r0 + self.SKINNY_MAX_ROWS)
                    self._ok(self.lib.psamd_linear_skinny(self._stream(), x[r0:r1].data_ptr(), w.data_ptr(),
                                                          out[r0:r1].data_ptr(), _code(out.dtype), r1 - r0, n, k, 0, 1))
                return
            if out.dtype == torch.bfloat16:
                torch.matmul(x, w.t(), out=out)
                return
        self._ok(self.lib.psamd_linear(self._stream(), x.data_ptr(), _code(x.dtype), w.data_ptr(), _code(w.dtype),
                                       out.data_ptr(), _code(out.dtype), m, n, k))

    def linear_to_residual(self, x, w, name: str, residual: torch.Tensor | None = None) -> torch.Tensor | None:
        """x @ w^T for a consumer that adds it to the residual stream (the fused add+norm).
        Returns [T, N] in the activation dtype or, for a small bfloat16 step whose product has
        few output columns, [S, T, N] float32 partial sums of a K-split, which the consumer adds
        up: splitting K over workgroups is what lets such a product use the whole chip. With the
        stream itself given as ``residual`` (float32 [T, N]), a step small enough to run without
        norm kernels adds the product into it here, K-slice by K-slice, and returns None."""
        m, k = x.shape
        n = w.shape[0]
        if (residual is not None and 0 < m and x.dtype == torch.bfloat16 and k % 8 == 0 and residual.shape == (m, n)
                and self.fuses_norm(m, n, x.dtype)):
            self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "the residual stream is float32")
            self._need(w.shape[1] == k and x.is_contiguous() and w.is_contiguous(), "linear_to_residual: operands")
            self._ok(self.lib.psamd_linear_skinny_add(self._stream(), x.data_ptr(), w.data_ptr(), residual.data_ptr(), m, n, k))
            return None
        if (residual is not None and m >= self.LIBRARY_ADD_MIN_ROWS and x.dtype == torch.bfloat16 and k % 8 == 0
                and residual.shape == (m, n) and residual.dtype == torch.float32 and self._direct_library):
            # A large step: the library's product adds into the float32 stream itself (out = x w^T + out),
            # so the sum is not rounded to bfloat16 on its way there and the norm that follows reads the
            # stream alone (2,048 rows of the 1B shape: o + norm 32.9 -> 30.2 us, down + norm 78.5 -> 76.7;
            # at 512 rows down lost, 37.3 -> 40.7, hence the bound).
            self._need(w.shape[1] == k and x.is_contiguous() and w.is_contiguous() and residual.is_contiguous(),
                       "linear_to_residual: operands")
            rc = self.lib.psamd_gemm_lt(self._stream(), x.data_ptr(), w.data_ptr(), residual.data_ptr(), _F32, m, n, k,
                                        0 if self.fixed_kv_len else 1, 1)
            if rc != 2:                          # 2: no algorithm for this shape: the ways below
                self._ok(rc)
                return None
        if x.dtype == torch.bfloat16 and k % 8 == 0 and 0 < m <= self.SKINNY_MAX_ROWS:
            ksplit = self.lib.psamd_linear_skinny_ksplit(m, n, k)
            if ksplit > 1:
                self._need(w.shape[1] == k and x.is_contiguous() and w.is_contiguous(), "linear_to_residual: operands")
                # Room for the most slices of the most rows, so that the buffer never grows.
                self._need(ksplit <= 8, "linear_to_residual: more slices than there is room for")
                room = self.ws.get(name + ".slices", (8 * self.SKINNY_MAX_ROWS * n,), torch.float32)
                kept = self._slice_views.get((name, ksplit, m))
                if kept is None or kept[0] is not room:
                    kept = self._slice_views[(name, ksplit, m)] = (room, room[:ksplit * m * n].view(ksplit, m, n))
                out = kept[1]
                self._ok(self.lib.psamd_linear_skinny(self._stream(), x.data_ptr(), w.data_ptr(), out.data_ptr(),
                                                      _F32, m, n, k, 0, ksplit))
                return out
        out = self.ws.get(name, (m, n), x.dtype)
        self.linear(x, w, out)
        return out

    def linear_swiglu(self, x, w_gate_up, out, activation: str = "silu") -> None:
        """out = act(x gate^T) * (x up^T) for w_gate_up = [gate; up]; ``activation`` is the gate's."""
        epi = 1 + GATE_ACTIVATIONS[activation]       # the fused kernels' epilogue code
        m, k = x.shape
        inter = out.shape[1]
        self._need(w_gate_up.shape == (2 * inter, k) and out.shape[0] == m, "linear_swiglu: shapes")
        if m == 0:
            return
        if isinstance(x, NormedRows):
            if w_gate_up.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and self.fuses_norm(m, k, x.dtype):
                resid, rows, nw, nw_code, eps = self._normed_args(x, k)
                self._need(w_gate_up.is_contiguous() and out.is_contiguous(), "linear_swiglu: operands")
                self._ok(self.lib.psamd_linear_normed(self._stream(), resid, rows, nw, nw_code, eps, w_gate_up.data_ptr(),
                                                      out.data_ptr(), _BF16, m, inter, k, epi))
                return
            x = self.normed(x)
        self._need(x.is_contiguous() and w_gate_up.is_contiguous() and out.is_contiguous(), "linear_swiglu: contiguous operands")
        small = x.dtype == torch.bfloat16 and k % 8 == 0 and m <= self.SKINNY_MAX_ROWS
        if small and m > self.FUSED_SWIGLU_MAX_ROWS and self._direct_library:
            # Between these row counts the library's product and the activation kernel behind it
            # take less time than the fused form, which streams the weights with too few rows a wave.
            gu = self.ws.get("mlp.gate_up", (m, 2 * inter), x.dtype)
            rc = self.lib.psamd_gemm_lt(self._stream(), x.data_ptr(), w_gate_up.data_ptr(), gu.data_ptr(), _BF16,
                                        m, 2 * inter, k, 0 if self.fixed_kv_len else 1, 0)
            if rc != 2:                          # 2: no algorithm for this shape: the fused form below
                self._ok(rc)
                self.swiglu(gu, out, activation)
                return
        if small:
            self._ok(self.lib.psamd_linear_skinny(self._stream(), x.data_ptr(), w_gate_up.data_ptr(), out.data_ptr(),
                                                  _BF16, m, inter, k, epi, 1))
            return
        gu = self.ws.get("mlp.gate_up", (m, 2 * inter), x.dtype)
        self.linear(x, w_gate_up, gu)
        self.swiglu(gu, out, activation)

    # ------------------------------------------------------------------ experts

    def moe_route(self, x, w_router, chosen, weight, w_router_act=None, bias=None, mode: int = 0) -> None:
        """chosen[t, :], weight[t, :] = the experts with the largest sigmoid(x[t] . w_router[e]) and
        those scores, largest first, the lower index among equals; scores in 32-bit. With the router
        also given in the activation dtype (``w_router_act``), a step of more than
        ``MOE_ROUTE_FUSED_MAX_TOKENS`` tokens takes its logits from the product kernels (float32 sums of
        exact products, float32 out) and the choice from a kernel of its own: the fused kernel reads
        the whole router once per token with one workgroup (8 tokens of a 32 x 2,048 router: 94 us
        against 5 + 4 for product and choice), so the bound is 0 and it serves callers without that copy.
        ``bias`` (float32 [E]) is added to the logits; ``mode`` 1: the largest logits are chosen and the
        weights are the softmax over the chosen logits alone."""
        if bias is not None:
            self._need(bias.dtype == torch.float32 and bias.numel() == w_router.shape[0] and bias.is_contiguous(),
                       "moe_route: the bias is float32 [E]")
        t, k = x.shape
        e, top = w_router.shape[0], chosen.shape[1]
        if (w_router_act is not None and t > self.MOE_ROUTE_FUSED_MAX_TOKENS and w_router_act.dtype == x.dtype
                and w_router_act.shape == w_router.shape and 1 <= top <= e):
            self._need(chosen.dtype == torch.int32 and weight.dtype == torch.float32 and chosen.shape == (t, top)
                       and weight.shape == (t, top) and chosen.is_contiguous() and weight.is_contiguous(),
                       "moe_route: outputs must be int32 and float32 [T, top]")
            logits = self.ws.get("moe.logits", (t, e), torch.float32)
            self.linear(x, w_router_act, logits)
            self._grouped_for = None
            if self._groups_pairs(x.dtype, t, k) and t <= 64 and e <= 1024:
                # A small step: the workgroup that chooses also sorts the pairs for the experts' kernels.
                ints = self._group_ints(t, top, e)
                self._ok(self.lib.psamd_moe_topk_group(self._stream(), logits.data_ptr(), chosen.data_ptr(), weight.data_ptr(),
                                                       ints.data_ptr(), t, e, top, _ptr(bias), int(mode)))
                self._grouped_for = (chosen.data_ptr(), t, top, e)
                return
            self._ok(self.lib.psamd_moe_topk(self._stream(), logits.data_ptr(), chosen.data_ptr(), weight.data_ptr(), t, e, top,
                                             _ptr(bias), int(mode)))
            return
        self._grouped_for = None
        self._need(x.is_contiguous() and w_router.dtype == torch.float32 and w_router.is_contiguous()
                   and w_router.shape[1] == k, "moe_route: x [T, K], router float32 [E, K]")
        self._need(chosen.dtype == torch.int32 and weight.dtype == torch.float32 and chosen.shape == (t, top)
                   and weight.shape == (t, top) and chosen.is_contiguous() and weight.is_contiguous() and 1 <= top <= e,
                   "moe_route: outputs must be int32 and float32 [T, top]")
        self._ok(self.lib.psamd_moe_route(self._stream(), x.data_ptr(), _code(x.dtype), w_router.data_ptr(),
                                          chosen.data_ptr(), weight.data_ptr(), t, k, e, top, _ptr(bias), int(mode)))

    def _groups_pairs(self, dtype: torch.dtype, t: int, k: int) -> bool:
        """Whether a step of ``t`` tokens of width ``k`` runs its experts grouped by expert."""
        return dtype == torch.bfloat16 and t > self.MOE_PAIRWISE_MAX_TOKENS and k % 8 == 0

    def _group_ints(self, t: int, top: int, e: int) -> torch.Tensor:
        tiles = int(self.lib.psamd_moe_grouped_max_tiles(t * top, e))
        return self.ws.get("moe.group", (t * top + 3 * tiles,), torch.int32)

    def moe_experts(self, x, chosen, weight, w_gate_up, w_down, act, out, gate_alpha: float, limit: float,
                    up_shift: float, weight_on_output: bool = False) -> None:
        """out[j, t] = down_e(act_e(weight[t, j] * x[t])) for e = chosen[t, j], as float32 slices [top, T, K];
        ``act`` [T * top, F] is scratch in the activation dtype. ``weight_on_output``: out[j, t] =
        weight[t, j] * down_e(act_e(x[t])) instead."""
        t, k = x.shape
        top = chosen.shape[1]
        e, f2, _ = w_gate_up.shape
        f = f2 // 2
        self._need(w_gate_up.shape == (e, 2 * f, k) and w_down.shape == (e, k, f) and w_gate_up.is_contiguous()
                   and w_down.is_contiguous() and w_gate_up.dtype == x.dtype and w_down.dtype == x.dtype,
                   "moe_experts: weights must be [E, 2F, K] and [E, K, F] in the activation dtype")
        self._need(x.is_contiguous() and chosen.shape == (t, top) and weight.shape == (t, top) and chosen.dtype == torch.int32
                   and weight.dtype == torch.float32 and chosen.is_contiguous() and weight.is_contiguous(),
                   "moe_experts: the router's outputs")
        self._need(act.shape == (t * top, f) and act.dtype == x.dtype and act.is_contiguous(), "moe_experts: act scratch")
        self._need(out.shape == (top, t, k) and out.dtype == torch.float32 and out.is_contiguous(), "moe_experts: output slices")
        if self._groups_pairs(x.dtype, t, k) and f % 8 == 0:
            # Sorted by expert and run in tiles on the matrix cores: an expert is read once per tile of pairs.
            ints = self._group_ints(t, top, e)
            done = int(getattr(self, "_grouped_for", None) == (chosen.data_ptr(), t, top, e))   # the router's kernel sorted them
            self._grouped_for = None
            self._ok(self.lib.psamd_moe_experts_grouped(self._stream(), x.data_ptr(), chosen.data_ptr(), weight.data_ptr(),
                                                        w_gate_up.data_ptr(), w_down.data_ptr(), act.data_ptr(),
                                                        out.data_ptr(), ints.data_ptr(), t, k, f, e, top, float(gate_alpha),
                                                        float(limit), float(up_shift), done, int(weight_on_output)))
            return
        self._ok(self.lib.psamd_moe_experts_rows(self._stream(), x.data_ptr(), chosen.data_ptr(), weight.data_ptr(),
                                                 w_gate_up.data_ptr(), w_down.data_ptr(), act.data_ptr(), out.data_ptr(),
                                                 _code(x.dtype), t, k, f, e, top, float(gate_alpha), float(limit),
                                                 float(up_shift), int(weight_on_output)))

    def row_gate(self, out, x, w) -> None:
        """out[t, :] *= sigmoid(x[t] . w): float32 out [T, N], x [T, K] in a kernel dtype, w float32 [K]."""
        t, k = x.shape
        self._need(out.dtype == torch.float32 and out.is_contiguous() and out.shape[0] == t and x.is_contiguous()
                   and w.dtype == torch.float32 and w.numel() == k and w.is_contiguous(), "row_gate: operands")
        self._ok(self.lib.psamd_row_gate(self._stream(), out.data_ptr(), x.data_ptr(), _code(x.dtype), w.data_ptr(), t,
                                         out.shape[1], k))

    # ------------------------------------------------------- layer norm, sinusoid

    def layernorm_step(self, residual, delta, post, pre, out, rows=None) -> None:
        """Layer norm with weight and bias around the stream; ``post`` and ``pre`` are (weight, bias, eps)
        with float32 [H] tensors, or None. With ``delta`` ([T, H] in a kernel dtype or [S, T, H] float32
        slices): residual += post(delta). With ``out``: out = pre(residual) in out's dtype; ``rows``
        (int32 [n], without a delta) picks the rows of the stream that ``out`` is made of."""
        t, h = residual.shape
        self._need(residual.dtype == torch.float32 and residual.is_contiguous(), "layernorm_step: the stream is float32")
        for terms in (post, pre):
            if terms is not None:
                self._need(all(v.dtype == torch.float32 and v.numel() == h and v.is_contiguous() for v in terms[:2]),
                           "layernorm_step: weight and bias are float32 [H]")
        self._need((delta is None) == (post is None) and (out is None) == (pre is None) and (delta is not None or out is not None),
                   "layernorm_step: a delta with the norm behind it, an output with the norm in front of it")
        n = t
        if rows is not None:
            self._need(delta is None and rows.dtype == torch.int32 and rows.is_contiguous(), "layernorm_step: rows are int32, without a delta")
            n = rows.numel()
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, delta.dtype if delta is not None else torch.float32)
        if out is not None:
            self._need(out.shape == (n, h) and out.is_contiguous(), "layernorm_step: bad output shape")
        pw, pb, pe = (post[0].data_ptr(), post[1].data_ptr(), float(post[2])) if post is not None else (None, None, 0.0)
        qw, qb, qe = (pre[0].data_ptr(), pre[1].data_ptr(), float(pre[2])) if pre is not None else (None, None, 0.0)
        self._ok(self.lib.psamd_layernorm_step(self._stream(), residual.data_ptr(), _ptr(rows), dptr, dcode, max(slices, 1), stride,
                                               pw, pb, pe, qw, qb, qe, _ptr(out), _code(out.dtype) if out is not None else _F32,
                                               n, h))

    def add_sinusoid(self, x, positions, freq) -> None:
        """x[t, 2i] += sin(positions[t] * freq[i]), x[t, 2i + 1] += cos(.); x float32 [T, H], freq float64 [(H + 1) // 2]."""
        t, h = x.shape
        self._need(x.dtype == torch.float32 and x.is_contiguous() and positions.dtype == torch.int32 and positions.numel() == t
                   and freq.dtype == torch.float64 and freq.numel() == (h + 1) // 2 and freq.is_contiguous(), "add_sinusoid: operands")
        self._ok(self.lib.psamd_add_sinusoid(self._stream(), x.data_ptr(), positions.data_ptr(), freq.data_ptr(), t, h))

    # ------------------------------------------------------------ delta rules

    def short_conv(self, rows, col: int, conv_w, out, state, state_offset: int, ctx, silu: bool = True, bias=None) -> None:
        """out[t, c] = act(bias[c] + sum_j conv_w[c, j] v(t - (taps - 1) + j, c)), v = rows[:, col + c], over each item's
        tokens, continued in front of an item's first token from the inputs its state slot saved
        (``state[slot, state_offset + j * channels + c]``, oldest first), which are then replaced by the
        item's last taps - 1 inputs. ``rows`` and ``out`` ([T, channels]) are float32 or bfloat16, each on its own;
        ``bias`` is float32 [channels] or None."""
        t, channels = out.shape
        taps = conv_w.shape[1]
        self._need(rows.is_contiguous() and rows.shape[0] == t and 0 <= col and col + channels <= rows.shape[1], "short_conv: rows")
        self._need(out.is_contiguous() and conv_w.dtype == torch.float32
                   and tuple(conv_w.shape) == (channels, taps) and conv_w.is_contiguous(), "short_conv: float32 taps [channels, taps] and output")
        if bias is not None:
            self._need(bias.dtype == torch.float32 and bias.numel() == channels and bias.is_contiguous(), "short_conv: the bias is float32 [channels]")
        self._need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous()
                   and 0 <= state_offset and state_offset + (taps - 1) * channels <= state.shape[1], "short_conv: the state's saved inputs")
        self._need(t == ctx.num_tokens, "short_conv: token count differs from the step batch")
        self._ok(self.lib.psamd_short_conv_to(self._stream(), rows.data_ptr() + col * rows.element_size(), _code(rows.dtype),
                                              rows.shape[1], conv_w.data_ptr(), _ptr(bias), out.data_ptr(), _code(out.dtype), channels,
                                              state.data_ptr() + 4 * state_offset, state.shape[1], ctx.tok_item.data_ptr(),
                                              ctx.item_start.data_ptr(), ctx.slots.data_ptr(), t, ctx.num_items, channels, taps,
                                              int(silu)))

    # ------------------------------------------ several streams, mixers side by side, recurrences through the delta scan

    def stream_rms_norm(self, x, weight, eps: float) -> None:
        """x (float32 [T, H]) <- weight * x / sqrt(mean(x^2) + eps), row by row and in place."""
        t, h = x.shape
        self._need(x.dtype == torch.float32 and x.is_contiguous() and weight.dtype == torch.float32 and weight.numel() == h
                   and weight.is_contiguous(), "stream_rms_norm: float32 rows and weight")
        self._ok(self.lib.psamd_stream_rms_norm(self._stream(), x.data_ptr(), weight.data_ptr(), float(eps), t, h))

    def _streams(self, streams, what: str) -> tuple[int, int, int]:
        self._need(streams.dtype == torch.float32 and streams.dim() == 3 and streams.is_contiguous() and 1 <= streams.shape[0] <= 16,
                   f"{what}: the streams are float32 [count <= 16, T, H]")
        return tuple(streams.shape)

    def hyper_read(self, streams, read, weight, eps: float, out, factor=None) -> None:
        """out = u / sqrt(mean(u^2) + eps) * weight (* factor), u = sum_s read[s] streams[s]; out [T, H] in its own dtype."""
        count, t, h = self._streams(streams, "hyper_read")
        for v, n in ((read, count), (weight, h)) + (((factor, h),) if factor is not None else ()):
            self._need(v.dtype == torch.float32 and v.numel() == n and v.is_contiguous(), "hyper_read: float32 parameters")
        self._need(out.shape == (t, h) and out.is_contiguous(), "hyper_read: output")
        self._ok(self.lib.psamd_hyper_read(self._stream(), streams.data_ptr(), count, read.data_ptr(), weight.data_ptr(), float(eps),
                                           _ptr(factor), out.data_ptr(), _code(out.dtype), t, h))

    def hyper_write(self, streams, mix, write, delta, scale: float = 1.0, delta2=None, scale2: float = 0.0) -> None:
        """streams[t'] <- sum_s mix[s, t'] streams[s] + write[t'] (scale delta + scale2 delta2), all copies at once from the
        old ones; a delta is [T, H] in a kernel dtype or [S, T, H] float32 slices; delta2 may be None."""
        count, t, h = self._streams(streams, "hyper_write")
        self._need(mix.dtype == torch.float32 and tuple(mix.shape) == (count, count) and mix.is_contiguous()
                   and write.dtype == torch.float32 and write.numel() == count and write.is_contiguous(), "hyper_write: float32 parameters")
        dptr, dcode, slices, stride = self._delta_args(delta, t, h, delta.dtype)
        d2 = (None, _F32, 1, 0) if delta2 is None else self._delta_args(delta2, t, h, delta2.dtype)
        self._ok(self.lib.psamd_hyper_write(self._stream(), streams.data_ptr(), count, mix.data_ptr(), write.data_ptr(), dptr, dcode,
                                            max(slices, 1), stride, float(scale), d2[0], d2[1], max(d2[2], 1), d2[3], float(scale2), t, h))

    def weighted_sum(self, a, a_scale: float, b, b_scale: float, out) -> None:
        """out (float32 [T, H]) = a_scale * a + b_scale * b; a and b are [T, H] in a kernel dtype or [S, T, H] float32 slices."""
        t, h = out.shape
        self._need(out.dtype == torch.float32 and out.is_contiguous(), "weighted_sum: the output is float32")
        ap, ac, asl, ast = self._delta_args(a, t, h, a.dtype)
        bp, bc, bsl, bst = self._delta_args(b, t, h, b.dtype)
        self._ok(self.lib.psamd_weighted_sum(self._stream(), ap, ac, max(asl, 1), ast, float(a_scale), bp, bc, max(bsl, 1), bst,
                                             float(b_scale), out.data_ptr(), t * h))

    def activation(self, x, kind: str) -> None:
        """x <- f(x) in place: "gelu" (exact), "gelu_tanh", "silu" or "relu"."""
        self._need(x.is_contiguous(), "activation: a contiguous tensor")
        self._ok(self.lib.psamd_activation(self._stream(), x.data_ptr(), _code(x.dtype), x.numel(), ACTIVATIONS[kind]))

    def gated_group_norm(self, y, x, x_col: int, skip, heads: int, gate_rows, gate_col: int, weight, groups: int, eps: float, out) -> None:
        """v = (y + skip[head] x) silu(gate); out = v / sqrt(mean(v^2) + eps) * weight over each of ``groups`` equal parts of
        a row. y float32 [T, inner]; x float32 rows from column ``x_col``; the gate in ``gate_rows`` from ``gate_col``."""
        t, inner = y.shape
        self._need(y.dtype == torch.float32 and y.is_contiguous() and x.dtype == torch.float32 and x.is_contiguous()
                   and x.shape[0] == t and 0 <= x_col and x_col + inner <= x.shape[1], "gated_group_norm: y and x are float32")
        self._need(inner % heads == 0 and inner % groups == 0, "gated_group_norm: sizes")
        for v, n in ((skip, heads), (weight, inner)):
            self._need(v.dtype == torch.float32 and v.numel() == n and v.is_contiguous(), "gated_group_norm: float32 parameters")
        self._need(gate_rows.is_contiguous() and gate_rows.shape[0] == t and 0 <= gate_col and gate_col + inner <= gate_rows.shape[1]
                   and out.dtype == gate_rows.dtype and out.shape == (t, inner) and out.is_contiguous(), "gated_group_norm: gate and output")
        self._ok(self.lib.psamd_gated_group_norm(self._stream(), y.data_ptr(), x.data_ptr() + 4 * x_col, x.shape[1], skip.data_ptr(), heads,
                                                 gate_rows.data_ptr() + gate_col * gate_rows.element_size(), _code(gate_rows.dtype),
                                                 gate_rows.shape[1], weight.data_ptr(), groups, float(eps), out.data_ptr(), t, inner))

    def state_space_prepare(self, dt, dt_bias, decay_log, coef) -> None:
        """dt float32 [T, heads] -> coef float32 [T, 3 heads] = [exp(-exp(decay_log) d) | 0 | d], d = softplus(dt + dt_bias)."""
        t, heads = dt.shape
        self._need(dt.dtype == torch.float32 and dt.is_contiguous() and coef.dtype == torch.float32 and coef.shape == (t, 3 * heads)
                   and coef.is_contiguous(), "state_space_prepare: dt [T, heads] and coef [T, 3 heads] are float32")
        for v in (dt_bias, decay_log):
            self._need(v.dtype == torch.float32 and v.numel() == heads and v.is_contiguous(), "state_space_prepare: float32 [heads]")
        self._ok(self.lib.psamd_state_space_prepare(self._stream(), dt.data_ptr(), dt_bias.data_ptr(), decay_log.data_ptr(),
                                                    coef.data_ptr(), t, heads))

    def matrix_memory_gates(self, gates, gate_bias, cap: float, coef, state, m_offset: int, ctx) -> None:
        """gates float32 [T, 2 heads] = [input | forget] inputs; i = cap tanh((. + b) / cap), f = logsigmoid(cap tanh(.)); with
        the running maximum m' = max(f + m, i) kept in ``state[slot, m_offset + h]``: coef float32 [T, 4 heads] =
        [exp(f + m - m') | 0 | exp(i - m') | exp(-m')], token by token over each item."""
        t = gates.shape[0]
        heads = gates.shape[1] // 2
        self._need(gates.dtype == torch.float32 and gates.is_contiguous() and coef.dtype == torch.float32
                   and coef.shape == (t, 4 * heads) and coef.is_contiguous() and gate_bias.dtype == torch.float32
                   and gate_bias.numel() == 2 * heads and gate_bias.is_contiguous(), "matrix_memory_gates: float32 operands")
        self._need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous() and 0 <= m_offset
                   and m_offset + heads <= state.shape[1] and t == ctx.num_tokens, "matrix_memory_gates: the state")
        self._ok(self.lib.psamd_matrix_memory_gates(self._stream(), gates.data_ptr(), gate_bias.data_ptr(), float(cap), coef.data_ptr(),
                                                    state.data_ptr() + 4 * m_offset, state.shape[1], ctx.item_start.data_ptr(),
                                                    ctx.slots.data_ptr(), ctx.num_items, heads))

    def matrix_memory_operands(self, rows, q_col: int, k_col: int, v_col: int, heads: int, dim: int, vdim: int, q_scale: float,
                               u, vals) -> None:
        """u float32 [T, 2 heads dim] = [q * q_scale | k]; vals float32 [T, heads (vdim + 1)] = per head [v | 1]."""
        t = rows.shape[0]
        self._need(rows.is_contiguous() and u.dtype == torch.float32 and u.shape == (t, 2 * heads * dim) and u.is_contiguous()
                   and vals.dtype == torch.float32 and vals.shape == (t, heads * (vdim + 1)) and vals.is_contiguous(),
                   "matrix_memory_operands: shapes")
        self._ok(self.lib.psamd_matrix_memory_operands(self._stream(), rows.data_ptr(), _code(rows.dtype), rows.shape[1], q_col, k_col,
                                                       v_col, heads, dim, vdim, float(q_scale), u.data_ptr(), vals.data_ptr(), t))

    def memory_read_norm_gate(self, raw, coef, floor_col: int, heads: int, vdim: int, read_eps: float, weight, eps: float,
                              gate_rows, gate_col: int, out) -> None:
        """raw float32 [T, heads (vdim + 1)] = per head [S^T q | n . q]: o = S^T q / (max(|n . q|, coef[t, floor_col + h]) +
        read_eps); out = o / sqrt(mean(o^2) + eps) * weight[h] * sigmoid(gate)."""
        t = raw.shape[0]
        self._need(raw.dtype == torch.float32 and raw.shape == (t, heads * (vdim + 1)) and raw.is_contiguous()
                   and coef.dtype == torch.float32 and coef.is_contiguous() and coef.shape[0] == t and 0 <= floor_col
                   and floor_col + heads <= coef.shape[1], "memory_read_norm_gate: raw and coef are float32")
        self._need(weight.dtype == torch.float32 and weight.numel() == heads * vdim and weight.is_contiguous(), "memory_read_norm_gate: weight")
        self._need(gate_rows.is_contiguous() and gate_rows.shape[0] == t and 0 <= gate_col and gate_col + heads * vdim <= gate_rows.shape[1]
                   and out.dtype == gate_rows.dtype and out.shape == (t, heads * vdim) and out.is_contiguous(), "memory_read_norm_gate: gate and output")
        self._ok(self.lib.psamd_memory_read_norm_gate(self._stream(), raw.data_ptr(), coef.data_ptr() + 4 * floor_col, coef.shape[1], heads,
                                                      vdim, float(read_eps), weight.data_ptr(), float(eps),
                                                      gate_rows.data_ptr() + gate_col * gate_rows.element_size(),
                                                      _code(gate_rows.dtype), gate_rows.shape[1], out.data_ptr(), t))

    def pool_kv_append(self, kv, pool_kv, ctx, group: int, pool_group: int, hkv: int, d: int, block: int) -> None:
        """For every token of the step that completes a block of ``block`` tokens (the pool group's ``write_slot`` >= 0): the mean
        of the block's keys and values as the token pages hold them goes to that place of the pool's pages."""
        g, pg = ctx.groups[group], ctx.groups[pool_group]
        for pages in (kv, pool_kv):
            self._need(pages.shape[1:] == (2, hkv, 16 * d) and pages.is_contiguous() and pages.dtype == kv.dtype,
                       "pool_kv_append: pages are [blocks, 2, kv_heads, 16*D] in one dtype")
        self._ok(self.lib.psamd_pool_kv_append(self._stream(), kv.data_ptr(), pool_kv.data_ptr(), _code(kv.dtype), ctx.positions.data_ptr(),
                                               ctx.tok_item.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(),
                                               pg.write_slot.data_ptr(), ctx.num_tokens, hkv, d, block))

    def gated_delta_prepare(self, u, groups: int, dim: int, gates, decay_log, decay_bias, coef, q_scale: float,
                            unit_eps: float) -> None:
        """u (float32 [T, >= 2 groups dim]) starts with the query and key vectors ([groups, dim] each): each is
        divided by sqrt(sum of squares + unit_eps) in place, the queries also times q_scale. gates float32
        [T, 2 heads] = [strength logits | decay inputs] -> coef float32 [T, 3 heads] = [g | -b | b] with
        b = sigmoid(.), g = exp(-exp(decay_log[h]) softplus(. + decay_bias[h]))."""
        t = u.shape[0]
        heads = decay_log.numel()
        self._need(u.dtype == torch.float32 and u.is_contiguous() and u.shape[1] >= 2 * groups * dim, "gated_delta_prepare: u")
        self._need(gates.dtype == torch.float32 and gates.shape == (t, 2 * heads) and gates.is_contiguous()
                   and coef.dtype == torch.float32 and coef.shape == (t, 3 * heads) and coef.is_contiguous(),
                   "gated_delta_prepare: gates [T, 2 heads] and coef [T, 3 heads] are float32")
        for v in (decay_log, decay_bias):
            self._need(v.dtype == torch.float32 and v.numel() == heads and v.is_contiguous(), "gated_delta_prepare: float32 [heads]")
        self._ok(self.lib.psamd_gated_delta_prepare(self._stream(), u.data_ptr(), u.shape[1], groups, dim, gates.data_ptr(),
                                                    decay_log.data_ptr(), decay_bias.data_ptr(), coef.data_ptr(), t, heads,
                                                    float(q_scale), float(unit_eps)))

    def general_delta_prepare(self, rows, r_col: int, k_col: int, v_col: int, a_col: int, l_col: int, rate_bias, decay_out,
                              decay_bias, operands, heads: int, dim: int, decay_floor: float, unit_eps: float) -> None:
        """From rows (a kernel dtype; r, k, v and the rate's logits [heads, dim] at their columns, the decay
        map's inner values [rank] at l_col) to operands float32 [T, 6 heads dim] = [r | k | v | w | p | c]:
        w = exp(-decay_floor sigmoid(tanh(l) decay_out + decay_bias)) with decay_out float32 [rank, heads dim], c = k / sqrt(sum k^2 + unit_eps) per head,
        p = -sigmoid(rate logits + rate_bias) * c."""
        t = rows.shape[0]
        hd = heads * dim
        rank = decay_out.shape[0]
        self._need(rows.is_contiguous() and max(r_col, k_col, v_col, a_col) + hd <= rows.shape[1] and l_col + rank <= rows.shape[1]
                   and min(r_col, k_col, v_col, a_col, l_col) >= 0, "general_delta_prepare: columns outside the rows")
        self._need(operands.dtype == torch.float32 and operands.shape == (t, 6 * hd) and operands.is_contiguous(),
                   "general_delta_prepare: operands are float32 [T, 6 heads dim]")
        for v, shape in ((rate_bias, (hd,)), (decay_out, (rank, hd)), (decay_bias, (hd,))):
            self._need(v.dtype == torch.float32 and tuple(v.shape) == shape and v.is_contiguous(), "general_delta_prepare: float32 parameters")
        self._ok(self.lib.psamd_general_delta_prepare(self._stream(), rows.data_ptr(), _code(rows.dtype), rows.shape[1], r_col, k_col,
                                                      v_col, a_col, l_col, rate_bias.data_ptr(), decay_out.data_ptr(),
                                                      decay_bias.data_ptr(), operands.data_ptr(), t, heads, dim, rank,
                                                      float(decay_floor), float(unit_eps)))

    def delta_scan(self, keys, directions, removals, queries, key_groups: int, decay_vectors, decay, removal_scale,
                   value_scale, values, out, state, state_offset: int, ctx, heads: int, dim: int, vdim: int,
                   reads_decayed: bool, no_removal: bool = False) -> None:
        """The delta-rule recurrence over each item's tokens from its state slot. Every operand is a pair
        (float32 tensor [T, row], first column) or None. Per head h (its key group g = h // (heads / key_groups))
        and token: S' = d S with d = decay_vectors[h, :] (per key channel) times decay[h] (a number), either may
        be None = 1; S = S' + (removal_scale[h] removals[g]) (directions[g]^T S*) + keys[g] (value_scale[h]
        values[h])^T with S* = S' if ``reads_decayed`` else the S before the token; out[h] = S^T queries[g].
        ``keys``, ``directions``, ``removals``, ``queries`` lie in one tensor, as do ``decay``, ``removal_scale``,
        ``value_scale``. The state of head h is ``state[slot, state_offset + (h vdim + j) dim + i]``; out is
        float32 [T, heads vdim]. ``no_removal``: the caller says that ``removal_scale`` is zero throughout (a linear
        recurrence S = d S + k (xs x)^T in the gated rule's form: keys, directions and removals one vector, a decay per
        head); the kernel then skips the removal and the sum it waits for."""
        t = out.shape[0]
        self._need(t == ctx.num_tokens and out.dtype == torch.float32 and out.shape == (t, heads * vdim) and out.is_contiguous(),
                   "delta_scan: out is float32 [T, heads vdim]")
        if no_removal:
            self._need(reads_decayed and decay_vectors is None and keys[1] == directions[1] == removals[1],
                       "delta_scan: without removal only in the gated rule's form")
        self._need(heads % key_groups == 0 and 1 <= dim <= 256 and vdim >= 1, "delta_scan: sizes")
        base = keys[0]
        for pair in (keys, directions, removals, queries):
            self._need(pair[0] is base and 0 <= pair[1] and pair[1] + key_groups * dim <= base.shape[1], "delta_scan: key-side operands share a tensor")
        self._need(base.dtype == torch.float32 and base.is_contiguous() and base.shape[0] == t, "delta_scan: float32 operands")
        scal = [p for p in (decay, removal_scale, value_scale) if p is not None]
        sbase = scal[0][0] if scal else None
        for pair in scal:
            self._need(pair[0] is sbase and 0 <= pair[1] and pair[1] + heads <= sbase.shape[1], "delta_scan: the numbers per head share a tensor")
        if sbase is not None:
            self._need(sbase.dtype == torch.float32 and sbase.is_contiguous() and sbase.shape[0] == t, "delta_scan: float32 numbers per head")
        if decay_vectors is not None:
            dv = decay_vectors[0]
            self._need(dv.dtype == torch.float32 and dv.is_contiguous() and dv.shape[0] == t and 0 <= decay_vectors[1]
                       and decay_vectors[1] + heads * dim <= dv.shape[1], "delta_scan: decay vectors")
        xv = values[0]
        self._need(xv.dtype == torch.float32 and xv.is_contiguous() and xv.shape[0] == t and 0 <= values[1]
                   and values[1] + heads * vdim <= xv.shape[1], "delta_scan: values")
        self._need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous() and 0 <= state_offset
                   and state_offset + heads * dim * vdim <= state.shape[1], "delta_scan: the state")

        def at(pair):
            return None if pair is None else pair[0].data_ptr() + 4 * pair[1]

        self._ok(self.lib.psamd_delta_scan(
            self._stream(), at(keys), at(directions), at(removals), at(queries), base.shape[1], key_groups,
            at(decay_vectors), 0 if decay_vectors is None else decay_vectors[0].shape[1], at(decay), at(removal_scale),
            at(value_scale), 0 if sbase is None else sbase.shape[1], at(values), xv.shape[1], out.data_ptr(), out.shape[1],
            state.data_ptr() + 4 * state_offset, state.shape[1], ctx.item_start.data_ptr(), ctx.slots.data_ptr(),
            ctx.num_items, heads, dim, vdim, 2 if no_removal else int(reads_decayed)))

    def heads_norm_gate(self, o, heads: int, vdim: int, weight, weight_per_head: bool, eps: float, gate_rows, gate_col: int,
                        activation: str, out) -> None:
        """out[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * weight * act(gate[t, h, :]): o float32
        [T, heads vdim]; weight float32 [vdim] shared by the heads, or [heads vdim]; the gate lies in
        ``gate_rows`` (a kernel dtype) from column ``gate_col``; act "silu" or "sigmoid"; out in that dtype."""
        t = o.shape[0]
        self._need(o.dtype == torch.float32 and o.shape == (t, heads * vdim) and o.is_contiguous(), "heads_norm_gate: o is float32")
        self._need(weight.dtype == torch.float32 and weight.numel() == (heads * vdim if weight_per_head else vdim)
                   and weight.is_contiguous(), "heads_norm_gate: weight")
        self._need(gate_rows.is_contiguous() and gate_rows.shape[0] == t and 0 <= gate_col
                   and gate_col + heads * vdim <= gate_rows.shape[1], "heads_norm_gate: the gate's columns")
        self._need(out.dtype == gate_rows.dtype and out.shape == (t, heads * vdim) and out.is_contiguous(), "heads_norm_gate: out")
        self._ok(self.lib.psamd_heads_norm_gate(self._stream(), o.data_ptr(), t, heads, vdim, weight.data_ptr(), int(weight_per_head),
                                                float(eps), gate_rows.data_ptr() + gate_col * gate_rows.element_size(),
                                                _code(gate_rows.dtype), gate_rows.shape[1], {"silu": 0, "sigmoid": 1}[activation],
                                                out.data_ptr()))

    # --------------------------------------------------------------- attention

    def decode_is_skewed(self, count: int, longest: int, total: int) -> bool:
        """The library's rule for when the single-token items of a step have one context far
        longer than the rest (it then cuts every request's keys into long runs, as many as the
        longest needs). A captured decode step is keyed by it."""
        return bool(self.lib.psamd_attention_decode_skewed(int(count), int(longest), int(total)))

    def decode_plan(self, count: int, kv_len: int, skewed: bool, hkv: int, window: int) -> tuple[int, int]:
        """(runs per request, shortest run in keys) for a step of ``count`` single-token items."""
        plan = self._plans.get((count, kv_len, skewed, hkv, window))
        if plan is None:
            nsplit, min_run = ctypes.c_int(0), ctypes.c_int(0)
            self._ok(self.lib.psamd_attention_decode_plan(count, kv_len, int(skewed), hkv, window, ctypes.byref(nsplit),
                                                          ctypes.byref(min_run)))
            if len(self._plans) > 4096:
                self._plans.clear()
            plan = self._plans[(count, kv_len, skewed, hkv, window)] = (nsplit.value, min_run.value)
        return plan

    def mfma_attention_supported(self, hq: int, hkv: int, d: int) -> bool:
        return bool(self.lib.psamd_attention_mfma_supports(hq, hkv, d))

    def paged_attention(self, qkv, out, kv, ctx, group: int, hq: int, hkv: int, d: int, scale: float,
                        window: int | None, exact_weights: bool = False, sink=None, dist_bias=None, keep_first: int = 0,
                        pooled=None, head_gate=None) -> None:
        """``exact_weights``: the softmax weights enter the product with the values as computed in
        32-bit (the matrix-core kernels then take them as three bfloat16 terms that sum to the float32
        weight exactly) instead of rounded to bfloat16; the 32-bit kernels always do. ``sink``
        (float32 [hq]): exp(sink) joins every softmax's denominator. ``dist_bias`` (float32 [hq, n]):
        entry [h, min(i - j, n - 1)] is added to the scaled score of query i and key j. ``keep_first``: the window also
        sees the first that many positions. ``pooled`` = (pages, group, block): one mean key and value per block of tokens
        wholly in front of the window, from pages of their own. ``head_gate`` (float32 [T, hq]): output times sigmoid."""
        if keep_first or pooled is not None or head_gate is not None:
            self._need(sink is None and dist_bias is None and window is not None and window >= 1,
                       "attention: kept positions, pooled blocks and a gate per head go with a window and without sink or bias")
            t = qkv.shape[0]
            g = ctx.groups[group]
            self._need(out.shape == (t, hq * d) and out.is_contiguous() and out.dtype == qkv.dtype and t == ctx.num_tokens, "attention: output")
            self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                       "attention: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
            pool_ptr = pool_off = pool_ids = None
            block = 0
            if pooled is not None:
                pkv, pgroup, block = pooled
                self._need(pkv.dtype == qkv.dtype and pkv.shape[1:] == (2, hkv, 16 * d) and pkv.is_contiguous() and block >= 1,
                           "attention: the pooled blocks' pages")
                pg = ctx.groups[pgroup]
                pool_ptr, pool_off, pool_ids = pkv.data_ptr(), pg.table_off.data_ptr(), pg.block_ids.data_ptr()
            if head_gate is not None:
                self._need(head_gate.dtype == torch.float32 and head_gate.shape == (t, hq) and head_gate.is_contiguous(),
                           "attention: the gate is float32 [T, hq]")
            if (qkv.dtype == torch.bfloat16 and qkv.shape[1] % 8 == 0 and d <= 192 and self.mfma_attention_supported(hq, hkv, d)
                    and self.MFMA_ATTENTION_EXTRAS and (self.fixed_kv_len or ctx.max_kv_len) <= 65536):
                # The matrix cores: portions as tiles of 32 queries, single tokens as tiles of one.
                kv_len = self.fixed_kv_len or ctx.max_kv_len
                self._ok(self.lib.psamd_attention_masked_mfma(
                    self._stream(), qkv.data_ptr(), qkv.shape[1], out.data_ptr(), kv.data_ptr(), ctx.pf_tiles.data_ptr(),
                    ctx.num_prefill_tiles, ctx.dec_items.data_ptr(), ctx.num_decode, kv_len, ctx.item_start.data_ptr(),
                    ctx.item_pos0.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, float(scale),
                    int(window), int(keep_first), pool_ptr, pool_off, pool_ids, int(block), _ptr(head_gate), int(exact_weights)))
                return
            self._ok(self.lib.psamd_attention_masked(
                self._stream(), qkv.data_ptr(), qkv.shape[1], out.data_ptr(), kv.data_ptr(), _code(qkv.dtype), t,
                ctx.positions.data_ptr(), ctx.tok_item.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d,
                float(scale), int(window), int(keep_first), pool_ptr, pool_off, pool_ids, int(block), _ptr(head_gate)))
            return
        if sink is not None:
            self._need(sink.dtype == torch.float32 and sink.numel() == hq and sink.is_contiguous(), "attention: sink is float32 [hq]")
        if dist_bias is not None:
            self._need(dist_bias.dtype == torch.float32 and dist_bias.dim() == 2 and dist_bias.shape[0] == hq
                       and dist_bias.shape[1] >= 1 and dist_bias.is_contiguous(), "attention: distance bias is float32 [hq, n]")
        extras = sink is not None or dist_bias is not None
        t = qkv.shape[0]
        g = ctx.groups[group]
        self._need(out.shape == (t, hq * d) and out.is_contiguous() and out.dtype == qkv.dtype, "attention: output")
        self._need(kv.dtype == qkv.dtype and kv.shape[1:] == (2, hkv, 16 * d) and kv.is_contiguous(),
                   "attention: cache must be [blocks, 2, kv_heads, 16*D] in the activation dtype")
        self._need(t == ctx.num_tokens, "attention: token count differs from the step batch")
        win = int(window) if window is not None else 0
        stride = qkv.shape[1]
        s = self._stream()
        if (qkv.dtype == torch.bfloat16 and stride % 8 == 0 and self.mfma_attention_supported(hq, hkv, d)
                and (not extras or self.MFMA_ATTENTION_EXTRAS)):
            if ctx.num_prefill_tiles:
                kv_len = self.fixed_kv_len or ctx.max_kv_len
                # Few query tiles on a long context: the kernel deals their keys out to several
                # workgroups, whose partial results pass through these buffers. They are kept at
                # the most rows any step of this shape can need (the library says how many), so
                # they never grow.
                nsplit = self.lib.psamd_attention_prefill_nsplit(ctx.num_prefill_tiles, kv_len, hq, hkv, d)
                rows = self._bounds.get((hq, hkv, d))
                if rows is None:
                    rows = self._bounds[(hq, hkv, d)] = int(self.lib.psamd_attention_prefill_part_rows(hq, hkv, d))
                part_o = self.ws.get("attn.prefill_part_o", (rows * hq * d,), torch.float32)
                part_ml = self.ws.get("attn.prefill_part_ml", (rows * hq * 2,), torch.float32)
                if nsplit > 1:
                    self._need(32 * ctx.num_prefill_tiles * nsplit <= rows, "attention: more split tiles than planned for")
                tail = (_ptr(sink), _ptr(dist_bias), 0 if dist_bias is None else dist_bias.shape[1]) if extras else ()
                self._ok((self.lib.psamd_attention_prefill_extras if extras else self.lib.psamd_attention_prefill)(
                    s, qkv.data_ptr(), stride, out.data_ptr(), kv.data_ptr(), ctx.pf_tiles.data_ptr(),
                    ctx.num_prefill_tiles, ctx.pf_blocks.data_ptr(), ctx.num_prefill_blocks, kv_len,
                    ctx.item_start.data_ptr(), ctx.item_pos0.data_ptr(),
                    g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, scale, win,
                    part_o.data_ptr() if nsplit > 1 else None, part_ml.data_ptr() if nsplit > 1 else None, nsplit,
                    int(exact_weights), *tail))
            if ctx.num_decode:
                kv_len = self.fixed_kv_len or ctx.max_kv_len
                skewed = self.fixed_skew if self.fixed_kv_len else ctx.decode_skewed
                nsplit, min_run = self.decode_plan(ctx.num_decode, kv_len, skewed, hkv, win)
                # Room for the (request, run) pairs of any plan: asked for once, never grown.
                parts = self._bounds.get(ctx.num_decode)
                if parts is None:
                    parts = self._bounds[ctx.num_decode] = int(self.lib.psamd_attention_decode_max_parts(ctx.num_decode))
                self._need(ctx.num_decode * nsplit <= parts, "attention: more (request, run) pairs than planned for")
                part_o = self.ws.get("attn.part_o", (parts * hq * d,), torch.float32)
                part_ml = self.ws.get("attn.part_ml", (parts * hq * 2,), torch.float32)
                tail = (_ptr(sink), _ptr(dist_bias), 0 if dist_bias is None else dist_bias.shape[1]) if extras else ()
                self._ok((self.lib.psamd_attention_decode_extras if extras else self.lib.psamd_attention_decode)(
                    s, qkv.data_ptr(), stride, out.data_ptr(), kv.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(),
                    ctx.dec_items.data_ptr(), ctx.num_decode, ctx.item_start.data_ptr(),
                    ctx.item_end.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, nsplit, scale,
                    win, min_run, int(exact_weights), *tail))
            return
        self._ok(self.lib.psamd_attention_generic(
            s, qkv.data_ptr(), stride, out.data_ptr(), kv.data_ptr(), _code(qkv.dtype), t, ctx.positions.data_ptr(),
            ctx.tok_item.data_ptr(), g.table_off.data_ptr(), g.block_ids.data_ptr(), hq, hkv, d, scale, win,
            _ptr(sink), _ptr(dist_bias), 0 if dist_bias is None else dist_bias.shape[1]))

    # ---------------------------------------------------------------- sampling

    def sample(self, logits, temperatures, uniforms, out) -> None:
        rows, vocab = logits.shape
        self._need(logits.dtype == torch.float32 and logits.is_contiguous(), "sample: logits must be float32")
        self._need(temperatures.dtype == torch.float32 and uniforms.dtype == torch.float32 and
                   temperatures.numel() == rows and uniforms.numel() == rows, "sample: one temperature and uniform per row")
        self._need(out.dtype == torch.int32 and out.numel() == rows, "sample: output must be int32 [rows]")
        need = int(self.lib.psamd_sample_scratch_floats(rows))
        if self._sample_scratch is None or self._sample_scratch.numel() < need:
            # Kept apart from the workspace: growing it must not drop captured graphs.
            self._sample_scratch = torch.empty(max(need, 64 * 128), dtype=torch.float32, device=self.device)
        self._ok(self.lib.psamd_sample(self._stream(), logits.data_ptr(), temperatures.data_ptr(), uniforms.data_ptr(),
                                       out.data_ptr(), self._sample_scratch.data_ptr(), rows, vocab))

    def argmax(self, logits, out) -> None:
        rows = logits.shape[0]
        zeros = self.ws.get("sample.zeros", (rows,), torch.float32)
        zeros.zero_()
        self.sample(logits, zeros, zeros, out)
