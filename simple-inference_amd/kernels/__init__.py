"""The device kernels, as an object the parts call.

``HipKernels`` loads the compiled HIP libraries and launches their entry points on
torch's current stream, with torch tensors as buffers.  It checks on the host that
operand shapes, dtypes and devices are what the kernels and their grids assume, and
raises before a launch that would not fit.  There is no other implementation in this
package: without a GPU or without ``hipcc`` to build a missing library it raises.
Matrix products of the bfloat16 path with more than 16 rows go to the vendor's BLAS library
(called directly, or through ``torch`` where that way is not available), as the reference's
go to its vendor's (``ops/attention.py:128-130``, ``ops/mlp.py:117,128``); products of fewer
rows and the whole 32-bit path use this package's own kernels.
"""

from __future__ import annotations

import contextlib
import ctypes
from typing import Dict, Optional

import torch

from . import build

_DT = {torch.float32: 0, torch.bfloat16: 1}
_ACTIVATIONS = {"relu2": 0, "gelu_tanh": 1, "gelu": 2}   # ``SiaActivation`` of csrc/common.h
_GLUS = {"silu": 0, "clamped": 1}                        # ``SiaGlu`` of csrc/common.h

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong

_SIGNATURES = {
    "sia_embed": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_ptr],
    "sia_norm_add": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "sia_activation": [_c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_ptr],
    "sia_qk_prepare": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                       _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr,
                       _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "sia_qk_prepare_max_head_dim": [],
    "sia_gated_add_rmsnorm": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                              _c_float, _c_int, _c_ptr],
    "sia_add_bias": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_head_gate": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_side_by_side": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_scale_softcap": [_c_ptr, _c_ll, _c_float, _c_float, _c_ptr],
    "sia_gla_max_dims": [],
    "sia_gla_recurrent": [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                          _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float,
                          _c_int, _c_ptr, _c_int, _c_ptr],
    "sia_gla_workspace": [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int],
    "sia_moe_route": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_moe_route_ex": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                         _c_float, _c_ptr],
    "sia_dyt_norm": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                     _c_int, _c_int, _c_int, _c_ptr],
    "sia_causal_conv": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_hgrn2_workspace": [_c_int, _c_int, _c_int, _c_int],
    "sia_hgrn2_scan": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                       _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr, _c_ptr],
    "sia_ssd_workspace": [_c_int, _c_int, _c_int, _c_int],
    "sia_ssd_scan": [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ptr, _c_ptr,
                     _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr,
                     _c_ptr],
    "sia_latent_prepare": [_c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_float,
                           _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int,
                           _c_ptr],
    "sia_headwise_linear": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                            _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "sia_moe_gate_up": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_moe_tiled_workspace": [_c_int, _c_int, _c_int, _c_int, _c_int],
    "sia_moe_tiled": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_moe_down": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                     _c_int, _c_ptr],
    "sia_gemm_skinny_act": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_add_rmsnorm": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "sia_swiglu": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_cast": [_c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr],
    "sia_rope_kv_write": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_attention_generic": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr, _c_int,
                              _c_ptr],
    "sia_attention_max_head_dim": [],
    "sia_attention_generic_max_head_dim": [],
    "sia_gemm_generic": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_prenorm_block": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "sia_sample": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_sample_workspace_bytes": [_c_int],
    "sia_sample_static": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_sample_static_max_rows": [],
    "sia_sample_static_init": [],
    "sia_gemm_skinny": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_gemm_skinny_max_rows": [],
    "sia_gemm_skinny_residual_blocks": [_c_int],
    "sia_gemm_skinny_swiglu": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_ptr],
    "sia_gemm_skinny_rope": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                             _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_ptr],
    "sia_gemm_skinny_residual": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "sia_gemm_skinny_residual_tiled": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "sia_gemm_skinny_tile_height": [_c_int],
    "sia_gemm_skinny_tiled": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "sia_place_tokens": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "sia_scale_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_ptr],
    "sia_stream_read": [_c_ptr, _c_ll, _c_ptr, _c_ptr],
    "sia_add_rmsnorm_scaled": [_c_ptr, _c_ptr, _c_float, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float,
                               _c_int, _c_ptr],
    "sia_scaled_sum": [_c_ptr, _c_float, _c_ptr, _c_float, _c_ptr, _c_ll, _c_int, _c_ptr],
    "sia_gemm_skinny_glu": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_float, _c_int, _c_float, _c_ptr],
    "sia_glu": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "sia_qk_prepare_ex": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                          _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr,
                          _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _c_ptr],
    "sia_decay_attention": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                            _c_int, _c_int, _c_float, _c_int, _c_ptr, _c_ptr],
    "sia_delta_rule_workspace": [_c_int, _c_int, _c_int],
    "sia_delta_rule": [_c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ptr,
                       _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr,
                       _c_ptr],
    "sia_moe_route_corrected": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "sia_moe_gate_up_ex": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                           _c_ptr],
    "sia_moe_down_ex": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                        _c_ptr, _c_int, _c_int, _c_ptr],
    "sia_moe_tiled_ex": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr],
}


_ATTN_SIGNATURES = {
    "sia_attn_decode": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                        _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "sia_attn_prefill": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                         _c_ptr],
    "sia_attn_decode_ex": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                           _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr, _c_int, _c_ptr],
    "sia_attn_decode_shared": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                               _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr, _c_int, _c_ptr],
    "sia_attn_prefill_ex": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                            _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                            _c_int, _c_int, _c_ptr, _c_ptr],
    "sia_attn_decode_max_splits": [_c_int, _c_int],
    "sia_attn_decode_workspace": [_c_int, _c_int, _c_int, _c_int, _c_int],
    "sia_attn_decode_mode": [_c_int, _c_int, _c_int, _c_int],
    "sia_attn_prefill_rows": [],
    "sia_attn_prefill_rows_split": [],
    "sia_attn_prefill_rows_long": [],
    "sia_attn_mfma_head_dim": [],
}


def attention_library_spec(head_dim: int):
    """(name, sources, defines) of the matrix-core attention library for one head size."""
    return (f"attn_mfma_d{head_dim}", ("attention_mfma.hip",), (f"SIA_HEAD_DIM={head_dim}",))


class KernelError(RuntimeError):
    pass


class PendingProduct:
    """A part's output that is still to be computed: ``x @ w^T``.  A residual stream takes it for a delta; the norm
    that follows may hand it to ``linear_into_residual``, anybody else gets the tensor from ``compute()``."""

    __slots__ = ("x", "w", "kernels")

    def __init__(self, x, w, kernels):
        self.x, self.w, self.kernels = x, w, kernels

    def compute(self):
        return self.kernels.linear(self.x, self.w)


class ScaledRows:
    """Rows of an RMS norm that are multiplied by the gain but not yet divided by their root mean square:
    ``norm(x) = rows * rsqrt(sum_p partials[p, m] / width + eps)``.  ``linear``, ``gated_linear`` and ``qkv_to_cache``
    take them in place of a tensor and scale the rows of their result instead, which is the same product."""

    __slots__ = ("rows", "partials", "eps")

    def __init__(self, rows, partials, eps):
        self.rows, self.partials, self.eps = rows, partials, eps

    shape = property(lambda self: self.rows.shape)
    dtype = property(lambda self: self.rows.dtype)
    device = property(lambda self: self.rows.device)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class _BlockOwn(ctypes.Structure):
    """``SiaBlockOwn`` of csrc/block.hip."""
    _fields_ = ([(n, ctypes.c_void_p) for n in ("mixer_norm_gain", "w_qkv", "w_o", "feed_forward_norm_gain", "w_gate_up",
                                               "w_down", "cos_table", "sin_table")]
                + [(n, ctypes.c_float) for n in ("mixer_norm_eps", "feed_forward_norm_eps", "scale")]
                + [(n, ctypes.c_int) for n in ("hidden", "n_heads", "n_kv", "head_dim", "rotary_dim", "inter", "window")])


class _BlockStep(ctypes.Structure):
    """``SiaBlockStep`` of csrc/block.hip."""
    _fields_ = ([(n, ctypes.c_void_p) for n in ("product", "attend_single", "attend_runs", "residual", "normed", "qkv",
                                               "attended", "mixed", "gate_up", "activated", "fed", "positions",
                                               "seq_of_token", "cu_q", "kv_len", "ws_acc", "ws_ml")]
                + [(n, ctypes.c_int) for n in ("n_tokens", "n_seqs", "n_single", "max_splits", "n_tiles", "n_tiles_split",
                                               "n_tiles_long", "q_bound", "kv_bound")])


def _bind(lib, signatures):
    for name, argtypes in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int


class HipKernels:
    name = "hip-gfx950"

    def __init__(self, device="cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError(
                "simple-inference_amd needs an AMD GPU: torch sees no device, and the engine has no "
                "other implementation of its kernels")
        self.device = torch.device(device)
        self.core = build.load_library("core")
        _bind(self.core, _SIGNATURES)
        self.core.sia_sample_workspace_bytes.restype = ctypes.c_longlong
        self.core.sia_gla_workspace.restype = ctypes.c_longlong
        self.core.sia_moe_tiled_workspace.restype = ctypes.c_longlong
        self.core.sia_hgrn2_workspace.restype = ctypes.c_longlong
        self.core.sia_ssd_workspace.restype = ctypes.c_longlong
        self.core.sia_delta_rule_workspace.restype = ctypes.c_longlong
        self.tiled_experts = True        # many slots in bfloat16: experts' products on the matrix cores, slots sorted by expert
        self._attn_libs = {}
        # the short way to the current stream's handle, where this torch has it (a few microseconds less a launch)
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._device_index = torch.device(device).index or 0
        self.use_mfma_attention = True   # tests switch it off to reach the plain kernel in bfloat16
        self.tiled_weights = True        # tests switch it off to compare with the product that reads W as it is
        self.use_skinny_gemm = True      # few-row bfloat16 products by this package's kernel, not the library
        self.fuse_norms = True           # few rows: residual add in the product before a norm, row scale in the one after
        self.fuse_rope = True            # few rows: rotation and cache write in the q/k/v product
        self.whole_blocks = True         # many rows: a block's launches in one call (``prenorm_block``)
        self._products_known: Dict[tuple, bool] = {}
        self._skinny_rows = self.core.sia_gemm_skinny_max_rows()
        self.blas = self._load_blas()    # the BLAS library called directly; None: its products go through torch

    def _load_blas(self):
        """The direct way to the vendor's BLAS library, which spares the host most of what a product through torch
        costs it.  It is a convenience, not a kernel of this package: if it cannot be built, loaded or initialised
        the products go through torch, to the same library."""
        try:
            lib = build.load_library("blas")
            lib.sia_blas_init.argtypes, lib.sia_blas_init.restype = [], ctypes.c_int
            lib.sia_blas_mm.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr]
            lib.sia_blas_mm.restype = ctypes.c_int
            lib.sia_blas_try_out.argtypes, lib.sia_blas_try_out.restype = [_c_int], ctypes.c_int
            lib.sia_blas_can.argtypes, lib.sia_blas_can.restype = [_c_int, _c_int, _c_int, _c_int], ctypes.c_int
            with torch.cuda.device(self.device):
                if lib.sia_blas_init() != 0:
                    return None
            return lib
        except (build.KernelBuildError, OSError, AttributeError):
            return None

    @contextlib.contextmanager
    def recurring_shapes(self):
        """Inside, the products that go to the BLAS library have the library's candidate algorithms timed on their
        own operands when their shape is first met (few rows only), and the fastest kept, for use inside this context
        only: products outside it keep the library's first choice.  For runs whose shapes will recur many times: the
        eager runs before a graph is captured, and the capture itself (which times nothing and records what those
        runs chose).  Which candidate wins is decided by the clock, so the last bits of a replayed step's products
        can differ from one process to the next; within a process a graph, once captured, never changes."""
        if self.blas is None:
            yield
            return
        with torch.cuda.device(self.device):
            self.blas.sia_blas_try_out(1)
        try:
            yield
        finally:
            with torch.cuda.device(self.device):
                self.blas.sia_blas_try_out(0)

    def _library_product(self, x, w, out_float32):
        """``x @ w^T`` for bfloat16 operands by the BLAS library, float accumulation."""
        if self.blas is not None:
            M, K = x.shape
            N = w.shape[0]
            y = torch.empty((M, N), dtype=torch.float32 if out_float32 else torch.bfloat16, device=x.device)
            if self.blas.sia_blas_mm(_ptr(x), _ptr(w), _ptr(y), M, N, K, int(out_float32), self._stream()) == 0:
                return y
        y = torch.mm(x, w.t())
        return self.cast(y, torch.float32) if out_float32 else y

    def _attn_lib(self, head_dim: int):
        """The matrix-core attention kernels for this head size, compiled at first use."""
        lib = self._attn_libs.get(head_dim)
        if lib is None:
            name, sources, defines = attention_library_spec(head_dim)
            lib = build.load_library(name, sources, defines)
            _bind(lib, _ATTN_SIGNATURES)
            lib.sia_attn_decode_workspace.restype = ctypes.c_longlong
            if lib.sia_attn_mfma_head_dim() != head_dim:
                raise KernelError(f"library {name} was built for another head size")
            self._attn_libs[head_dim] = lib
        return lib

    # -- helpers -------------------------------------------------------------
    def _stream(self):
        """Handle of torch's current stream on the device (during graph capture: the capturing stream)."""
        if self._raw_stream is not None:
            return self._raw_stream(self._device_index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def _check(self, code: int, what: str):
        if code != 0:
            if code == 10001:
                raise KernelError(f"{what}: the kernel refused its arguments (sizes or types it does not take)")
            raise KernelError(f"{what}: HIP error {code}")

    def _want(self, t: torch.Tensor, what: str, dtype=None, shape=None):
        if t.device.type != "cuda":
            raise KernelError(f"{what} must be on the GPU, is on {t.device}")
        if not t.is_contiguous():
            raise KernelError(f"{what} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{what} must be {dtype}, is {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{what} must have shape {tuple(shape)}, has {tuple(t.shape)}")

    # -- measurement -----------------------------------------------------------
    def measured_read_bandwidth(self, megabytes: int = 2048, repeats: int = 5) -> float:
        """GB/s that a plain streaming read of a buffer far larger than the caches reaches on this card (the best
        of ``repeats``): the ceiling a decode step's reads can be priced against beside the published one."""
        n = int(megabytes) * (1 << 20)
        buf = torch.empty(n, dtype=torch.uint8, device=self.device)
        buf.zero_()
        sink = torch.zeros(1, dtype=torch.int32, device=self.device)
        best = 0.0
        for _ in range(repeats + 1):   # the first run warms up
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            self._check(self.core.sia_stream_read(_ptr(buf), n, _ptr(sink), self._stream()), "stream_read")
            end.record()
            end.synchronize()
            best = max(best, n / (start.elapsed_time(end) * 1e-3) / 1e9)
        return best

    # -- embedding -------------------------------------------------------------
    def place_tokens(self, token_ids, dst_rows, src_tokens, src_rows):
        """``token_ids[dst_rows[i]] = src_tokens[src_rows[i]]`` (all int32, on the device)."""
        for t, what in ((token_ids, "token ids"), (dst_rows, "destination rows"), (src_tokens, "source tokens"),
                        (src_rows, "source rows")):
            self._want(t, what, torch.int32)
        if dst_rows.numel() != src_rows.numel():
            raise KernelError(f"{dst_rows.numel()} destination rows for {src_rows.numel()} source rows")
        self._check(self.core.sia_place_tokens(_ptr(token_ids), _ptr(dst_rows), _ptr(src_tokens), _ptr(src_rows),
                                               dst_rows.numel(), self._stream()), "place_tokens")

    def embed(self, token_ids, table, scale=1.0):
        self._want(token_ids, "token_ids", torch.int32)
        self._want(table, "embedding table")
        if table.dtype not in _DT or table.dim() != 2:
            raise KernelError(f"embedding table must be a float32 or bfloat16 matrix, is {table.dtype} {tuple(table.shape)}")
        n, hidden = token_ids.numel(), table.shape[1]
        out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
        self._check(self.core.sia_embed(_ptr(token_ids), _ptr(table), _ptr(out), n, hidden, _DT[table.dtype],
                                        float(scale), self._stream()), "embed")
        return out

    # -- rms norm of a sublayer's output, added into the residual -------------------
    def norm_add(self, residual, y, weight, eps, out_dtype):
        """``residual += y * rsqrt(mean(y^2) + eps) * weight`` (float); returns the new residual in ``out_dtype``
        (the residual itself if that is float32)."""
        n, hidden = residual.shape
        self._want(residual, "residual", torch.float32)
        self._want(weight, "norm weight", torch.float32, (hidden,))
        if out_dtype not in _DT:
            raise KernelError(f"norm output dtype {out_dtype} is not float32 or bfloat16")
        self._want(y, "sublayer output", out_dtype, (n, hidden))
        lowered = None if out_dtype == torch.float32 else torch.empty((n, hidden), dtype=out_dtype, device=residual.device)
        self._check(self.core.sia_norm_add(_ptr(residual), _ptr(y), _ptr(weight), _ptr(lowered), n, hidden, float(eps),
                                           _DT[out_dtype], self._stream()), "norm_add")
        return residual if lowered is None else lowered

    # -- residual add + rms norm ---------------------------------------------
    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None, gate=None, gate_bias=None,
                    delta_bias=None, terms=None):
        """``residual += delta`` and the RMS norm of the sum.  With ``gate`` (the logits of an elementwise gate:
        ``[n, hidden]``, which may be columns of a wider matrix) the sum is
        ``residual += (delta + delta_bias) * sigmoid(gate + gate_bias)``.  With ``terms`` (``[(tensor, factor)]``, in
        place of ``delta``) the sum is ``residual += sum_i factor_i * tensor_i``; without a ``weight`` only that sum is
        made and nothing returned."""
        n, hidden = residual.shape
        self._want(residual, "residual", torch.float32)
        if terms is not None:
            return self._add_terms(residual, terms, weight, eps, out_dtype, rows)
        self._want(weight, "norm weight", torch.float32, (hidden,))
        if out_dtype not in _DT:
            raise KernelError(f"norm output dtype {out_dtype} is not float32 or bfloat16")
        if gate is not None:
            return self._gated_add(residual, delta, gate, gate_bias, delta_bias, weight, eps, out_dtype, rows)
        if gate_bias is not None or delta_bias is not None:
            raise KernelError("a bias of the gate or of the delta comes with a gate only")
        if delta is not None:
            self._want(delta, "delta", out_dtype, (n, hidden))
        n_out = n
        if rows is not None:
            self._want(rows, "rows", torch.int32)
            n_out = rows.numel()
        out = torch.empty((n_out, hidden), dtype=out_dtype, device=residual.device)
        self._check(self.core.sia_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows),
                                              n_out, hidden, float(eps), _DT[out_dtype], self._stream()),
                    "add_rmsnorm")
        return out

    def _add_terms(self, residual, terms, weight, eps, out_dtype, rows):
        n, hidden = residual.shape
        terms = list(terms)
        if not terms:
            raise KernelError("a sum of scaled terms needs at least one (tensor, factor) pair")
        dtype = terms[0][0].dtype
        if dtype not in _DT or (weight is not None and out_dtype != dtype):
            raise KernelError(f"scaled terms are float32 or bfloat16 and of the norm's output type, got {dtype}")
        for y, _ in terms:
            self._want(y, "scaled term", dtype, (n, hidden))
        if len(terms) > 2:      # the kernel takes two: what is beyond is added up beforehand
            terms = [(self.scaled_sum(terms[:-1]), 1.0), terms[-1]]
        (d1, f1), (d2, f2) = terms[0], (terms[1] if len(terms) > 1 else (None, 0.0))
        n_out, out = n, None
        if rows is not None:
            self._want(rows, "rows", torch.int32)
            n_out = rows.numel()
        if weight is not None:
            self._want(weight, "norm weight", torch.float32, (hidden,))
            out = torch.empty((n_out, hidden), dtype=dtype, device=residual.device)
        elif rows is not None:
            raise KernelError("a sum alone is made over all rows")
        self._check(self.core.sia_add_rmsnorm_scaled(_ptr(residual), _ptr(d1), float(f1), _ptr(d2), float(f2), _ptr(weight),
                                                     _ptr(out), _ptr(rows), n_out, hidden, float(eps), _DT[dtype],
                                                     self._stream()), "add_rmsnorm_scaled")
        return out

    def scaled_sum(self, terms):
        """``sum_i factor_i * tensor_i`` in float, rounded to the tensors' type."""
        terms = list(terms)
        first = terms[0][0]
        if first.dtype not in _DT:
            raise KernelError(f"scaled terms are float32 or bfloat16, got {first.dtype}")
        for y, _ in terms:
            self._want(y, "scaled term", first.dtype, tuple(first.shape))
        total, factor = first, float(terms[0][1])
        rest = terms[1:] or [(None, 0.0)]
        for y, f in rest:
            out = torch.empty_like(first)
            self._check(self.core.sia_scaled_sum(_ptr(total), factor, _ptr(y), float(f), _ptr(out), first.numel(),
                                                 _DT[first.dtype], self._stream()), "scaled_sum")
            total, factor = out, 1.0
        return total

    def gated_add(self, residual, delta, gate=None, gate_bias=None, delta_bias=None):
        """``residual += (delta + delta_bias) * sigmoid(gate + gate_bias)`` and nothing else (without ``gate`` the
        factor is 1)."""
        self._want(residual, "residual", torch.float32)
        self._gated_add(residual, delta, gate, gate_bias, delta_bias, None, 0.0, delta.dtype, None)

    def _columns(self, t, what, dtype, shape):
        """Row stride of a matrix that may be a run of columns of a wider one (elements of a row contiguous)."""
        if t.device.type != "cuda" or t.dtype != dtype or t.dim() != 2 or tuple(t.shape) != tuple(shape):
            raise KernelError(f"{what} must be {dtype} {tuple(shape)} on the GPU, is {t.dtype} {tuple(t.shape)} on {t.device}")
        if t.shape[1] > 1 and t.stride(1) != 1:
            raise KernelError(f"the elements of a row of {what} must be contiguous")
        return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])

    def _gated_add(self, residual, delta, gate, gate_bias, delta_bias, weight, eps, out_dtype, rows):
        n, hidden = residual.shape
        self._want(delta, "delta", out_dtype, (n, hidden))
        stride = self._columns(gate, "gate logits", out_dtype, (n, hidden)) if gate is not None else 0
        for t, what in ((gate_bias, "gate bias"), (delta_bias, "delta bias")):
            if t is not None:
                self._want(t, what, torch.float32, (hidden,))
        n_out, out = n, None
        if rows is not None:
            self._want(rows, "rows", torch.int32)
            n_out = rows.numel()
        if weight is not None:
            out = torch.empty((n_out, hidden), dtype=out_dtype, device=residual.device)
        self._check(self.core.sia_gated_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(delta_bias), _ptr(gate), stride,
                                                    _ptr(gate_bias), _ptr(weight), _ptr(out), _ptr(rows), n_out, hidden,
                                                    float(eps), _DT[out_dtype], self._stream()), "gated_add_rmsnorm")
        return out

    def add_bias(self, y, bias):
        """``y += bias`` over the rows, in place."""
        self._want(y, "rows")
        if y.dtype not in _DT or y.dim() != 2:
            raise KernelError(f"add_bias takes a float32 or bfloat16 matrix, got {y.dtype} {tuple(y.shape)}")
        self._want(bias, "bias", torch.float32, (y.shape[1],))
        self._check(self.core.sia_add_bias(_ptr(y), _ptr(bias), y.shape[0], y.shape[1], _DT[y.dtype], self._stream()),
                    "add_bias")
        return y

    def head_gate(self, out, logits, n_heads):
        """``out[n, h, :] *= sigmoid(logits[n, h])`` in place; ``logits`` may be columns of a wider matrix."""
        self._want(out, "attention output")
        n, width = out.shape
        if out.dtype not in _DT or width % n_heads:
            raise KernelError(f"head gate takes float32 or bfloat16 rows of {n_heads} heads, got {out.dtype} {tuple(out.shape)}")
        stride = self._columns(logits, "head gate logits", out.dtype, (n, n_heads))
        self._check(self.core.sia_head_gate(_ptr(out), _ptr(logits), stride, n, n_heads, width // n_heads,
                                            _DT[out.dtype], self._stream()), "head_gate")
        return out

    def side_by_side(self, a, b, dtype):
        """``[a, b]`` along the columns, lowered to ``dtype``: two float streams as the input of one product."""
        self._want(a, "first stream", torch.float32)
        self._want(b, "second stream", torch.float32, tuple(a.shape))
        if dtype not in _DT or a.dim() != 2:
            raise KernelError(f"side_by_side makes float32 or bfloat16 rows of two matrices, got {dtype} of {tuple(a.shape)}")
        out = torch.empty((a.shape[0], 2 * a.shape[1]), dtype=dtype, device=a.device)
        self._check(self.core.sia_side_by_side(_ptr(a), _ptr(b), _ptr(out), a.shape[0], a.shape[1], _DT[dtype],
                                               self._stream()), "side_by_side")
        return out

    def scale_softcap(self, logits, scale=1.0, cap=None):
        """``logits * scale`` and then, with ``cap``, ``cap * tanh(. / cap)``: in place, float."""
        self._want(logits, "logits", torch.float32)
        if cap is not None and not cap > 0:
            raise KernelError(f"a soft cap must be positive, got {cap}")
        self._check(self.core.sia_scale_softcap(_ptr(logits), logits.numel(), float(scale), float(cap or 0.0),
                                                self._stream()), "scale_softcap")
        return logits

    # -- linear attention with a state ---------------------------------------------
    def gla_recurrent(self, proj, columns, a2, a2_bias, norm_weight, n_heads, key_dim, value_dim, tau, q_scale, eps,
                      ctx, cache):
        """Gated linear attention over the step's runs of tokens, from the projected rows ``proj`` whose column
        offsets ``columns = (q, k, v, g, a)`` name the queries and keys ``[n_heads * key_dim]``, the values and output
        gates ``[n_heads * value_dim]`` and the low-rank decay input ``[rank]``; ``a2 [n_heads * key_dim, rank]``.
        The state ``cache.state [slots, n_heads, key_dim, value_dim]`` (float) is read and left updated.  Returns
        the normed and gated output ``[tokens, n_heads * value_dim]``."""
        self._want(proj, "projected rows")
        n, width = proj.shape
        if proj.dtype not in _DT or n != ctx.n_tokens:
            raise KernelError(f"projected rows {proj.dtype} {tuple(proj.shape)} do not fit a step of {ctx.n_tokens} tokens")
        rank = a2.shape[1]
        self._want(a2, "decay matrix", proj.dtype, (n_heads * key_dim, rank))
        if a2_bias is not None:
            self._want(a2_bias, "decay bias", torch.float32, (n_heads * key_dim,))
        self._want(norm_weight, "output norm weight", torch.float32, (value_dim,))
        q, k, v, g, a = (int(c) for c in columns)
        for first, size, what in ((q, n_heads * key_dim, "q"), (k, n_heads * key_dim, "k"), (v, n_heads * value_dim, "v"),
                                  (g, n_heads * value_dim, "g"), (a, rank, "decay input")):
            if first < 0 or first + size > width:
                raise KernelError(f"columns {first} .. {first + size} of {what} lie outside a row of {width}")
        state = cache.state
        if state is None:
            raise KernelError("gated linear attention needs its state rows")
        self._want(state, "state", torch.float32)
        if tuple(state.shape[1:]) != (n_heads, key_dim, value_dim):
            raise KernelError(f"state rows {tuple(state.shape[1:])} are not [{n_heads}, {key_dim}, {value_dim}]")
        limit = self.core.sia_gla_max_dims()
        if not (0 < key_dim <= limit and 0 < value_dim <= limit):
            raise KernelError(f"head sizes {key_dim} x {value_dim} are outside what the kernel takes (up to {limit})")
        out = torch.empty((n, n_heads * value_dim), dtype=proj.dtype, device=proj.device)
        # float scratch for the decays and, where a prompt's step shares a head's columns out between workgroups, for
        # their raw outputs (kept with the step: its layers run in turn)
        floats = self.core.sia_gla_workspace(n, ctx.n_seqs, ctx.max_q_len, n_heads, key_dim, value_dim)
        workspace = getattr(ctx, "recurrent_workspace", None)
        if workspace is None or workspace.numel() < floats:
            workspace = torch.empty((floats,), dtype=torch.float32, device=proj.device)
            try:
                ctx.recurrent_workspace = workspace
            except AttributeError:
                pass
        self._check(self.core.sia_gla_recurrent(
            _ptr(proj), width, q, k, v, g, a, _ptr(a2), _ptr(a2_bias), _ptr(norm_weight), _ptr(state), _ptr(ctx.cu_q),
            _ptr(ctx.state_slots), _ptr(out), ctx.n_seqs, ctx.max_q_len, n_heads, key_dim, value_dim, rank, float(tau),
            float(q_scale), float(eps), _DT[proj.dtype], _ptr(workspace), n, self._stream()), "gla_recurrent")
        return out

    def check_recurrent_geometry(self, key_dim: int, value_dim: int) -> None:
        limit = self.core.sia_gla_max_dims()
        if not (0 < key_dim <= limit and 0 < value_dim <= limit):
            raise KernelError(f"head sizes {key_dim} x {value_dim} are outside what the recurrent kernel takes (up to {limit})")

    # -- mixture of experts ------------------------------------------------------------
    def moe_route(self, h, router, top, score="softmax", groups=None, scale=1.0, correction=None):
        """The ``top`` experts of every row with the largest router logits ``h @ router^T`` (float; ties go to the
        lower index) and the softmax over their logits alone: ``(ids [n, top] int32, weights [n, top] float32)``.
        ``score="sigmoid"``: the scores are the logits' sigmoids; with ``groups = (count, keep)`` only experts of the
        ``keep`` groups (of ``count`` equal groups of neighbours) whose two largest scores sum highest can be chosen;
        the weights are the chosen scores over their sum, times ``scale``."""
        if score not in ("softmax", "sigmoid", "softmax_all"):
            raise KernelError(f"score must be 'softmax', 'sigmoid' or 'softmax_all', got {score!r}")
        if correction is not None and score != "softmax_all":
            raise KernelError("a correction of the choice comes with scores over all experts")
        if score != "sigmoid" and (groups is not None or scale != 1.0):
            raise KernelError("expert groups and a scale on the weights come with sigmoid scores")
        self._want(h, "router input")
        n, width = h.shape
        experts = router.shape[0]
        self._want(router, "router", torch.float32, (experts, width))
        if h.dtype not in _DT:
            raise KernelError(f"router input must be float32 or bfloat16, is {h.dtype}")
        ids = torch.empty((n, top), dtype=torch.int32, device=h.device)
        weights = torch.empty((n, top), dtype=torch.float32, device=h.device)
        count, keep = (int(groups[0]), int(groups[1])) if groups else (0, 0)
        if groups and (count <= 0 or experts % count or not 0 < keep <= count or top > experts // count * keep):
            raise KernelError(f"{experts} experts in {count} groups of which {keep} are kept cannot give {top}")
        if not 0 < top <= experts:
            raise KernelError(f"top {top} is not between 1 and the number of experts {experts}")
        if score == "softmax_all":
            # scores: the softmax over all experts; the choice goes by score + correction, the weights by the scores
            if correction is not None:
                self._want(correction, "choice correction", torch.float32, (experts,))
            self._check(self.core.sia_moe_route_corrected(_ptr(h), _ptr(router), _ptr(correction), _ptr(ids), _ptr(weights),
                                                          n, width, experts, int(top), _DT[h.dtype], self._stream()),
                        "moe_route")
            return ids, weights
        self._check(self.core.sia_moe_route_ex(_ptr(h), _ptr(router), _ptr(ids), _ptr(weights), n, width, experts,
                                               int(top), _DT[h.dtype], int(score == "sigmoid"), count, keep, float(scale),
                                               self._stream()), "moe_route")
        return ids, weights

    # -- norm without a statistic ---------------------------------------------------------
    def dyt_norm(self, residual, delta, post, pre, out_dtype, rows=None):
        """``x = residual (+ d)`` and ``norm(x)`` by a dynamic tanh, one kernel.  ``d`` is ``delta`` as it is, or with
        ``post = (w, b, alpha, scale | None)`` the norm ``(tanh(alpha * delta) * w + b) * scale`` of it; ``pre`` holds
        the same four terms of the norm whose rows are returned in ``out_dtype`` (None: only the sum is made).
        Without ``rows`` the float residual is left updated; with ``rows`` (int32 indices) only those rows are
        computed and the residual stays as it was."""
        self._want(residual, "residual", torch.float32)
        n, width = residual.shape
        if out_dtype not in _DT:
            raise KernelError(f"the norm's rows are float32 or bfloat16, not {out_dtype}")
        if delta is not None:
            self._want(delta, "delta", out_dtype, (n, width))
        elif pre is None:
            return None
        terms = []
        for t, what in ((post if delta is not None else None, "the delta's norm"), (pre, "norm")):
            if t is None:
                terms += [None, None, None, None]
                continue
            w, b, alpha, scale = t
            self._want(w, f"{what} weight", torch.float32, (width,))
            self._want(b, f"{what} bias", torch.float32, (width,))
            self._want(alpha, f"{what} alpha", torch.float32, (1,))
            if scale is not None:
                self._want(scale, f"{what} scale", torch.float32, (width,))
            terms += [w, b, alpha, scale]
        n_out = n
        if rows is not None:
            self._want(rows, "rows", torch.int32)
            n_out = rows.numel()
        out = torch.empty((n_out, width), dtype=out_dtype, device=residual.device) if pre is not None else None
        self._check(self.core.sia_dyt_norm(_ptr(residual), _ptr(delta), *(_ptr(t) for t in terms), _ptr(out), _ptr(rows),
                                           n_out, width, _DT[out_dtype], self._stream()), "dyt_norm")
        return out

    # -- short convolution and recurrences with a state --------------------------------------
    def _state_rows(self, state, ctx, least):
        if state is None:
            raise KernelError("a mixer with a state needs its state rows")
        self._want(state, "state", torch.float32)
        stride = state[0].numel()
        if stride < least:
            raise KernelError(f"a state row of {stride} floats does not hold {least}")
        return stride

    def _float_workspace(self, ctx, floats, device):
        workspace = getattr(ctx, "recurrent_workspace", None)
        if workspace is None or workspace.numel() < floats:
            workspace = torch.empty((max(int(floats), 1),), dtype=torch.float32, device=device)
            try:
                ctx.recurrent_workspace = workspace
            except AttributeError:
                pass
        return workspace

    def causal_conv(self, proj, first_col, weight, bias, activation, ctx, state, state_offset):
        """A causal convolution per channel over each sequence's tokens: ``out[t, c] = act(bias[c] + sum_j weight[c, j]
        * u[t - (taps - 1) + j, c])`` with ``u`` the columns ``first_col .. first_col + channels - 1`` of ``proj``.  The
        ``taps - 1`` inputs before a step's first token of a sequence are read from the sequence's state row at
        ``state_offset`` (``[taps - 1, channels]`` floats, oldest first) and the row is left holding the last ones."""
        self._want(proj, "projected rows")
        n, width = proj.shape
        channels, taps = weight.shape
        if proj.dtype not in _DT or n != ctx.n_tokens:
            raise KernelError(f"projected rows {proj.dtype} {tuple(proj.shape)} do not fit a step of {ctx.n_tokens} tokens")
        self._want(weight, "convolution weight", torch.float32)
        if bias is not None:
            self._want(bias, "convolution bias", torch.float32, (channels,))
        if activation not in (None, "silu"):
            raise KernelError(f"the convolution's activation is silu or none, not {activation!r}")
        if first_col < 0 or first_col + channels > width:
            raise KernelError(f"columns {first_col} .. {first_col + channels} lie outside a row of {width}")
        stride = self._state_rows(state, ctx, state_offset + channels * (taps - 1))
        out = torch.empty((n, channels), dtype=proj.dtype, device=proj.device)
        self._check(self.core.sia_causal_conv(
            _ptr(proj), width, int(first_col), _ptr(weight), _ptr(bias), _ptr(state), stride, int(state_offset),
            _ptr(ctx.cu_q), _ptr(ctx.seq_of_token), _ptr(ctx.state_slots), _ptr(out), n, ctx.n_seqs, ctx.max_q_len,
            channels, taps, int(activation == "silu"), _DT[proj.dtype], self._stream()), "causal_conv")
        return out

    def ssd_scan(self, proj, xbc, dt_bias, a_log, d_skip, norm_weight, n_heads, head_dim, state_size, groups,
                 norm_groups, eps, ctx, state):
        """The state-space recurrence with a scalar decay per head over the step's runs of tokens.  ``proj`` rows are
        ``[z (heads * head_dim) | ... | dt (heads)]``, ``xbc`` rows ``[x (heads * head_dim) | B (groups * state_size) |
        C (groups * state_size)]``.  ``dt = softplus(dt + dt_bias)``; per head ``S <- exp(-exp(a_log) dt) S + dt B x^T``,
        ``y = S^T C + d_skip x``; the result ``y * silu(z)`` is divided by the root mean square of each of
        ``norm_groups`` equal parts and multiplied by ``norm_weight``.  The matrices ``[heads, state_size, head_dim]``
        are the first floats of a sequence's state row."""
        self._want(proj, "projected rows")
        self._want(xbc, "convolved rows", proj.dtype)
        n, width = proj.shape
        inner = n_heads * head_dim
        if proj.dtype not in _DT or n != ctx.n_tokens or xbc.shape[0] != n:
            raise KernelError(f"rows {proj.dtype} {tuple(proj.shape)} do not fit a step of {ctx.n_tokens} tokens")
        if width < inner + n_heads or xbc.shape[1] != inner + 2 * groups * state_size:
            raise KernelError(f"rows of {width} and {xbc.shape[1]} do not hold {n_heads} heads of {head_dim} with "
                              f"{groups} groups of {state_size}")
        for t, what, size in ((dt_bias, "dt bias", n_heads), (a_log, "decay", n_heads), (d_skip, "skip", n_heads),
                              (norm_weight, "norm weight", inner)):
            self._want(t, what, torch.float32, (size,))
        self.check_recurrent_geometry(state_size, head_dim)
        if n_heads % groups or inner % norm_groups:
            raise KernelError(f"{n_heads} heads of {head_dim} do not split into {groups} groups and {norm_groups} parts")
        stride = self._state_rows(state, ctx, n_heads * state_size * head_dim)
        out = torch.empty((n, inner), dtype=proj.dtype, device=proj.device)
        workspace = self._float_workspace(ctx, self.core.sia_ssd_workspace(n, n_heads, state_size, head_dim), proj.device)
        self._check(self.core.sia_ssd_scan(
            _ptr(proj), width, _ptr(xbc), xbc.shape[1], _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(norm_weight),
            _ptr(state), stride, _ptr(ctx.cu_q), _ptr(ctx.state_slots), _ptr(out), n, ctx.n_seqs, ctx.max_q_len, n_heads,
            head_dim, state_size, groups, norm_groups, float(eps), _DT[proj.dtype], _ptr(workspace), self._stream()),
            "ssd_scan")
        return out

    def hgrn2_scan(self, proj, f_bias, lower, norm_weight, n_heads, key_dim, value_dim, eps, ctx, state):
        """The gated linear recurrence whose forget gate also decides what is written.  ``proj`` rows are ``[q | f | v]``
        (``heads * key_dim``, the same, ``heads * value_dim``) and are used up (the q columns are overwritten).
        ``f = lower + (1 - lower) * sigmoid(f + f_bias)``; per head ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T silu(q)``;
        every head's ``o`` is divided by its root mean square and multiplied by ``norm_weight``.  The state rows are
        ``[heads, key_dim, value_dim]`` floats."""
        self._want(proj, "projected rows")
        n, width = proj.shape
        qk = n_heads * key_dim
        if proj.dtype not in _DT or n != ctx.n_tokens or width != 2 * qk + n_heads * value_dim:
            raise KernelError(f"projected rows {proj.dtype} {tuple(proj.shape)} do not fit {ctx.n_tokens} tokens of "
                              f"{n_heads} heads of {key_dim} and {value_dim}")
        self._want(f_bias, "forget bias", torch.float32, (qk,))
        self._want(lower, "lower bound", torch.float32, (qk,))
        self._want(norm_weight, "output norm weight", torch.float32, (value_dim,))
        self.check_recurrent_geometry(key_dim, value_dim)
        if state is None or tuple(state.shape[1:]) != (n_heads, key_dim, value_dim):
            raise KernelError(f"state rows are not [{n_heads}, {key_dim}, {value_dim}]")
        self._state_rows(state, ctx, qk * value_dim)
        out = torch.empty((n, n_heads * value_dim), dtype=proj.dtype, device=proj.device)
        workspace = self._float_workspace(ctx, self.core.sia_hgrn2_workspace(n, n_heads, key_dim, value_dim), proj.device)
        self._check(self.core.sia_hgrn2_scan(
            _ptr(proj), width, _ptr(f_bias), _ptr(lower), _ptr(norm_weight), _ptr(state), _ptr(ctx.cu_q),
            _ptr(ctx.state_slots), _ptr(out), n, ctx.n_seqs, ctx.max_q_len, n_heads, key_dim, value_dim, float(eps),
            _DT[proj.dtype], _ptr(workspace), self._stream()), "hgrn2_scan")
        return out

    def delta_rule(self, qkv, proj, columns, a_log, dt_bias, norm_weight, n_heads, n_kv_heads, key_dim, value_dim, eps,
                   ctx, state):
        """The gated delta rule over the step's runs of tokens.  ``qkv`` rows are the convolved ``[q (kv_heads *
        key_dim) | k (the same) | v (heads * value_dim)]``; ``columns = (g, b, a)`` name the output gates ``[heads *
        value_dim]``, the write strengths' logits and the step sizes' inputs ``[heads]`` in the rows of ``proj``.  q
        and k are made unit vectors per head (q also times ``key_dim ** -0.5``); ``beta = sigmoid(b)``, ``decay =
        exp(-exp(a_log) * softplus(a + dt_bias))``; per head ``S <- decay S; S += k (beta (v - S^T k))^T; o = S^T q``;
        ``o`` is divided by its root mean square, multiplied by ``norm_weight`` and by ``silu(g)``.  The matrices
        ``[heads, key_dim, value_dim]`` are the first floats of a sequence's state row."""
        self._want(qkv, "convolved rows")
        self._want(proj, "projected rows", qkv.dtype)
        n, width = qkv.shape
        qk, inner = n_kv_heads * key_dim, n_heads * value_dim
        if qkv.dtype not in _DT or n != ctx.n_tokens or proj.shape[0] != n or width != 2 * qk + inner:
            raise KernelError(f"rows {qkv.dtype} {tuple(qkv.shape)} do not fit {ctx.n_tokens} tokens of {n_kv_heads} "
                              f"query/key heads of {key_dim} and {n_heads} value heads of {value_dim}")
        g, b, a = (int(c) for c in columns)
        for first, size, what in ((g, inner, "gate"), (b, n_heads, "write strength"), (a, n_heads, "step size")):
            if first < 0 or first + size > proj.shape[1]:
                raise KernelError(f"columns {first} .. {first + size} of the {what} lie outside a row of {proj.shape[1]}")
        for t, what in ((a_log, "decay rate"), (dt_bias, "step bias")):
            self._want(t, what, torch.float32, (n_heads,))
        self._want(norm_weight, "output norm weight", torch.float32, (value_dim,))
        self.check_recurrent_geometry(key_dim, value_dim)
        if n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise KernelError(f"{n_heads} value heads cannot share {n_kv_heads} query/key heads evenly")
        stride = self._state_rows(state, ctx, n_heads * key_dim * value_dim)
        out = torch.empty((n, inner), dtype=qkv.dtype, device=qkv.device)
        workspace = self._float_workspace(ctx, self.core.sia_delta_rule_workspace(n, n_heads, value_dim), qkv.device)
        self._check(self.core.sia_delta_rule(
            _ptr(qkv), width, _ptr(proj), proj.shape[1], g, b, a, _ptr(a_log), _ptr(dt_bias), _ptr(norm_weight),
            _ptr(state), stride, _ptr(ctx.cu_q), _ptr(ctx.state_slots), _ptr(out), n, ctx.n_seqs, ctx.max_q_len, n_heads,
            n_kv_heads, key_dim, value_dim, float(eps), _DT[qkv.dtype], _ptr(workspace), self._stream()), "delta_rule")
        return out

    def decay_attention(self, proj, decays, norm_weight, n_heads, key_dim, value_dim, eps, ctx, state):
        """Linear attention with a constant decay per head.  ``proj`` rows are ``[q | k (heads * key_dim each) | v | g
        (heads * value_dim each)]`` and are used up (q, k and v are overwritten by their ``silu``).  Per head ``S <-
        decays[h] S + k v^T``, ``o = S^T q``; the row of all heads' ``o`` is divided by its root mean square, multiplied
        by ``norm_weight [heads * value_dim]`` and by ``sigmoid(g)``.  The state rows are ``[heads, key_dim,
        value_dim]`` floats."""
        self._want(proj, "projected rows")
        n, width = proj.shape
        qk, inner = n_heads * key_dim, n_heads * value_dim
        if proj.dtype not in _DT or n != ctx.n_tokens or width != 2 * qk + 2 * inner:
            raise KernelError(f"projected rows {proj.dtype} {tuple(proj.shape)} do not fit {ctx.n_tokens} tokens of "
                              f"{n_heads} heads of {key_dim} and {value_dim}")
        self._want(decays, "decays", torch.float32, (n_heads,))
        self._want(norm_weight, "output norm weight", torch.float32, (inner,))
        self.check_recurrent_geometry(key_dim, value_dim)
        if state is None or tuple(state.shape[1:]) != (n_heads, key_dim, value_dim):
            raise KernelError(f"state rows are not [{n_heads}, {key_dim}, {value_dim}]")
        self._state_rows(state, ctx, qk * value_dim)
        out = torch.empty((n, inner), dtype=proj.dtype, device=proj.device)
        workspace = self._float_workspace(
            ctx, self.core.sia_gla_workspace(n, ctx.n_seqs, ctx.max_q_len, n_heads, key_dim, value_dim), proj.device)
        self._check(self.core.sia_decay_attention(
            _ptr(proj), width, _ptr(decays), _ptr(norm_weight), _ptr(state), _ptr(ctx.cu_q), _ptr(ctx.state_slots),
            _ptr(out), n, ctx.n_seqs, ctx.max_q_len, n_heads, key_dim, value_dim, float(eps), _DT[proj.dtype],
            _ptr(workspace), self._stream()), "decay_attention")
        return out

    # -- latent attention ---------------------------------------------------------------------
    def _rotation_tables(self, rotary_dim, cos, sin, ctx_or_len):
        if not rotary_dim:
            return None, None
        for t, what in ((cos, "cos table"), (sin, "sin table")):
            self._want(t, what, torch.float32)
            if t.shape[1] != rotary_dim // 2 or t.shape[0] <= ctx_or_len - 1:
                raise KernelError(f"{what} {tuple(t.shape)} does not cover position {ctx_or_len - 1} with "
                                  f"{rotary_dim // 2} pairs")
        return cos, sin

    def latent_prepare(self, proj, q_rank, q_gain, kv_rank, kv_gain, rot_dim, rotary_dim, cos, sin, eps, ctx, cache,
                       page_dim=None):
        """From projected rows ``[a_q (q_rank) | a (kv_rank) | b (rot_dim)]``: returns ``rms(a_q) * q_gain`` and, if
        ``kv_rank`` is not 0, writes ``[rms(a) * kv_gain | rotate(b)]`` as the position's key row and ``rms(a) *
        kv_gain`` as its value into the pages (one key/value head; rows ``page_dim`` wide if given).  The rotation
        turns neighbouring pairs of the first ``rotary_dim`` elements of ``b``."""
        self._want(proj, "projected rows")
        n, width = proj.shape
        if proj.dtype not in _DT or n != ctx.n_tokens or width != q_rank + (kv_rank + rot_dim if kv_rank else 0):
            raise KernelError(f"projected rows {proj.dtype} {tuple(proj.shape)} do not fit {ctx.n_tokens} tokens of "
                              f"{q_rank} + {kv_rank} + {rot_dim} columns")
        self._want(q_gain, "query latent gain", torch.float32, (q_rank,))
        cq = torch.empty((n, q_rank), dtype=proj.dtype, device=proj.device)
        table = k_pages = v_pages = None
        page_size = key_width = value_rows = 0
        if kv_rank:
            self._want(kv_gain, "latent gain", torch.float32, (kv_rank,))
            cos, sin = self._rotation_tables(rotary_dim, cos, sin, ctx.max_kv_len)
            key_width = page_dim or (kv_rank + rot_dim)
            value_rows = page_dim or kv_rank
            k_pages, v_pages, table, page_size = cache.k_pages, cache.v_pages, cache.block_table, cache.page_size
            self._check_pages(k_pages, v_pages, table, page_size, 1, key_width, proj.dtype, ctx, value_rows)
        self._check(self.core.sia_latent_prepare(
            _ptr(proj), width, q_rank, _ptr(q_gain), kv_rank, _ptr(kv_gain), rot_dim, rotary_dim if kv_rank else 0,
            _ptr(cos) if kv_rank else None, _ptr(sin) if kv_rank else None, float(eps), _ptr(ctx.positions),
            _ptr(ctx.seq_of_token), _ptr(table), table.shape[1] if table is not None else 0, _ptr(k_pages),
            _ptr(v_pages), page_size, key_width, value_rows, _ptr(cq), n, _DT[proj.dtype], self._stream()),
            "latent_prepare")
        return cq

    def headwise_linear(self, x, w, in_stride, out_stride, tail=0, rotation=None):
        """A product per head: ``y[n, h, :out] = w[h] x[n, h, :in]`` for ``w [heads, out, in]``, ``x`` rows holding
        ``in_stride`` elements a head and ``y`` rows ``out_stride``.  The ``tail`` elements behind a head's inputs are
        copied behind its outputs, their first ``rotary_dim`` elements turned in neighbouring pairs by ``rotation =
        (rotary_dim, cos, sin, positions)``; what is left of a head's ``out_stride`` is zero."""
        self._want(x, "headwise input")
        self._want(w, "headwise weights", x.dtype)
        if x.dtype not in _DT or w.dim() != 3:
            raise KernelError(f"a product per head takes float32 or bfloat16 rows and weights [heads, out, in]")
        n, width = x.shape
        heads, out_dim, in_dim = w.shape
        if width != heads * in_stride or in_dim + tail > in_stride or out_dim + tail > out_stride:
            raise KernelError(f"rows of {width} do not hold {heads} heads of {in_stride}, or {in_dim} + {tail} inputs and "
                              f"{out_dim} + {tail} outputs do not fit strides {in_stride} and {out_stride}")
        rotary_dim, cos, sin, positions = rotation if (rotation is not None and tail) else (0, None, None, None)
        if rotary_dim:
            if rotary_dim > tail or rotary_dim % 2:
                raise KernelError(f"a rotation of {rotary_dim} elements does not fit a tail of {tail}")
            self._want(positions, "positions", torch.int32, (n,))
            for t, what in ((cos, "cos table"), (sin, "sin table")):
                self._want(t, what, torch.float32)
                if t.shape[1] != rotary_dim // 2:
                    raise KernelError(f"{what} {tuple(t.shape)} does not hold {rotary_dim // 2} pairs")
        y = torch.empty((n, heads * out_stride), dtype=x.dtype, device=x.device)
        self._check(self.core.sia_headwise_linear(
            _ptr(x), width, in_stride, _ptr(w), _ptr(y), heads * out_stride, out_stride, n, heads, in_dim, out_dim,
            int(tail), int(rotary_dim), _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None,
            _ptr(positions) if rotary_dim else None, _DT[x.dtype], self._stream()), "headwise_linear")
        return y

    @staticmethod
    def _glu(activation):
        """(kind, limit) of a gated activation as the kernels take it: None is ``silu(g) * u``, ``("clamped", limit)`` is
        ``g * sigmoid(1.702 g) * (u + 1)`` with ``g = min(g, limit)`` and ``u = clamp(u, -limit, limit)``."""
        if activation is None:
            return _GLUS["silu"], 0.0
        kind, limit = activation
        if kind not in _GLUS or not float(limit) > 0:
            raise KernelError(f"gated activation {activation!r} is not one of {', '.join(_GLUS)} with a positive limit")
        return _GLUS[kind], float(limit)

    def moe_experts(self, h, w_gate_up, w_down, ids, weights, shared=None, shared_gate=None, activation=None,
                    identity=0):
        """``sum_k weights[n, k] * expert_{ids[n, k]}(h[n])`` with ``expert_e(x) = W2_e (silu(Wg_e x) * (Wu_e x))``,
        ``w_gate_up [E, 2 ff, width]`` (gate rows first), ``w_down [E, width, ff]``; plus ``shared`` ``[n, width]``
        (times ``sigmoid(shared_gate [n, 1])`` if given), the sum rounded once.  ``activation``: another gated
        activation than ``silu(g) * u`` (see ``_glu``); ``identity``: ids ``E .. E + identity - 1`` name experts
        without tensors, which return their input."""
        glu, limit = self._glu(activation)
        self._want(h, "expert input")
        n, width = h.shape
        experts, two_ff, _ = w_gate_up.shape
        ff, top = two_ff // 2, ids.shape[1]
        self._want(w_gate_up, "expert gate/up weights", h.dtype, (experts, 2 * ff, width))
        self._want(w_down, "expert down weights", h.dtype, (experts, width, ff))
        self._want(ids, "expert ids", torch.int32, (n, top))
        self._want(weights, "expert weights", torch.float32, (n, top))
        if h.dtype not in _DT:
            raise KernelError(f"expert input must be float32 or bfloat16, is {h.dtype}")
        gate_stride = 0
        if shared is not None:
            self._want(shared, "shared expert output", h.dtype, (n, width))
            if shared_gate is not None:
                gate_stride = self._columns(shared_gate, "shared expert gate", h.dtype, (n, 1))
        elif shared_gate is not None:
            raise KernelError("a shared expert's gate comes with its output")
        act = torch.empty((n * top, ff), dtype=h.dtype, device=h.device)
        out = torch.empty((n, width), dtype=h.dtype, device=h.device)
        ints = self.core.sia_moe_tiled_workspace(n, top, experts, width, ff) if (
            self.tiled_experts and h.dtype == torch.bfloat16) else 0
        if ints:
            workspace = torch.empty((ints,), dtype=torch.int32, device=h.device)
            y = torch.empty((n * top, width), dtype=h.dtype, device=h.device)
            self._check(self.core.sia_moe_tiled_ex(
                _ptr(h), _ptr(w_gate_up), _ptr(w_down), _ptr(ids), _ptr(weights), _ptr(shared), _ptr(shared_gate),
                gate_stride, _ptr(act), _ptr(y), _ptr(out), _ptr(workspace), n, width, ff, top, experts, glu, limit,
                self._stream()), "moe_tiled")
            return out
        self._check(self.core.sia_moe_gate_up_ex(_ptr(h), _ptr(w_gate_up), _ptr(ids), _ptr(act), n, width, ff, top,
                                                 experts, glu, limit, _DT[h.dtype], self._stream()), "moe_gate_up")
        self._check(self.core.sia_moe_down_ex(_ptr(act), _ptr(w_down), _ptr(ids), _ptr(weights), _ptr(shared),
                                              _ptr(shared_gate), gate_stride, _ptr(out), n, width, ff, top, _ptr(h),
                                              experts, _DT[h.dtype], self._stream()), "moe_down")
        return out

    # -- matrix product --------------------------------------------------------
    def linear(self, x, w, out_float32=False):
        """``x [M, K] @ w [N, K]^T`` with float accumulation."""
        x = self.finish_rows(x)
        self._want(x, "linear input")
        self._want(w, "linear weight")
        if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
            raise KernelError(f"linear shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}")
        if x.dtype not in _DT or w.dtype not in _DT:
            raise KernelError(f"linear takes float32 or bfloat16, got {x.dtype} and {w.dtype}")
        M, K = x.shape
        N = w.shape[0]
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
            # up to 16 rows: this package's kernel, whose sums do not depend on the number of rows
            if self.use_skinny_gemm and M <= self._skinny_rows and K % 64 == 0:
                y = torch.empty((M, N), dtype=torch.float32 if out_float32 else torch.bfloat16, device=x.device)
                tiled = None if out_float32 else self._tiled_copy(w)
                if tiled is not None:   # a weight that has a copy in the order of this kernel's loads: the same bits
                    self._check(self.core.sia_gemm_skinny_tiled(_ptr(x), _ptr(tiled), _ptr(y), M, N, K, self._stream()),
                                "gemm_skinny_tiled")
                    return y
                self._check(self.core.sia_gemm_skinny(_ptr(x), _ptr(w), _ptr(y), M, N, K, int(out_float32),
                                                      self._stream()), "gemm_skinny")
                return y
            return self._library_product(x, w, out_float32)
        # True 32-bit product.  A float32-stored matrix meeting bfloat16 activations widens them.
        back = None
        if x.dtype == torch.bfloat16:
            back = torch.bfloat16
            x = self.cast(x, torch.float32)
        if w.dtype == torch.bfloat16:
            w = self.cast(w, torch.float32)
        y = torch.empty((M, N), dtype=torch.float32, device=x.device)
        self._check(self.core.sia_gemm_generic(_ptr(x), _ptr(w), _ptr(y), M, N, K, 0, 1, self._stream()),
                    "gemm_generic")
        if back is not None and not out_float32:
            y = self.cast(y, back)
        return y

    def gated_linear(self, x, w_gate_up, activation=None):
        """``silu(x Wg^T) * (x Wu^T)`` for ``w_gate_up = [Wg; Wu]``: one kernel for few rows, else product + SwiGLU.
        ``activation``: another gated activation (see ``_glu``), by the product and a kernel of its own."""
        self._want(w_gate_up, "gate/up weight")
        M, K = x.shape
        two_i = w_gate_up.shape[0]
        if activation is not None:
            glu, limit = self._glu(activation)
            if (self.use_skinny_gemm and x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
                    and M <= self._skinny_rows and two_i % 2 == 0 and K % 64 == 0 and w_gate_up.shape[1] == K):
                rows, partials, n_partials, eps = self._scaled(x)      # few rows: the activation inside the product
                self._want(rows, "gated linear input")
                y = torch.empty((M, two_i // 2), dtype=torch.bfloat16, device=rows.device)
                self._check(self.core.sia_gemm_skinny_glu(_ptr(rows), _ptr(w_gate_up), _ptr(y), M, two_i // 2, K,
                                                          _ptr(partials), n_partials, eps, glu, limit, self._stream()),
                            "gemm_skinny_glu")
                return y
            gu = self.linear(x, w_gate_up)
            if gu.dtype not in _DT or two_i % 2:
                raise KernelError(f"a gated activation takes [tokens, 2 * intermediate] rows, got {gu.dtype} {tuple(gu.shape)}")
            out = torch.empty((M, two_i // 2), dtype=gu.dtype, device=gu.device)
            for n0 in range(0, M, 65535):
                n1 = min(M, n0 + 65535)
                self._check(self.core.sia_glu(_ptr(gu[n0:n1]), _ptr(out[n0:n1]), n1 - n0, two_i // 2, glu, limit,
                                              _DT[gu.dtype], self._stream()), "glu")
            return out
        if (self.use_skinny_gemm and x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
                and M <= self._skinny_rows and two_i % 2 == 0 and K % 64 == 0 and w_gate_up.shape[1] == K):
            rows, partials, n_partials, eps = self._scaled(x)
            self._want(rows, "gated linear input")
            y = torch.empty((M, two_i // 2), dtype=torch.bfloat16, device=rows.device)
            self._check(self.core.sia_gemm_skinny_swiglu(_ptr(rows), _ptr(w_gate_up), _ptr(y), M, two_i // 2, K,
                                                         _ptr(partials), n_partials, eps, self._stream()),
                        "gemm_skinny_swiglu")
            return y
        return self.swiglu(self.linear(x, w_gate_up))

    def activated_linear(self, x, w, activation):
        """``act(x @ w^T)`` for an activation without a gate (``relu2``, ``gelu_tanh``): one kernel for few rows,
        else the product and the activation."""
        if activation not in _ACTIVATIONS:
            raise KernelError(f"activation {activation!r} is not one of {', '.join(_ACTIVATIONS)}")
        x = self.finish_rows(x)
        self._want(x, "linear input")
        self._want(w, "linear weight")
        if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
            raise KernelError(f"linear shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}")
        M, K = x.shape
        N = w.shape[0]
        if (self.use_skinny_gemm and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
                and 0 < M <= self._skinny_rows and K % 64 == 0):
            y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            self._check(self.core.sia_gemm_skinny_act(_ptr(x), _ptr(w), _ptr(y), M, N, K, _ACTIVATIONS[activation],
                                                      self._stream()), "gemm_skinny_act")
            return y
        return self.activation(self.linear(x, w), activation)

    def activation(self, z, activation):
        self._want(z, "activation input")
        if z.dtype not in _DT:
            raise KernelError(f"activation takes float32 or bfloat16, got {z.dtype}")
        out = torch.empty_like(z)
        self._check(self.core.sia_activation(_ptr(z), _ptr(out), z.numel(), _ACTIVATIONS[activation], _DT[z.dtype],
                                             self._stream()), "activation")
        return out

    # -- a product whose result goes into the residual, and the norm after it ---------
    def pending_linear(self, x, w):
        """``linear(x, w)`` as the last product of a part.  For few rows in bfloat16 it is not computed yet: the norm
        that follows has it computed by ``linear_into_residual``, which saves the norm's own kernel."""
        if (self.use_skinny_gemm and self.fuse_norms and isinstance(x, torch.Tensor) and x.dim() == 2 and w.dim() == 2
                and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] == w.shape[1]
                and 0 < x.shape[0] <= self._skinny_rows and w.shape[1] % 64 == 0):
            return PendingProduct(x, w, self)
        return self.linear(x, w)

    def linear_into_residual(self, pending, residual, gain, eps):
        """``residual += x @ w^T`` (the product rounded to bfloat16 first, as ``linear`` rounds it) and the rows of
        the RMS norm of the sum as ``ScaledRows``."""
        x, w = pending.x, pending.w
        self._want(x, "linear input", torch.bfloat16)
        self._want(w, "linear weight", torch.bfloat16)
        self._want(residual, "residual", torch.float32)
        self._want(gain, "norm weight", torch.float32)
        M, K = x.shape
        N = w.shape[0]
        if (w.shape[1] != K or tuple(residual.shape) != (M, N) or tuple(gain.shape) != (N,) or M > self._skinny_rows
                or K % 64):
            raise KernelError(f"product into the residual does not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, "
                              f"residual {tuple(residual.shape)}, gain {tuple(gain.shape)}")
        rows = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        partials = torch.empty((self.core.sia_gemm_skinny_residual_blocks(N), 16), dtype=torch.float32, device=x.device)
        tiled = self._tiled_copy(w)
        if tiled is not None:
            self._check(self.core.sia_gemm_skinny_residual_tiled(_ptr(x), _ptr(tiled), M, N, K, _ptr(residual),
                                                                 _ptr(gain), _ptr(rows), _ptr(partials), self._stream()),
                        "gemm_skinny_residual_tiled")
        else:
            self._check(self.core.sia_gemm_skinny_residual(_ptr(x), _ptr(w), M, N, K, _ptr(residual), _ptr(gain),
                                                           _ptr(rows), _ptr(partials), self._stream()),
                        "gemm_skinny_residual")
        return ScaledRows(rows, partials, float(eps))

    # A weight whose product goes into the residual in steps of few rows may have a second copy, laid out in the
    # order in which that kernel's workgroups read it (every load instruction one run of memory: the o and down
    # products of a decode step take 10 to 15 % less).  The copy hangs on the weight tensor itself, so it lives as long
    # as the weight does, and remembers the version of the tensor it was made from: a weight changed in place since
    # is read as it is.  Steps of more rows, which go to the library, read the weight as it is anyway.
    def prepare_pending_weight(self, w) -> bool:
        """Makes the tiled copy of a weight that ``pending_linear`` will be given; True if one was made."""
        if (not self.tiled_weights or not isinstance(w, torch.Tensor) or w.dim() != 2 or w.dtype != torch.bfloat16
                or not w.is_cuda or not w.is_contiguous() or w.shape[1] % 64 or torch.cuda.is_current_stream_capturing()):
            return False
        N, K = w.shape
        height = self.core.sia_gemm_skinny_tile_height(N)
        if height <= 0:
            return False
        blocks = -(-N // height)
        rows = torch.arange(blocks * height, device=w.device).clamp_(max=N - 1)   # the last block repeats the last row
        # element (block, step, half, row, lane group, e) = W[block * height + row][64 step + 16 group + 8 half + e]
        tiled = w[rows].view(blocks, height, K // 64, 4, 2, 8).permute(0, 2, 4, 1, 3, 5).contiguous()
        w._sia_tiled = (tiled, w._version)
        return True

    def _tiled_copy(self, w):
        kept = getattr(w, "_sia_tiled", None) if self.tiled_weights else None
        if kept is None or kept[1] != w._version:
            return None
        return kept[0]

    @staticmethod
    def _scaled(x):
        """(rows, partials, n_partials, eps) of an input that may be ``ScaledRows``."""
        if isinstance(x, ScaledRows):
            return x.rows, x.partials, x.partials.shape[0], x.eps
        return x, None, 0, 0.0

    def finish_rows(self, x):
        """The tensor that ``ScaledRows`` stand for (a tensor is returned as it is)."""
        if not isinstance(x, ScaledRows):
            return x
        out = torch.empty_like(x.rows)
        self._check(self.core.sia_scale_rows(_ptr(x.rows), _ptr(x.partials), _ptr(out), x.rows.shape[0],
                                             x.rows.shape[1], x.partials.shape[0], x.eps, self._stream()),
                    "scale_rows")
        return out

    def gemm_generic(self, x, w, out_float32=False):
        """The plain kernel for either dtype (tests compare it with the library product)."""
        self._want(x, "gemm input")
        self._want(w, "gemm weight", x.dtype)
        M, K = x.shape
        N = w.shape[0]
        out_dtype = torch.float32 if (out_float32 or x.dtype == torch.float32) else x.dtype
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        self._check(self.core.sia_gemm_generic(_ptr(x), _ptr(w), _ptr(y), M, N, K, _DT[x.dtype],
                                               int(out_dtype == torch.float32), self._stream()), "gemm_generic")
        return y

    def cast(self, x, dtype):
        self._want(x, "cast input")
        if x.dtype == dtype:
            return x
        if {x.dtype, dtype} != {torch.float32, torch.bfloat16}:
            raise KernelError(f"cast is between float32 and bfloat16 only, got {x.dtype} -> {dtype}")
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
        self._check(self.core.sia_cast(_ptr(x), _ptr(out), x.numel(), _DT[x.dtype], self._stream()), "cast")
        return out

    # -- feed-forward activation ---------------------------------------------
    def swiglu(self, gu):
        self._want(gu, "swiglu input")
        if gu.dtype not in _DT or gu.dim() != 2 or gu.shape[1] % 2:
            raise KernelError(f"swiglu takes a [tokens, 2*intermediate] float32/bfloat16 matrix, got {gu.dtype} {tuple(gu.shape)}")
        n, two_i = gu.shape
        out = torch.empty((n, two_i // 2), dtype=gu.dtype, device=gu.device)
        for n0 in range(0, n, 65535):  # grid.y limit
            n1 = min(n, n0 + 65535)
            self._check(self.core.sia_swiglu(_ptr(gu[n0:n1]), _ptr(out[n0:n1]), n1 - n0, two_i // 2,
                                             _DT[gu.dtype], self._stream()), "swiglu")
        return out

    # -- rotation + cache write ------------------------------------------------
    def rope_kv_write(self, qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache):
        self._want(qkv, "qkv")
        n, width = qkv.shape
        if qkv.dtype not in _DT:
            raise KernelError(f"qkv must be float32 or bfloat16, is {qkv.dtype}")
        if width != (n_heads + 2 * n_kv_written) * head_dim:
            raise KernelError(f"qkv row of {width} does not hold {n_heads} + 2*{n_kv_written} heads of {head_dim}")
        if n != ctx.n_tokens:
            raise KernelError(f"qkv has {n} rows, the step {ctx.n_tokens} tokens")
        if rotary_dim:
            for t, what in ((cos, "cos table"), (sin, "sin table")):
                self._want(t, what, torch.float32)
                if t.shape[1] != rotary_dim // 2 or t.shape[0] <= ctx.max_kv_len - 1:
                    raise KernelError(f"{what} {tuple(t.shape)} does not cover position {ctx.max_kv_len - 1} "
                                      f"with {rotary_dim // 2} pairs")
        table = table_w = k_pages = v_pages = None
        page_size = 0
        if n_kv_written:
            k_pages, v_pages, table, page_size = cache.k_pages, cache.v_pages, cache.block_table, cache.page_size
            self._check_pages(k_pages, v_pages, table, page_size, n_kv_written, head_dim, qkv.dtype, ctx)
        table_w = table.shape[1] if table is not None else 0
        self._check(self.core.sia_rope_kv_write(
            _ptr(qkv), width, _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None,
            _ptr(ctx.positions), _ptr(ctx.seq_of_token), _ptr(table), table_w, _ptr(k_pages), _ptr(v_pages),
            n, n_heads, n_kv_written, head_dim, rotary_dim, page_size, _DT[qkv.dtype], self._stream()),
            "rope_kv_write")

    def qkv_to_cache(self, x, w_qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache,
                     value_dim=None, bias=None, qk_norm=None, page_dim=None, q_temp=None, extra_columns=0,
                     values_are_keys=False):
        """The q/k/v product, the rotation of q and k and the write of k and v into the pages.  Returns the
        ``[tokens, (n_heads + 2 n_kv_written) head_dim]`` matrix whose q columns hold the rotated queries; its
        k and v columns are not to be read (for few rows one kernel does all three and never writes them).

        ``value_dim``: width of a v head if not ``head_dim``; ``bias``: float ``[row width]``, added to the product;
        ``qk_norm``: ``(q_gain, k_gain, eps)``, an RMS norm over every q and k head before the rotation.  With any
        of these the product is followed by one kernel that does all of bias, norm, rotation and cache write.

        ``page_dim`` (see ``attention_page_dim``): the pages' keys and values are both that wide; the result is then
        ``[tokens, n_heads * page_dim]``, the queries with zeros behind every head, and attention is called with
        ``page_dim`` for the head size.

        ``q_temp``: ``(coef, every)``, every query is multiplied by ``1 + coef * ln(floor((pos + 1) / every) + 1)``
        after its norm.  ``extra_columns``: the weight has that many further rows behind v, whose products are only
        carried along; the result is then the pair (that matrix, the further columns of the projected rows).
        ``values_are_keys``: the weight has no v rows; a position's values are its keys as projected (with their bias,
        before norm and rotation)."""
        M, K = x.shape
        if (value_dim is not None or bias is not None or qk_norm is not None or page_dim is not None
                or q_temp is not None or extra_columns or values_are_keys):
            qkv = self.linear(x, w_qkv)
            q_out = None
            if page_dim is not None:
                # one matrix a step and geometry, shared by the step's layers: its zeros between the heads are written
                # once, the kernel only ever writes the heads' own elements
                kept = getattr(ctx, "padded_queries", None)
                if kept is None:
                    kept = ctx.padded_queries = {}
                key = (n_heads, page_dim, qkv.dtype)
                q_out = kept.get(key)
                if q_out is None:
                    q_out = kept[key] = torch.zeros((M, n_heads * page_dim), dtype=qkv.dtype, device=qkv.device)
            self.qk_prepare(qkv, n_heads, n_kv_written, head_dim, value_dim or head_dim, rotary_dim, cos, sin, bias,
                            qk_norm, ctx, cache, page_dim, q_out, q_temp, extra_columns, values_are_keys)
            queries = qkv if q_out is None else q_out
            if extra_columns:
                return queries, qkv[:, qkv.shape[1] - extra_columns:]
            return queries
        if (self.use_skinny_gemm and self.fuse_rope and n_kv_written and x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16
                and M <= self._skinny_rows and rotary_dim == head_dim and head_dim % 2 == 0 and K % 64 == 0):
            x, partials, n_partials, norm_eps = self._scaled(x)
            self._want(x, "q/k/v input")
            self._want(w_qkv, "q/k/v weight")
            width = (n_heads + 2 * n_kv_written) * head_dim
            if tuple(w_qkv.shape) != (width, K):
                raise KernelError(f"q/k/v weight {tuple(w_qkv.shape)} is not [{width}, {K}]")
            if M != ctx.n_tokens:
                raise KernelError(f"q/k/v input has {M} rows, the step {ctx.n_tokens} tokens")
            for t, what in ((cos, "cos table"), (sin, "sin table")):
                self._want(t, what, torch.float32)
                if t.shape[1] != rotary_dim // 2 or t.shape[0] <= ctx.max_kv_len - 1:
                    raise KernelError(f"{what} {tuple(t.shape)} does not cover position {ctx.max_kv_len - 1} "
                                      f"with {rotary_dim // 2} pairs")
            self._check_pages(cache.k_pages, cache.v_pages, cache.block_table, cache.page_size, n_kv_written,
                              head_dim, x.dtype, ctx)
            qkv = torch.empty((M, width), dtype=torch.bfloat16, device=x.device)
            self._check(self.core.sia_gemm_skinny_rope(
                _ptr(x), _ptr(w_qkv), _ptr(qkv), M, K, _ptr(cos), _ptr(sin), _ptr(ctx.positions),
                _ptr(ctx.seq_of_token), _ptr(cache.block_table), cache.block_table.shape[1], _ptr(cache.k_pages),
                _ptr(cache.v_pages), n_heads, n_kv_written, head_dim, cache.page_size, _ptr(partials), n_partials,
                norm_eps, self._stream()),
                "gemm_skinny_rope")
            return qkv
        qkv = self.linear(x, w_qkv)
        self.rope_kv_write(qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache)
        return qkv

    def attention_page_dim(self, head_dim: int, value_dim: int, dtype):
        """The one width at which a mixer should keep both its keys and its values in the pages so that the
        matrix-core attention kernel, which is compiled for one head size, can run on them; None where the pages can
        be as wide as the heads are (the widths are alike and a multiple of 16, or no such kernel would run
        anyway).  The elements beyond a head's own are zero: a zero in a key adds nothing to a score, a zero row of
        values gives a zero that the output projection, widened by as many zero columns, ignores."""
        if dtype != torch.bfloat16:
            return None
        wide = -(-max(head_dim, value_dim) // 16) * 16
        if (wide == head_dim and wide == value_dim) or wide > 256:
            return None
        return wide

    def qk_prepare(self, qkv, n_heads, n_kv_written, head_dim, value_dim, rotary_dim, cos, sin, bias, qk_norm, ctx,
                   cache, page_dim=None, q_out=None, q_temp=None, extra_columns=0, values_are_keys=False):
        """Bias, per-head RMS norm of q and k, rotation, and the write of k and v into the pages, on the projected
        rows ``[q heads | k heads | v heads]`` (q and k heads ``head_dim`` wide, v heads ``value_dim``); q is left in
        place."""
        self._want(qkv, "qkv")
        n, width = qkv.shape
        if qkv.dtype not in _DT:
            raise KernelError(f"qkv must be float32 or bfloat16, is {qkv.dtype}")
        if values_are_keys and (value_dim != head_dim or extra_columns):
            raise KernelError("values that are the keys have the keys' width, and nothing rides behind them")
        own = n_heads * head_dim + n_kv_written * (head_dim + (0 if values_are_keys else value_dim))
        if width != own + extra_columns:
            raise KernelError(f"qkv row of {width} does not hold {n_heads} q heads and {n_kv_written} k heads of "
                              f"{head_dim}, as many v heads of {value_dim} and {extra_columns} further columns")
        if n != ctx.n_tokens:
            raise KernelError(f"qkv has {n} rows, the step {ctx.n_tokens} tokens")
        if not 0 < head_dim <= self.core.sia_qk_prepare_max_head_dim():
            raise KernelError(f"head size {head_dim} is outside what the kernel takes")
        if rotary_dim:
            for t, what in ((cos, "cos table"), (sin, "sin table")):
                self._want(t, what, torch.float32)
                if t.shape[1] != rotary_dim // 2 or t.shape[0] <= ctx.max_kv_len - 1:
                    raise KernelError(f"{what} {tuple(t.shape)} does not cover position {ctx.max_kv_len - 1} "
                                      f"with {rotary_dim // 2} pairs")
        if bias is not None:
            self._want(bias, "q/k/v bias", torch.float32, (own,))
        temp_coef, temp_every = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else (0.0, 0)
        if q_temp is not None and temp_every <= 0:
            raise KernelError(f"a query temperature steps every so many positions, got {temp_every}")
        q_gain = k_gain = None
        eps = 0.0
        if qk_norm is not None:
            q_gain, k_gain, eps = qk_norm
            self._want(q_gain, "q norm gain", torch.float32, (head_dim,))
            self._want(k_gain, "k norm gain", torch.float32, (head_dim,))
        table = k_pages = v_pages = None
        page_size = 0
        k_row, v_rows = head_dim, value_dim
        if page_dim is not None:
            if page_dim < max(head_dim, value_dim) or q_out is None:
                raise KernelError(f"pages of width {page_dim} do not hold heads of {head_dim} and values of {value_dim}")
            self._want(q_out, "padded queries", qkv.dtype, (n, n_heads * page_dim))
            k_row = v_rows = page_dim
        if n_kv_written:
            k_pages, v_pages, table, page_size = cache.k_pages, cache.v_pages, cache.block_table, cache.page_size
            self._check_pages(k_pages, v_pages, table, page_size, n_kv_written, k_row, qkv.dtype, ctx, v_rows)
        self._check(self.core.sia_qk_prepare_ex(
            _ptr(qkv), width, _ptr(bias), _ptr(q_gain), _ptr(k_gain), float(eps),
            _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None, _ptr(ctx.positions),
            _ptr(ctx.seq_of_token), _ptr(table), table.shape[1] if table is not None else 0, _ptr(k_pages),
            _ptr(v_pages), n, n_heads, n_kv_written, head_dim, value_dim, rotary_dim, page_size, k_row, v_rows,
            _ptr(q_out), n_heads * page_dim if page_dim else 0, page_dim or 0, temp_coef, temp_every,
            int(bool(values_are_keys)), _DT[qkv.dtype], self._stream()), "qk_prepare")

    def _check_pages(self, k_pages, v_pages, table, page_size, n_kv, head_dim, dtype, ctx, value_dim=None):
        value_dim = value_dim or head_dim
        self._want(k_pages, "key pages", dtype)
        self._want(v_pages, "value pages", dtype)
        pages = k_pages.shape[0]
        if tuple(k_pages.shape) != (pages, n_kv, page_size, head_dim):
            raise KernelError(f"key pages {tuple(k_pages.shape)} are not [pages, {n_kv}, {page_size}, {head_dim}]")
        if tuple(v_pages.shape) != (pages, n_kv, value_dim, page_size):
            raise KernelError(f"value pages {tuple(v_pages.shape)} are not [pages, {n_kv}, {value_dim}, {page_size}]")
        self._want(table, "block table", torch.int32)
        if table.dim() != 2 or table.shape[0] != ctx.n_seqs or table.shape[1] * page_size < ctx.max_kv_len:
            raise KernelError(f"block table {tuple(table.shape)} does not cover {ctx.n_seqs} sequences of up to "
                              f"{ctx.max_kv_len} positions with pages of {page_size}")

    # -- attention ---------------------------------------------------------------
    def check_attention_geometry(self, n_heads: int, n_kv_heads: int, head_dim: int, own_writer: bool = False) -> None:
        """Raises for head counts and sizes that no attention kernel here takes.  A mixer calls it when the model is
        built, so that such a model is refused before it is loaded, not at its first step.  ``own_writer``: the mixer
        fills the pages with a kernel of its own that has no limit, so the page attention's limit is the only one."""
        limit = self.core.sia_attention_generic_max_head_dim() if own_writer else self.core.sia_attention_max_head_dim()
        if not 0 < head_dim <= limit:
            raise KernelError(f"head size {head_dim} is outside what the attention kernels take (1 to {limit})")
        if n_kv_heads <= 0 or n_heads <= 0 or n_heads % n_kv_heads:
            raise KernelError(f"{n_heads} query heads cannot share {n_kv_heads} key/value heads evenly")
        if n_heads > 65535:
            raise KernelError(f"{n_heads} query heads exceed the kernels' grids (65,535)")

    def paged_attention(self, qkv, n_heads, n_kv_heads, head_dim, scale, window, ctx, cache, value_dim=None,
                        chunk=None, sinks=None):
        """Attention of the rows' q columns over the pages.  ``chunk``: a query sees only the keys of its own block
        of that many positions; ``sinks``: float ``[n_heads]``, one more term ``exp(sink_h)`` in every softmax
        denominator of head h; ``value_dim``: width of the value rows if not ``head_dim`` (the result is
        ``[tokens, n_heads * value_dim]``)."""
        self._want(qkv, "qkv")
        n, width = qkv.shape
        value_dim = int(value_dim or head_dim)
        if width < n_heads * head_dim or n != ctx.n_tokens:
            raise KernelError(f"qkv {tuple(qkv.shape)} does not hold {ctx.n_tokens} rows of {n_heads} heads of {head_dim}")
        self._check_pages(cache.k_pages, cache.v_pages, cache.block_table, cache.page_size, n_kv_heads, head_dim,
                          qkv.dtype, ctx, value_dim)
        if sinks is not None:
            self._want(sinks, "sinks", torch.float32, (n_heads,))
        if chunk is not None and chunk <= 0:
            raise KernelError(f"chunk must be positive, got {chunk}")
        out = torch.empty((n, n_heads * value_dim), dtype=qkv.dtype, device=qkv.device)
        page = cache.page_size
        if (self.use_mfma_attention and qkv.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256
                and value_dim == head_dim and page >= 8 and width % 8 == 0 and scale > 0):
            self._mfma_attention(qkv, out, n_heads, n_kv_heads, head_dim, scale, int(window or 0), ctx, cache,
                                 int(chunk or 0), sinks)
            return out
        self._check(self.core.sia_attention_generic(
            _ptr(qkv), width, _ptr(cache.k_pages), _ptr(cache.v_pages), _ptr(cache.block_table),
            cache.block_table.shape[1], _ptr(ctx.seq_of_token), _ptr(ctx.positions), _ptr(out), n, n_heads,
            n_kv_heads, head_dim, value_dim, page, float(scale), int(window or 0), int(chunk or 0), _ptr(sinks),
            _DT[qkv.dtype], self._stream()), "attention_generic")
        return out

    def _attention_plan(self, lib, device, n_heads, n_kv_heads, head_dim, window, ctx, chunk=0):
        """What the attention launches of a step need beside the tensors: the same for every layer with this
        geometry, so it is worked out once per step and kept with the step's context (workspaces included: a step's
        layers run one after the other)."""
        key = (n_heads, n_kv_heads, head_dim, window, chunk)
        plans = getattr(ctx, "attention_plans", None)
        span = min(b for b in (window, chunk) if b > 0) if (window > 0 or chunk > 0) else 0   # most keys a query sees
        if plans is not None and key in plans:
            return plans[key]
        # the decode kernel takes up to 16 query heads a key/value head (and what its LDS holds of their states): more
        # are dealt out as several groups that read the same head
        group = n_heads // n_kv_heads
        share = next(s for s in range(1, group + 1)
                     if group % s == 0 and group // s <= 16 and 4 * (group // s) * (head_dim + 2) * 4 <= 65536)
        n_dec = ctx.n_decode_seqs
        max_splits, ws_acc, ws_ml = 1, None, None
        if n_dec:
            # How many workgroups share a (sequence, kv head) is the kernel's decision, from that sequence's own
            # length; the step's longest possible sequence only sizes the grid and the workspaces.
            max_splits = lib.sia_attn_decode_max_splits(int(ctx.kv_bound or ctx.max_kv_len), span)
            ws_acc, ws_ml = (
                torch.empty((floats,), dtype=torch.float32, device=device) if floats else None
                for floats in (lib.sia_attn_decode_workspace(n_dec, n_heads, n_kv_heads * share, max_splits, which)
                               for which in (0, 1)))
        tiles = (0, 0, 0, 0, 0)
        if n_dec < ctx.n_seqs:
            # row tiles at each of the kernel's workgroup sizes, and what bounds a sequence's tokens and keys in this
            # step: a portion over a long past takes another workgroup shape than a prompt from its start
            tiles = tuple(sum(-(-q // rows) for q in ctx.q_lens[n_dec:]) if rows else 0
                          for rows in (lib.sia_attn_prefill_rows(), lib.sia_attn_prefill_rows_split(),
                                       lib.sia_attn_prefill_rows_long()))
            tiles += (int(max(ctx.q_lens[n_dec:])), int(getattr(ctx, "max_run_kv_len", 0) or ctx.max_kv_len))
        plan = (n_dec, max_splits, ws_acc, ws_ml, tiles, share)
        if plans is None:
            try:
                ctx.attention_plans = plans = {}
            except AttributeError:      # a context that takes no further attributes: nothing is kept
                return plan
        plans[key] = plan
        return plan

    def _mfma_attention(self, qkv, out, n_heads, n_kv_heads, head_dim, scale, window, ctx, cache, chunk=0, sinks=None):
        lib = self._attn_lib(head_dim)
        width = qkv.shape[1]
        table = cache.block_table
        n_dec, max_splits, ws_acc, ws_ml, (n_tiles, n_tiles_split, n_tiles_long, q_bound, kv_bound), share = \
            self._attention_plan(lib, qkv.device, n_heads, n_kv_heads, head_dim, window, ctx, chunk)
        if n_dec:
            self._check(lib.sia_attn_decode_shared(
                _ptr(qkv), width, _ptr(cache.k_pages), _ptr(cache.v_pages), _ptr(table), table.shape[1],
                _ptr(ctx.cu_q), _ptr(ctx.kv_len), _ptr(out), _ptr(ws_acc), _ptr(ws_ml), n_dec, n_heads,
                n_kv_heads * share, share, cache.page_size, float(scale), window, chunk, _ptr(sinks), max_splits,
                self._stream()), "attn_decode")
        if n_dec < ctx.n_seqs:
            self._check(lib.sia_attn_prefill_ex(
                _ptr(qkv), width, _ptr(cache.k_pages), _ptr(cache.v_pages), _ptr(table), table.shape[1],
                _ptr(ctx.cu_q), _ptr(ctx.kv_len), _ptr(out), n_dec, ctx.n_seqs, n_tiles, n_tiles_split, n_tiles_long,
                q_bound, kv_bound, n_heads, n_kv_heads, cache.page_size, float(scale), window, chunk, _ptr(sinks),
                self._stream()), "attn_prefill")

    # -- a whole block in one call -------------------------------------------------
    def _library_can(self, M, N, K) -> bool:
        key = (M, N, K)
        known = self._products_known.get(key)
        if known is None:
            with torch.cuda.device(self.device):
                known = self._products_known[key] = self.blas.sia_blas_can(M, N, K, 0) == 0
        return known

    def _block_own(self, block):
        """The block as the one-call form takes it (a structure of pointers and constants, with the tensors it points
        into), or False if its parts are not of the kinds that form covers.  Made once and kept with the block."""
        forms = block.plain_forms
        if forms is not None:
            return forms
        block.plain_forms = False
        # the block says what it is: its kind and its parts' own descriptions.  The one-call form exists for a
        # pre-norm block of an RMS norm, paged attention, an RMS norm and a SwiGLU feed-forward.
        whole = getattr(block, "plain_form", lambda: None)()
        if not whole or whole.get("kind") != "prenorm":
            return False
        parts = [whole.get(name) for name in ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")]
        if any(f is None for f in parts) or [f["kind"] for f in parts] != ["rmsnorm", "paged_attention", "rmsnorm", "swiglu"]:
            return False
        n1, at, n2, ff = parts
        H, nh, nkv, D, I = at["hidden"], at["n_heads"], at["n_kv_heads"], at["head_dim"], ff["inter"]
        bf, f32 = torch.bfloat16, torch.float32
        wanted = ((n1["weight"], f32, (H,)), (n2["weight"], f32, (H,)), (at["w_qkv"], bf, ((nh + 2 * nkv) * D, H)),
                  (at["w_o"], bf, (H, nh * D)), (ff["w_gate_up"], bf, (2 * I, H)), (ff["w_down"], bf, (H, I)))
        rd = at["rotary_dim"]
        if rd:
            wanted += ((at["cos"], f32, None), (at["sin"], f32, None))
        for t, dtype, shape in wanted:
            if (not isinstance(t, torch.Tensor) or t.device.type != "cuda" or t.dtype != dtype or not t.is_contiguous()
                    or (shape is not None and tuple(t.shape) != shape)):
                return False
        if (ff["hidden"] != H or n1["size"] != H or n2["size"] != H or D % 16 or D > 256 or not at["scale"] > 0
                or (rd and (at["cos"].shape[1] != rd // 2 or at["sin"].shape != at["cos"].shape))):
            return False
        own = _BlockOwn(_ptr(n1["weight"]), _ptr(at["w_qkv"]), _ptr(at["w_o"]), _ptr(n2["weight"]), _ptr(ff["w_gate_up"]),
                        _ptr(ff["w_down"]), _ptr(at["cos"]) if rd else None, _ptr(at["sin"]) if rd else None,
                        float(n1["eps"]), float(n2["eps"]), float(at["scale"]), H, nh, nkv, D, rd, I, int(at["window"] or 0))
        block.plain_forms = (own, [t for t, _, _ in wanted], at["cos"].shape[0] if rd else None)
        return block.plain_forms

    def _block_step(self, own, ctx, device):
        """What a step brings to the one-call form of its blocks of this geometry: buffers, metadata, the attention
        plan.  Made once per step and geometry and kept with the step's context; None if the library has no
        algorithm for one of the products at this number of rows."""
        key = (own.hidden, own.n_heads, own.n_kv, own.head_dim, own.inter, own.window)
        steps = getattr(ctx, "block_steps", None)
        if steps is None:
            try:
                ctx.block_steps = steps = {}
            except AttributeError:
                return None
        if key in steps:
            return steps[key]
        M, H, Q, I = ctx.n_tokens, own.hidden, own.n_heads * own.head_dim, own.inter
        width = (own.n_heads + 2 * own.n_kv) * own.head_dim
        steps[key] = None
        if not all(self._library_can(M, n, k) for n, k in ((width, H), (H, Q), (2 * I, H), (H, I))):
            return None
        lib = self._attn_lib(own.head_dim)
        n_dec, max_splits, ws_acc, ws_ml, tiles, share = self._attention_plan(lib, device, own.n_heads, own.n_kv,
                                                                              own.head_dim, own.window, ctx)
        if share != 1:      # the library's step calls the decode kernel with the heads' own grouping
            return None
        new = lambda n: torch.empty((M, n), dtype=torch.bfloat16, device=device)
        buffers = [new(H), new(width), new(Q), new(H), new(2 * I), new(I), new(H)]
        fn = lambda f: ctypes.cast(f, ctypes.c_void_p).value
        step = _BlockStep(fn(self.blas.sia_blas_mm), fn(lib.sia_attn_decode), fn(lib.sia_attn_prefill), None,
                          *[_ptr(b) for b in buffers], _ptr(ctx.positions), _ptr(ctx.seq_of_token), _ptr(ctx.cu_q),
                          _ptr(ctx.kv_len), _ptr(ws_acc), _ptr(ws_ml), M, ctx.n_seqs, n_dec, max_splits, *tiles)
        steps[key] = (step, buffers)
        return steps[key]

    def prenorm_block(self, block, stream, ctx, cache) -> bool:
        """Runs a pre-norm block of RMS norms, paged attention and SwiGLU on a step of many rows with one call into
        the library (the same launches, in the same order, as the parts' own calls make); False, with nothing done,
        where that form does not apply: the caller then goes part by part."""
        if not self.whole_blocks or self.blas is None or not self.use_mfma_attention:
            return False
        residual = stream.residual
        M = ctx.n_tokens
        if (M <= self._skinny_rows or M > 65535 or getattr(ctx, "extra", None)
                or residual.dtype != torch.float32 or cache.k_pages is None or cache.page_size < 8):
            return False
        made = self._block_own(block)
        if not made:
            return False
        own, _, positions_covered = made
        if (tuple(residual.shape) != (M, own.hidden) or not residual.is_contiguous() or cache.k_pages.dtype != torch.bfloat16
                or (positions_covered is not None and positions_covered <= ctx.max_kv_len - 1)):
            return False
        step = self._block_step(own, ctx, residual.device)
        if step is None:
            return False
        delta = stream.delta    # computes it if it is a product not yet computed
        if delta is not None and (delta.dtype != torch.bfloat16 or tuple(delta.shape) != (M, own.hidden)
                                  or not delta.is_contiguous()):
            return False
        self._check_pages(cache.k_pages, cache.v_pages, cache.block_table, cache.page_size, own.n_kv, own.head_dim,
                          torch.bfloat16, ctx)
        step_struct, buffers = step
        step_struct.residual = _ptr(residual)
        self._check(self.core.sia_prenorm_block(
            ctypes.addressof(own), ctypes.addressof(step_struct), _ptr(delta), _ptr(cache.block_table),
            cache.block_table.shape[1], _ptr(cache.k_pages), _ptr(cache.v_pages), cache.page_size, self._stream()),
            "prenorm_block")
        stream.delta = buffers[-1]
        return True

    # -- sampling ------------------------------------------------------------------
    def sample(self, logits, temperature, top_k, top_p, uniform, all_greedy=False, filters=None):
        """One token per row.  What the caller knows on the host spares launches: ``all_greedy`` (every
        temperature is 0; the parameter tensors may then be None), or ``filters``, the sum of 1 if some row
        may have a top-k filter and 2 if some row may have a top-p filter below 1 (None: both)."""
        rows, vocab = logits.shape
        self._want(logits, "logits", torch.float32)
        if all_greedy:
            filters = 0
            temperature = top_k = top_p = uniform = None
        else:
            filters = 4 | (3 if filters is None else int(filters) & 3)
            self._want(temperature, "temperature", torch.float32, (rows,))
            self._want(top_k, "top_k", torch.int32, (rows,))
            self._want(top_p, "top_p", torch.float32, (rows,))
            self._want(uniform, "uniform", torch.float32, (rows,))
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        # One workspace, kept and grown as needed: the kernels set to zero what they need at zero, and calls follow
        # one another on the stream.  (Callers on several streams at once need a kernels object each.)
        need = self.core.sia_sample_workspace_bytes(rows)
        workspace = getattr(self, "_sample_workspace", None)
        if workspace is None or workspace.numel() < need or workspace.device != logits.device:
            workspace = self._sample_workspace = torch.empty((need,), dtype=torch.uint8, device=logits.device)
        self._check(self.core.sia_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
                                         _ptr(out), _ptr(workspace), rows, vocab, filters, self._stream()), "sample")
        return out
