"""Python face of the HIP kernels: checks shapes on the host, then launches on
torch's current stream.  Tensors are torch tensors used as device memory; no
torch operator computes anything here.

The reference's façade (python/lyapunov_engine/ops.py:12-216) falls back to
eager PyTorch when its extension is missing.  There is no fallback here: a
library that cannot be loaded, or an input on the wrong device, is an error.
"""
from __future__ import annotations

import ctypes
import math
import os
from ctypes import c_double, c_float, c_int, c_longlong, c_void_p

import torch

from . import build

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

STORE_ACT, STORE_F32, ACCUM_F32 = 0, 1, 2


class KernelError(RuntimeError):
    pass


def _load(path) -> ctypes.CDLL:
    try:
        return ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelError(f"cannot load the kernel library {path}: {e}") from None


_core = None
_attn: dict[int, ctypes.CDLL] = {}


def core() -> ctypes.CDLL:
    global _core
    if _core is None:
        lib = _load(build.core_library())
        lib.lyp_last_error.restype = ctypes.c_char_p
        lib.lyp_embedding.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p]
        lib.lyp_table_load.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p]
        lib.lyp_rmsnorm.argtypes = [c_void_p, c_void_p, c_int, c_longlong, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                    c_int, c_int, c_float, c_void_p]
        lib.lyp_rmsnorm_act.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p]
        lib.lyp_rope_kv_write.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_swiglu.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_gemm_parts_hint.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int]
        lib.lyp_gemm_nt_parts.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p]
        lib.lyp_gemm_swiglu.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                        c_int, c_void_p]
        lib.lyp_gemm_rope_kv.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                         c_int, c_int, c_int, c_void_p]
        lib.lyp_gemm_residual_parts.argtypes = [c_int, c_int, c_int]
        lib.lyp_gemm_residual.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p]
        lib.lyp_gemm_swiglu_normed.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p,
                                               c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_gemm_rope_kv_normed.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p,
                                                c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                                c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                                c_void_p]
        lib.lyp_cast.argtypes = [c_void_p, c_int, c_void_p, c_int, c_longlong, c_void_p]
        lib.lyp_sum_parts.argtypes = [c_void_p, c_int, c_longlong, c_void_p, c_int, c_void_p]
        lib.lyp_gemm_nt.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int, c_void_p]
        lib.lyp_sample.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p]
        lib.lyp_sample_cand.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_void_p, c_void_p, c_void_p]
        lib.lyp_lm_head.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p, c_int, c_void_p]
        lib.lyp_sample_workspace.argtypes = [c_int]
        lib.lyp_sample_workspace.restype = c_longlong
        lib.lyp_norm_threads_override.argtypes = [c_int]
        lib.lyp_skinny_row_tiles_override.argtypes = [c_int]
        lib.lyp_skinny_workgroups.argtypes = [c_int, c_int, c_int, c_int]
        lib.lyp_skinny_slices.argtypes = [c_int, c_int]
        lib.lyp_stream_read.argtypes = [c_void_p, c_longlong, c_int, c_void_p, c_void_p]
        lib.lyp_stream_rows.argtypes = [c_void_p, c_longlong, c_int, c_int, c_int, c_void_p, c_void_p]
        lib.lyp_gemm_nt_batched.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                            c_int, c_int, c_int, c_longlong, c_longlong, c_longlong, c_void_p]
        lib.lyp_branch_join.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p,
                                        c_int, c_void_p, c_int, c_int, c_float, c_float, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_int, c_void_p]
        lib.lyp_add_row.argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p]
        lib.lyp_short_conv.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                       c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]
        lib.lyp_activation.argtypes = [c_void_p, c_void_p, c_int, c_longlong, c_int, c_void_p, c_void_p]
        lib.lyp_mingru_scan.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_int, c_int, c_void_p]
        lib.lyp_mingru_scan_chunks.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_longlong, c_void_p]
        lib.lyp_latent_prep.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                        c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p]
        lib.lyp_latent_query_rotate.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                                c_int, c_int, c_int, c_void_p]
        lib.lyp_latent_attn_rows.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                             c_int, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                             c_void_p]
        lib.lyp_qk_norm_rope_kv.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int,
                                            c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                            c_void_p]
        lib.lyp_attn_rows.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p,
                                      c_void_p, c_int, c_void_p, c_float, c_int, c_int, c_void_p, c_int, c_int, c_int,
                                      c_int, c_int, c_int, c_int, c_float, c_void_p, c_void_p]
        lib.lyp_stream_add.argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p, c_longlong, c_void_p]
        lib.lyp_moe_route.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]
        lib.lyp_moe_route_splits.argtypes = [c_int, c_int]
        lib.lyp_moe_route_fused.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                            c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p]
        lib.lyp_moe_route_sort.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                           c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p]
        lib.lyp_moe_tile_rows.argtypes = [c_int, c_int]
        lib.lyp_moe_most_tiles.argtypes = [c_int, c_int, c_int]
        lib.lyp_moe_sort.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_void_p]
        lib.lyp_moe_gemm.argtypes = [c_void_p, c_int, c_void_p, c_longlong, c_int, c_void_p, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                     c_float, c_float, c_int, c_void_p]
        lib.lyp_glu_clamped.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_void_p]
        lib.lyp_moe_combine.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                        c_int, c_void_p]
        lib.lyp_group_rmsnorm.argtypes = [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_void_p, c_int,
                                          c_void_p, c_int, c_int, c_int, c_float, c_void_p]
        lib.lyp_add_sinusoid.argtypes = [c_void_p, c_void_p, c_int, c_int, c_double, c_void_p]
        lib.lyp_glu_act.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_gate_mul.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_weighted_sum.argtypes = [c_void_p, c_int, c_void_p, c_float, c_void_p, c_int, c_float, c_void_p, c_int,
                                         c_int, c_void_p]
        lib.lyp_qkv_bias_temper_kv.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_float, c_int, c_void_p, c_void_p,
                                               c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                               c_void_p]
        lib.lyp_linear_scan_lanes.argtypes = [c_int]
        lib.lyp_linear_scan.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_int,
                                        c_void_p, c_void_p, c_float, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                        c_float, c_void_p, c_int, c_int, c_void_p]
        lib.lyp_head_norm_gate.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int,
                                           c_int, c_float, c_int, c_int, c_void_p]
        lib.lyp_lowrank_up.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                       c_void_p, c_float, c_int, c_int, c_int, c_void_p]
        lib.lyp_qkv_prepare.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                        c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_shift_mix.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int, c_int, c_int, c_int, c_void_p]
        lib.lyp_skip_gate_group_norm.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                                 c_int, c_int, c_int, c_int, c_int, c_float, c_void_p]
        lib.lyp_gather_gelu_mul.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int,
                                            c_int, c_int, c_void_p]
        lib.lyp_moe_choose_grouped.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                               c_void_p, c_void_p, c_void_p]
        lib.lyp_moe_route_grouped.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                              c_int, c_int, c_float, c_void_p, c_void_p, c_void_p]
        _core = lib
    return _core


def attention_lib(head_dim: int) -> ctypes.CDLL:
    lib = _attn.get(head_dim)
    if lib is None:
        lib = _load(build.attention_library(head_dim))
        lib.lyp_last_error.restype = ctypes.c_char_p
        if lib.lyp_attn_head_dim() != head_dim:
            raise KernelError(f"attention library for head size {head_dim} reports {lib.lyp_attn_head_dim()}")
        lib.lyp_attn_prefill.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                         c_float, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_float, c_void_p,
                                         c_void_p]
        lib.lyp_attn_prefill_plan.argtypes = [c_int, c_int, c_int, c_int, c_int, c_int]
        lib.lyp_attn_decode.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                        c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                        c_int, c_int, c_int, c_float, c_int, c_void_p, c_float, c_void_p, c_void_p]
        lib.lyp_attn_decode_plan.argtypes = [c_int, c_int, c_int, c_int]
        _attn[head_dim] = lib
    return lib


def require_gpu() -> None:
    """The kernels are built for one architecture; say so before the first
    launch rather than after a failed one."""
    if not torch.cuda.is_available():
        raise KernelError("no GPU: this package has no CPU path")
    name = torch.cuda.get_device_properties(0).gcnArchName.split(":")[0]
    if name != build.GPU_ARCH:
        raise KernelError(f"the kernels are built for {build.GPU_ARCH}, this device is {name}")


# torch's current stream as a raw handle.  torch.cuda.current_stream() builds a
# Stream object on every call (several microseconds, a tenth of the host's time
# in an eager step); the two private accessors below, where this torch has
# them, give the same handle directly.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


# Addresses go to the libraries as plain integers: every function declares its pointer arguments,
# so ctypes converts them, and no c_void_p object is built per argument.
def _stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _p(t) -> int:
    return 0 if t is None else t.data_ptr()


def _check(rc: int, lib: ctypes.CDLL) -> None:
    if rc != 0:
        raise KernelError(lib.lyp_last_error().decode())


def _dev(*ts) -> None:
    for t in ts:
        if t is not None and (not t.is_cuda or not t.is_contiguous()):
            raise KernelError(f"kernel operand must be a contiguous GPU tensor, got {tuple(t.shape)} on {t.device} "
                              f"contiguous={t.is_contiguous()}")


def _code(dt: torch.dtype) -> int:
    try:
        return _CODE[dt]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dt}") from None


# ------------------------------------------------------------------ row kernels
def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] * scale as float (the residual stream)."""
    _dev(ids, table, out)
    T, H = out.shape
    if ids.dtype != torch.int32 or ids.numel() != T or table.shape[1] != H or out.dtype != torch.float32:
        raise KernelError(f"embedding: ids {tuple(ids.shape)} {ids.dtype}, table {tuple(table.shape)}, out {tuple(out.shape)} {out.dtype}")
    lib = core()
    _check(lib.lyp_embedding(_p(ids), _p(table), _code(table.dtype), _p(out), T, H, float(scale), _stream()), lib)
    return out


# ------------------------------------------------- work handed on to a consumer
# A step with few rows is bound by the number of kernels, so two kinds of work
# may be passed on as a description for the next kernel to fold in, instead of
# being run on their own:
#   PendingLinear  a projection whose output is only ever added to the residual
#                  stream (``linear(..., pending=True)``): the adding kernel is
#                  the product itself (``linear_residual``);
#   PendingNorm    RMS-normed rows of the residual stream (``rmsnorm_pending``):
#                  the kernel that added to the stream also left the rows times
#                  the norm's weights and their sums of squares; ``linear_rope_kv``
#                  and ``linear_swiglu`` multiply those rows and divide by the
#                  rms at the end.
# Whoever cannot fold one in calls its ``run()`` and gets the plain tensor.
PENDING_MAX_ROWS = 16


class PendingLinear:
    def __init__(self, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype):
        self.x, self.w, self.out_dtype = x, w, out_dtype

    def run(self) -> torch.Tensor:
        """The product, as ``linear(..., may_split=True)`` gives it."""
        return linear(self.x, self.w, out_dtype=self.out_dtype, may_split=True)


class PendingNorm:
    """Rows of the residual stream ``h`` (already holding the sum) that are to be
    RMS-normed.  ``xs`` is h * weight in the activations' type and ``ssq_part``
    [parts, 16] the rows' sums of squares in parts: what the kernel that
    added to h left behind for the product that comes next."""

    def __init__(self, h: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype, xs: torch.Tensor,
                 ssq_part: torch.Tensor):
        self.h, self.weight, self.eps, self.dtype = h, weight, float(eps), dtype
        self.xs, self.ssq_part = xs, ssq_part
        self.shape = h.shape

    def run(self) -> torch.Tensor:
        out = torch.empty(self.h.shape, dtype=self.dtype, device=self.h.device)
        return rmsnorm(self.h, self.weight, self.eps, out)


class JoiningBranch:
    """A branch's output that passes a norm of its own and a multiplier on its way into the residual
    stream: h += mult * rmsnorm(y) * weight (+ shift, a vector for every row).  The norm that follows
    (one with ``joins_branches``) does the sum in its own kernel; ``join(h)`` does it alone.
    ``y`` [T, H] is in the activations' type or float, ``weight`` and ``shift`` are float."""

    def __init__(self, y: torch.Tensor, weight: torch.Tensor, eps: float, mult: float = 1.0,
                 shift: torch.Tensor | None = None):
        self.y, self.weight, self.eps, self.mult, self.shift = y, weight, float(eps), float(mult), shift
        self.shape = y.shape

    def join(self, h: torch.Tensor) -> None:
        """Carry the sum out on h; nothing is left to add (returns None)."""
        branch_join(h, self.y, self.weight, self.mult, self.eps, shift=self.shift)
        return None


def shifted(h: torch.Tensor, delta, v: torch.Tensor):
    """The residual stream h with what is still to be added to it (``delta``), plus the vector v on
    every row.  A branch that is about to join takes v along; otherwise v is added to h now.
    Returns what is still to be added."""
    if isinstance(delta, JoiningBranch):
        if delta.shift is None:
            return JoiningBranch(delta.y, delta.weight, delta.eps, delta.mult, v)
        delta = delta.join(h)
    add_row(h, v)
    return delta


def as_delta(delta, dtype: torch.dtype):
    """What a mixer or feed-forward returned, as one plain tensor [T, H] of
    ``dtype`` (for a norm that adds it by itself)."""
    if delta is None:
        return None
    if isinstance(delta, PendingLinear):
        delta = delta.run()
    return sum_parts(delta, dtype)


def _few_rows_product(M: int, w: torch.Tensor, act_dtype: torch.dtype) -> bool:
    """Whether x [M, K] @ w.T runs in the weight-streaming kernel of this package."""
    return (M <= 64 and w.dtype == act_dtype and w.shape[1] % 64 == 0 and w.stride(1) == 1
            and not _library_product(M, w.shape[0], w.shape[1], act_dtype))


def linear_residual(h: torch.Tensor, p: PendingLinear, next_weight: torch.Tensor | None = None):
    """h += p.x @ p.w.T on the float residual stream, in the product's kernel.
    With ``next_weight`` (the weights of the RMS norm that follows) the kernel
    also leaves what a PendingNorm carries, and (xs, ssq_part) is returned;
    without it, True.  False (nothing done) when that kernel does not apply."""
    x, w = p.x, p.w
    M, K = x.shape
    N = w.shape[0]
    if h.dtype != torch.float32 or tuple(h.shape) != (M, N) or w.shape[1] != K or not _few_rows_product(M, w, x.dtype):
        return False
    _dev(h, x, w, next_weight)
    lib = core()
    xs = ssq = None
    if next_weight is not None:
        if M > PENDING_MAX_ROWS or next_weight.numel() != N:
            return False
        xs = torch.empty((M, N), dtype=x.dtype, device=h.device)
        ssq = torch.empty((lib.lyp_gemm_residual_parts(M, N, K), 16), dtype=torch.float32, device=h.device)
    rc = lib.lyp_gemm_residual(_p(x), _p(w), _p(h), _code(x.dtype), M, N, K, x.stride(0), w.stride(0), h.stride(0),
                               _p(next_weight), _code(next_weight.dtype) if next_weight is not None else 0, _p(xs), N,
                               _p(ssq), _stream())
    if rc < 0:
        _check(rc, lib)
    if rc != 0:
        return False
    return (xs, ssq) if next_weight is not None else True


def rmsnorm_pending(h: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype, delta=None):
    """Add ``delta`` to h and describe the normed rows instead of computing
    them.  Returns (PendingNorm, None), or (None, delta) when the rows had
    better be normed by ``rmsnorm``: ``delta`` is then what still has to be
    added.  Only a delta that is a product still to be run can be folded: its
    kernel is the one that prepares the norm."""
    if (not isinstance(delta, PendingLinear) or h.shape[0] > PENDING_MAX_ROWS or h.dtype != torch.float32
            or delta.x.dtype != dtype):
        return None, delta
    done = linear_residual(h, delta, weight)
    if done is False:
        return None, delta
    return PendingNorm(h, weight, eps, dtype, *done), None


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor, delta: torch.Tensor | None = None,
            rows: torch.Tensor | None = None) -> torch.Tensor:
    """out = rmsnorm(h [+ delta]) * weight.  h is the float residual stream and
    takes the sum, unless ``rows`` picks the rows to norm.  ``delta`` is [T, H]
    in out's dtype, float partial sums [S, T, H], or a product still to be run
    (see ``linear``)."""
    if isinstance(delta, PendingLinear):
        delta = delta.run()
    _dev(h, weight, out, delta, rows)
    H = h.shape[1]
    n = out.shape[0]
    if h.dtype != torch.float32 or weight.numel() != H or out.shape[1] != H:
        raise KernelError(f"rmsnorm: h {tuple(h.shape)} {h.dtype}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    parts, stride = 0, 0
    if delta is not None:
        if delta.dim() == 3:
            if delta.dtype != torch.float32 or tuple(delta.shape[1:]) != tuple(h.shape):
                raise KernelError(f"rmsnorm: partial sums {tuple(delta.shape)} {delta.dtype} against h {tuple(h.shape)}")
            parts, stride = delta.shape[0], delta.shape[1] * delta.shape[2]
        elif delta.shape != h.shape or delta.dtype != out.dtype:
            raise KernelError(f"rmsnorm: delta {tuple(delta.shape)} {delta.dtype} against h {tuple(h.shape)}, out {out.dtype}")
    if rows is not None:
        if rows.dtype != torch.int32 or rows.numel() != n:
            raise KernelError("rmsnorm: rows must be int32, one per output row")
    elif n != h.shape[0]:
        raise KernelError("rmsnorm: output rows differ from input rows")
    lib = core()
    _check(lib.lyp_rmsnorm(_p(h), _p(delta), parts, stride, _p(weight), _code(weight.dtype), _p(out), _code(out.dtype),
                           _p(rows), n, H, float(eps), _stream()), lib)
    return out


def stream_read(src: torch.Tensor, sink: torch.Tensor, blocks: int) -> None:
    """Read all of ``src`` once with ``blocks`` workgroups (a yardstick for the
    kernels that stream weights); ``sink``: int32, blocks * 4 values."""
    _dev(src, sink)
    nbytes = src.numel() * src.element_size()
    if sink.dtype != torch.int32 or sink.numel() < blocks * 4:
        raise KernelError("stream_read: the sink must hold four int32 values per workgroup")
    lib = core()
    _check(lib.lyp_stream_read(_p(src), nbytes, blocks, _p(sink), _stream()), lib)


def stream_rows(src: torch.Tensor, sink: torch.Tensor, blocks: int, row_bytes: int, whole_lines: bool = False) -> None:
    """Read all of ``src`` once as a matrix of rows of ``row_bytes``, the way the
    weight-streaming products do (16 rows a wave, 64 bytes of each per load; with
    ``whole_lines`` 8 rows a wave and 128 bytes of each)."""
    _dev(src, sink)
    nbytes = src.numel() * src.element_size()
    if sink.dtype != torch.int32 or sink.numel() < blocks * 4:
        raise KernelError("stream_rows: the sink must hold four int32 values per workgroup")
    lib = core()
    _check(lib.lyp_stream_rows(_p(src), nbytes, row_bytes, int(whole_lines), blocks, _p(sink), _stream()), lib)


def norm_threads_override(threads: int) -> None:
    """Threads per row of the two-pass norm kernels (0: the built-in rule); for measurements."""
    lib = core()
    _check(lib.lyp_norm_threads_override(threads), lib)


def skinny_row_tiles_override(row_tiles: int) -> None:
    """Row tiles (of 16 rows of the weights) per workgroup of the weight-streaming product in steps
    of more than 16 rows (0: the built-in rule); for measurements."""
    lib = core()
    _check(lib.lyp_skinny_row_tiles_override(row_tiles), lib)


def rmsnorm_act(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
    _dev(x, weight, out)
    n, H = x.shape
    if out.shape != x.shape or out.dtype != x.dtype or weight.numel() != H:
        raise KernelError("rmsnorm_act: shapes or dtypes differ")
    lib = core()
    _check(lib.lyp_rmsnorm_act(_p(x), _p(weight), _code(weight.dtype), _p(out), _code(x.dtype), n, H, float(eps),
                               _stream()), lib)
    return out


def _rope_check(T: int, dtype: torch.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads: int,
                head_dim: int, page_size: int, has_kv: bool) -> int:
    """Checks the operands that the rotation and the page write share; returns the rotary size."""
    if positions.numel() != T or positions.dtype != torch.int32:
        raise KernelError(f"rope_kv_write: positions {tuple(positions.shape)} {positions.dtype} for {T} tokens")
    rot = 0
    if cos_sin is not None:
        rot = cos_sin.shape[1]
        if cos_sin.dtype != torch.float32 or rot > head_dim or rot % 2:
            raise KernelError(f"rope_kv_write: table {tuple(cos_sin.shape)} {cos_sin.dtype} for heads of {head_dim}")
    if has_kv:
        n_pages = kpool.shape[0]
        if (slots is None or slots.numel() != T or slots.dtype != torch.int32
                or tuple(kpool.shape) != (n_pages, num_kv_heads, page_size, head_dim)
                or tuple(vpool.shape) != (n_pages, num_kv_heads, head_dim, page_size)
                or kpool.dtype != dtype or vpool.dtype != dtype):
            raise KernelError(f"rope_kv_write: pools {tuple(kpool.shape)} / {tuple(vpool.shape)} {kpool.dtype} do not "
                              f"fit {num_kv_heads} heads of {head_dim}, pages of {page_size}, dtype {dtype}")
    return rot


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor | None,
                  slots: torch.Tensor | None, kpool: torch.Tensor | None, vpool: torch.Tensor | None, *, num_heads: int,
                  num_kv_heads: int, head_dim: int, page_size: int, has_kv: bool = True) -> None:
    """Rotate the query (and key) heads of ``qkv`` in place by each token's
    position and store keys and values in the token's cache slot."""
    _dev(qkv, positions, cos_sin, slots, kpool, vpool)
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim if has_kv else num_heads * head_dim
    if qkv.shape[1] != width:
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} against width {width}")
    rot = _rope_check(T, qkv.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads, head_dim, page_size, has_kv)
    lib = core()
    _check(lib.lyp_rope_kv_write(_p(qkv), _code(qkv.dtype), _p(positions), _p(cos_sin), _p(slots), _p(kpool),
                                 _p(vpool), T, num_heads, num_kv_heads, head_dim, rot, page_size, int(has_kv),
                                 _stream()), lib)


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, interleave: int = 0) -> torch.Tensor:
    """out = silu(gate) * up.  interleave 0: gate_up[:, :I] are the gates and
    gate_up[:, I:] the ups; interleave 8: columns come in tiles of 16, eight
    gates then the eight ups that go with them."""
    _dev(gate_up, out)
    T, I = out.shape
    if tuple(gate_up.shape) != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError(f"swiglu: {tuple(gate_up.shape)} -> {tuple(out.shape)}")
    lib = core()
    _check(lib.lyp_swiglu(_p(gate_up), _p(out), _code(out.dtype), T, I, interleave, _stream()), lib)
    return out


def linear_rope_kv(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor | None,
                   slots: torch.Tensor | None, kpool: torch.Tensor | None, vpool: torch.Tensor | None, *,
                   num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                   has_kv: bool = True) -> torch.Tensor:
    """The fused q/k/v projection of x (w: query heads, then key heads, then
    value heads; query heads alone without ``has_kv``), query and key heads
    rotated by position, keys and values stored in the tokens' cache slots.
    Returns a tensor whose first ``num_heads * head_dim`` columns are the
    rotated query heads.  With few rows this is one kernel; its results equal
    ``linear`` followed by ``rope_kv_write`` bit for bit."""
    M, K = x.shape
    N = w.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim if has_kv else num_heads * head_dim
    if N != width or w.shape[1] != K:
        raise KernelError(f"linear_rope_kv: weight {tuple(w.shape)} for {width} features of {K}")
    if isinstance(x, PendingNorm):
        p = x
        if _few_rows_product(M, w, p.dtype):
            _dev(p.xs, p.ssq_part, w, positions, cos_sin, slots, kpool, vpool)
            rot = _rope_check(M, p.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads, head_dim, page_size,
                              has_kv)
            out = torch.empty((M, num_heads * head_dim), dtype=p.dtype, device=w.device)
            lib = core()
            rc = lib.lyp_gemm_rope_kv_normed(_p(p.xs), p.xs.stride(0), _p(p.ssq_part), p.ssq_part.shape[0],
                                             p.h.shape[1], p.eps,
                                             _p(w), _p(out), _code(p.dtype), M, K, w.stride(0), out.stride(0),
                                             _p(positions), _p(cos_sin), _p(slots), _p(kpool), _p(vpool), num_heads,
                                             num_kv_heads, head_dim, rot, page_size, int(has_kv), _stream())
            if rc == 0:
                return out
            if rc < 0:
                _check(rc, lib)
        x = p.run()
    if w.dtype == x.dtype and M <= 64 and not _library_product(M, N, K, x.dtype):
        _dev(x, w, positions, cos_sin, slots, kpool, vpool)
        rot = _rope_check(M, x.dtype, positions, cos_sin, slots, kpool, vpool, num_kv_heads, head_dim, page_size,
                          has_kv)
        out = torch.empty((M, num_heads * head_dim), dtype=x.dtype, device=x.device)
        lib = core()
        rc = lib.lyp_gemm_rope_kv(_p(x), _p(w), _p(out), _code(x.dtype), M, K, x.stride(0), w.stride(0),
                                  out.stride(0), _p(positions), _p(cos_sin), _p(slots), _p(kpool), _p(vpool),
                                  num_heads, num_kv_heads, head_dim, rot, page_size, int(has_kv), _stream())
        if rc == 0:
            return out
        if rc < 0:
            _check(rc, lib)
    qkv = linear(x, w, out_dtype=x.dtype)
    rope_kv_write(qkv, positions, cos_sin, slots, kpool, vpool, num_heads=num_heads, num_kv_heads=num_kv_heads,
                  head_dim=head_dim, page_size=page_size, has_kv=has_kv)
    return qkv


def linear_swiglu(x: torch.Tensor, w: torch.Tensor, interleave: int) -> torch.Tensor:
    """silu(x @ Wgate.T) * (x @ Wup.T) for the fused matrix w [2 I, K] laid out
    as ``swiglu`` describes.  With few rows and interleave 8 it is one kernel."""
    I = w.shape[0] // 2
    if isinstance(x, PendingNorm):
        p, M = x, x.shape[0]
        if interleave == 8 and p.h.shape[1] == w.shape[1] and _few_rows_product(M, w, p.dtype):
            _dev(p.xs, p.ssq_part, w)
            out = torch.empty((M, I), dtype=p.dtype, device=w.device)
            lib = core()
            rc = lib.lyp_gemm_swiglu_normed(_p(p.xs), p.xs.stride(0), _p(p.ssq_part), p.ssq_part.shape[0],
                                            p.h.shape[1], p.eps, _p(w), _p(out), _code(p.dtype), M, w.shape[0],
                                            w.shape[1], w.stride(0), I, _stream())
            if rc == 0:
                return out
            if rc < 0:
                _check(rc, lib)
        x = p.run()
    if w.dtype != x.dtype:
        if w.dtype != torch.float32:
            raise KernelError(f"linear_swiglu: weight {w.dtype} against activations {x.dtype}")
        return cast(linear_swiglu(cast(x, torch.float32), w, interleave), x.dtype)
    out = torch.empty((x.shape[0], I), dtype=x.dtype, device=x.device)
    if interleave == 8 and x.shape[0] <= 64 and not _library_product(x.shape[0], w.shape[0], w.shape[1], x.dtype):
        _dev(x, w)
        lib = core()
        rc = lib.lyp_gemm_swiglu(_p(x), _p(w), _p(out), _code(x.dtype), x.shape[0], w.shape[0], w.shape[1],
                                 x.stride(0), w.stride(0), I, _stream())
        if rc == 0:
            return out
        if rc < 0:
            _check(rc, lib)
    gate_up = torch.empty((x.shape[0], 2 * I), dtype=x.dtype, device=x.device)
    gemm_nt(x, w, gate_up)
    return swiglu(gate_up, out, interleave)


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    if x.dtype == dtype:
        return x
    _dev(x)
    out = torch.empty_like(x, dtype=dtype)
    lib = core()
    _check(lib.lyp_cast(_p(x), _code(x.dtype), _p(out), _code(dtype), x.numel(), _stream()), lib)
    return out


# ------------------------------------------------------------------------ GEMM
# Large bfloat16 products go to the vendor's matrix library (hipBLASLt, called
# directly with the plan of every shape kept), as the reference's projections go
# to cuBLAS (nn.Linear, models/llama.py:45-48, 112-117, 177).  Products with few
# rows (decode steps), every float product (true 32-bit) and everything when
# LYAPUNOV_AMD_GEMM=own use the kernels of this package.
LIBRARY_GEMM_MODE = os.environ.get("LYAPUNOV_AMD_GEMM", "library")
if LIBRARY_GEMM_MODE not in ("library", "own"):
    raise KernelError(f"LYAPUNOV_AMD_GEMM is 'library' or 'own', not {LIBRARY_GEMM_MODE!r}")
LIBRARY_GEMM = LIBRARY_GEMM_MODE != "own"
LIBRARY_WORKSPACE_BYTES = 76 << 20    # what the library may use beside the operands (stream-K partial tiles)
LIBRARY_GEMM_MIN_ROWS = 65
# Between 17 and 64 rows the weight-streaming kernel is one burst of loads per workgroup: every
# workgroup reads the step's activations over its share of K, asks for all of its weights at once,
# sums its waves' parts and is done.  That beats the library's tiled kernels while the whole matrix
# is taken in one round of workgroups on the machine (as many workgroups as compute units, at most),
# and loses to them when the launch needs several rounds (``_library_product``).  Measured cold on
# 256 compute units at 64 rows, this kernel against the library (with the passes the library cannot
# fold in): q/k/v 3072x2048 14.7 against 18.3 us (192 workgroups), o 2048x2048 7.8 against 13.4 (256),
# down 2048x8192 16.8 against 22.8 (256), gate/up 16384x2048 28.4 against 21.9 (512: the library's).
# The burst also has to stay small: a workgroup reads its rows of the matrix and the step's
# activations over all of its share of K; past about 64 KiB of weights or 192 KiB of activations per
# workgroup the library's tiles are ahead again.  Whole decode steps at context 2,304, this package's
# kernel for every product that fits one round against the library for every product of 17 to 64 rows:
# 1B shape, batch 24 / 32 / 48 / 64: 15,510 / 19,430 / 24,630 / 29,280 against 14,820 / 18,870 / 24,250 /
# 29,680 tokens a second (64 rows of 2,048 values are 256 KiB of activations; the gains are the q/k/v and
# o products'); 8B shape, whose products of one round have 128 KiB and more of weights per workgroup:
# 4,030 / 4,930 / 6,040 / 7,410 against 4,130 / 5,090 / 6,180 / 7,760.
# (LYAPUNOV_AMD_LIBRARY_ROUNDS sets the number of rounds this package's kernel may take: 0 sends every
# product of 17 to 64 rows to the library, a large number none.)
LIBRARY_ROUNDS = float(os.environ.get("LYAPUNOV_AMD_LIBRARY_ROUNDS", "1"))
LIBRARY_ACTIVATION_BYTES = 192 << 10
LIBRARY_WEIGHT_BYTES = 64 << 10
# In an engine's warm-up step and in the run before a graph is captured, a library product's algorithm is
# chosen by measurement among this many of the library's candidates (at the shape's first call).
# Which candidate wins a timing may differ from process to process, and with it the last bits of
# bfloat16 results; LYAPUNOV_AMD_GEMM_TUNE=0 leaves every choice to the library's own heuristic, which
# gives the same bits in every run.
LIBRARY_TUNE_CANDIDATES = int(os.environ.get("LYAPUNOV_AMD_GEMM_TUNE", "16"))


_blas_lib = None
_blas_workspace: dict = {}
_blas_tuning = (0, 0)   # (candidates, without a workspace): the library's setting, kept here while it is not loaded


def blas() -> ctypes.CDLL:
    global _blas_lib
    if _blas_lib is None:
        require_gpu()
        try:
            lib = _load(build.blas_library())
        except (RuntimeError, KernelError) as e:
            raise KernelError(f"{e}\n(LYAPUNOV_AMD_GEMM=own runs every product in this package's kernels)") from None
        lib.lyp_last_error.restype = ctypes.c_char_p
        lib.lyp_library_gemm_nt.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                            c_int, c_void_p, c_longlong, c_void_p]
        lib.lyp_library_gemm_plans.restype = c_int
        lib.lyp_library_gemm_rejected.restype = c_int
        lib.lyp_library_gemm_solution.argtypes = [c_int] * 8
        lib.lyp_library_gemm_tuning.argtypes = [c_int, c_int]
        lib.lyp_library_gemm_tuning(*_blas_tuning)   # what a tuning context asked for before the library was there
        _blas_lib = lib
    return _blas_lib


class library_gemm_tuning:
    """While this context is open, a library product of a shape not seen before
    in this process is given the fastest of the library's first ``candidates``
    algorithms, found by running them on the call's operands (which waits for
    the stream); shapes seen before keep their plan.  Meant for a warm-up step."""

    def __init__(self, candidates: int | None = None, for_graph: bool = False):
        """``for_graph``: the products are about to be recorded into a graph;
        only algorithms that need no workspace are taken (one with a workspace
        may clear it with a memset node, which replayed graphs must not hold)."""
        self.candidates = LIBRARY_TUNE_CANDIDATES if candidates is None else candidates
        self.for_graph = for_graph
        self.before = None

    def __enter__(self):
        if LIBRARY_GEMM_MODE == "library" and (self.candidates > 1 or self.for_graph):
            self.before = _blas_tuning
            _set_blas_tuning(self.candidates, int(self.for_graph))
        return self

    def __exit__(self, *exc):
        if self.before is not None:
            _set_blas_tuning(*self.before)
        return False


def _set_blas_tuning(candidates: int, no_workspace: int) -> None:
    """The library is loaded by the first product that needs it (a 32-bit
    engine never does); until then the setting waits here."""
    global _blas_tuning
    _blas_tuning = (candidates, no_workspace)
    if _blas_lib is not None:
        _blas_lib.lyp_library_gemm_tuning(candidates, no_workspace)


def library_gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out [M, N] (bfloat16 or float) = a [M, K] @ w [N, K].T for bfloat16
    operands, by the vendor's library."""
    M, K = a.shape
    N = w.shape[0]
    if (a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != K or tuple(out.shape) != (M, N)
            or out.dtype not in (torch.bfloat16, torch.float32) or a.stride(1) != 1 or w.stride(1) != 1
            or out.stride(1) != 1 or not (a.is_cuda and w.is_cuda and out.is_cuda)):
        raise KernelError(f"library gemm: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}, "
                          f"out {tuple(out.shape)} {out.dtype}")
    lib = blas()
    ws = _blas_workspace.get(a.device)
    if ws is None:
        ws = _blas_workspace[a.device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=a.device)
    _check(lib.lyp_library_gemm_nt(_p(a), _p(w), _p(out), _code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                                   out.stride(0), _p(ws), ws.numel(), _stream()), lib)
    return out


def library_gemm_rejected() -> int:
    """Candidates that tuning measured and turned down because their output was off the
    heuristic's first choice by more than rounding, so far in this process."""
    return blas().lyp_library_gemm_rejected()


def library_gemm_solution(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, for_graph: bool = False) -> int:
    """The library's number for the algorithm kept for this product, -1 if the shape has no plan yet."""
    return blas().lyp_library_gemm_solution(a.shape[0], w.shape[0], a.shape[1], a.stride(0), w.stride(0), out.stride(0),
                                            _code(out.dtype), int(for_graph))


_compute_units: dict = {}


def compute_units(device=None) -> int:
    """Compute units of the device (asked once)."""
    index = torch.cuda.current_device() if device is None or torch.device(device).index is None else torch.device(device).index
    n = _compute_units.get(index)
    if n is None:
        n = _compute_units[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return n


def _library_product(M: int, N: int, K: int, dtype: torch.dtype, sliced: bool = False) -> bool:
    """Whether a bfloat16 product of M rows with a matrix [N, K] goes to the vendor's library.
    ``sliced``: the caller takes partial sums over slices of K (which gives this package's kernel
    more workgroups to spread a matrix of few rows over)."""
    if not LIBRARY_GEMM or dtype != torch.bfloat16:
        return False
    if M >= LIBRARY_GEMM_MIN_ROWS:
        return True
    if M <= PENDING_MAX_ROWS:
        return False
    lib = core()
    workgroups = lib.lyp_skinny_workgroups(M, N, K, int(sliced))
    if workgroups == 0 or workgroups > LIBRARY_ROUNDS * compute_units():
        return True
    slices = lib.lyp_skinny_slices(N, K) if sliced else 1
    k_per_workgroup = K // slices
    rows_per_workgroup = -(-N // (workgroups // slices))
    return (-(-M // 16) * 16 * k_per_workgroup * 2 > LIBRARY_ACTIVATION_BYTES
            or rows_per_workgroup * k_per_workgroup * 2 > LIBRARY_WEIGHT_BYTES)


def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
    """out = a @ w.T (or out += ...).  a [M, K], w [N, K] of one dtype; out
    [M, N] of that dtype or float.  Rows may lie further apart than they are
    long (column ranges of wider tensors); a row's values must be neighbours."""
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(out.shape) != (M, N) or a.dtype != w.dtype:
        raise KernelError(f"gemm: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}, out {tuple(out.shape)}")
    for name, t in (("a", a), ("w", w), ("out", out)):
        if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.stride(0) < t.shape[1]:
            raise KernelError(f"gemm: {name} {tuple(t.shape)} with strides {t.stride()} on {t.device}: the values of "
                              f"a row must be neighbours in GPU memory")
    if out.dtype == torch.bfloat16 and not accumulate and _library_product(M, N, K, a.dtype):
        return library_gemm_nt(a, w, out)
    if accumulate:
        if out.dtype != torch.float32:
            raise KernelError("gemm: accumulation needs a float output")
        mode = ACCUM_F32
    elif out.dtype == torch.float32:
        mode = STORE_F32
    elif out.dtype == a.dtype:
        mode = STORE_ACT
    else:
        raise KernelError(f"gemm: output dtype {out.dtype} for operands of {a.dtype}")
    lib = core()
    _check(lib.lyp_gemm_nt(_p(a), _p(w), _p(out), _code(a.dtype), mode, M, N, K, a.stride(0), w.stride(0),
                           out.stride(0), _stream()), lib)
    return out


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None,
           may_split: bool = False, pending: bool = False):
    """x @ w.T for a projection weight [out_features, in_features].  A weight
    kept in 32-bit is multiplied in 32-bit whatever the activations are.

    With ``may_split`` the result may come back as float partial sums
    [S, rows, out_features] instead (few rows, few output features: the inner
    dimension is then cut into S slices so that every compute unit has work);
    ``rmsnorm`` takes such a delta and adds the slices up, ``sum_parts`` does it
    for any other consumer.  With ``pending`` (the result will only be added to
    the residual stream) a product of few rows is not run at all but handed on
    as a ``PendingLinear``."""
    out_dtype = out_dtype or x.dtype
    if pending and x.shape[0] <= PENDING_MAX_ROWS and _few_rows_product(x.shape[0], w, x.dtype):
        return PendingLinear(x, w, out_dtype)
    if w.dtype != x.dtype:
        if w.dtype != torch.float32:
            raise KernelError(f"linear: weight {w.dtype} against activations {x.dtype}")
        x = cast(x, torch.float32)
    if may_split and x.shape[0] <= 64 and not _library_product(x.shape[0], w.shape[0], w.shape[1], x.dtype, sliced=True):
        _dev(x, w)
        lib = core()
        M, K, N = x.shape[0], x.shape[1], w.shape[0]
        slices = lib.lyp_gemm_parts_hint(_p(x), _p(w), _code(x.dtype), M, N, K, x.stride(0), w.stride(0))
        if slices > 1:
            parts = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
            _check(lib.lyp_gemm_nt_parts(_p(x), _p(w), _p(parts), _code(x.dtype), slices, M, N, K, x.stride(0),
                                         w.stride(0), _stream()), lib)
            return parts
    if out_dtype == torch.float32 and _library_product(x.shape[0], w.shape[0], w.shape[1], x.dtype):
        _dev(x, w)   # the library's float accumulators written out as they are
        return library_gemm_nt(x, w, torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device))
    if out_dtype in (x.dtype, torch.float32):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device)
        return gemm_nt(x, w, out)
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32, device=x.device)
    return cast(gemm_nt(x, w, out), out_dtype)


LM_HEAD_MAX_ROWS = 32     # what the output-head kernels may take (the library call says no where the general products are ahead)
LM_HEAD_BLOCKS = 1024     # most workgroups of the output-head kernels (the library says how many it used)


def lm_head(x: torch.Tensor, w: torch.Tensor) -> tuple:
    """-> (float logits x @ w.T for the output head [vocab, hidden], row maxima
    or None).  Few rows (a decode step's) take a kernel of their own that reads
    the matrix with few long-lived waves and leaves, beside the logits, every
    workgroup's largest logit per row: an int32 tensor [rows, workgroups, 2] of
    (value bits, index) pairs, which ``sample`` takes as ``row_maxima`` instead
    of a pass over the row.  Anything else goes through ``linear``."""
    M, K = x.shape
    if M <= LM_HEAD_MAX_ROWS and w.dtype == x.dtype and w.shape[1] == K and w.stride(1) == 1 and x.stride(1) == 1:
        _dev(x)
        lib = core()
        V = w.shape[0]
        out = torch.empty((M, V), dtype=torch.float32, device=x.device)
        cand = torch.empty((M, LM_HEAD_BLOCKS, 2), dtype=torch.int32, device=x.device)
        rc = lib.lyp_lm_head(_p(x), _p(w), _p(out), _code(x.dtype), M, V, K, x.stride(0), w.stride(0), out.stride(0),
                             _p(cand), LM_HEAD_BLOCKS, _stream())
        if rc < 0:
            _check(rc, lib)
        if rc > 0:
            return out, (cand if rc == LM_HEAD_BLOCKS else cand.view(-1)[:M * rc * 2].view(M, rc, 2))
    return linear(x, w, out_dtype=torch.float32), None


def sum_parts(parts: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Add up the partial sums ``linear(..., may_split=True)`` may return (slice
    by slice, in 32-bit), as a tensor [rows, features] of ``dtype``."""
    if parts.dim() == 2:
        return parts if parts.dtype == dtype else cast(parts, dtype)
    if parts.dim() != 3 or parts.dtype != torch.float32:
        raise KernelError(f"sum_parts: float partial sums [slices, rows, features], not {tuple(parts.shape)} {parts.dtype}")
    _dev(parts)
    out = torch.empty(parts.shape[1:], dtype=dtype, device=parts.device)
    lib = core()
    _check(lib.lyp_sum_parts(_p(parts), parts.shape[0], out.numel(), _p(out), _code(dtype), _stream()), lib)
    return out


def gemm_nt_heads(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[:, g, :] = a[:, g, :] @ w[g].T for every head g in one launch: a [M, G, K], w [G, N, K],
    out [M, G, N] of a's dtype or float; views into wider tensors are fine as long as the last
    dimension's values are neighbours."""
    M, G, K = a.shape
    N = w.shape[1]
    if tuple(w.shape) != (G, N, K) or tuple(out.shape) != (M, G, N) or a.dtype != w.dtype or \
            out.dtype not in (a.dtype, torch.float32):
        raise KernelError(f"gemm_nt_heads: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}, out {tuple(out.shape)}")
    for name, t in (("a", a), ("w", w), ("out", out)):
        if not t.is_cuda or t.stride(2) != 1:
            raise KernelError(f"gemm_nt_heads: {name} {tuple(t.shape)} with strides {t.stride()} on {t.device}")
    mode = STORE_ACT if out.dtype == a.dtype else STORE_F32
    lib = core()
    _check(lib.lyp_gemm_nt_batched(_p(a), _p(w), _p(out), _code(a.dtype), mode, G, M, N, K, a.stride(0), w.stride(1),
                                   out.stride(0), a.stride(1), w.stride(0), out.stride(1), _stream()), lib)
    return out


# ------------------------------------------- branches with norms, filters, recurrences
def _f32(*ts) -> None:
    for t in ts:
        if t is not None and t.dtype != torch.float32:
            raise KernelError(f"small parameter vectors are kept in float32, got {t.dtype}")


def branch_join(h: torch.Tensor, y: torch.Tensor | None, branch_weight: torch.Tensor | None, mult: float,
                eps_branch: float, *, shift: torch.Tensor | None = None, next_weight: torch.Tensor | None = None,
                eps_next: float = 0.0, out: torch.Tensor | None = None, rows: torch.Tensor | None = None,
                conv: tuple | None = None):
    """h += mult * rmsnorm(y) * branch_weight (+ shift, a vector added to every row), in 32-bit on the
    residual stream; with ``next_weight`` the sum's RMS norm times that weight goes to ``out``
    (activations); ``out`` without ``next_weight`` receives the joined rows themselves in its type (for
    a consumer that reads the stream as it is).  ``rows`` picks the rows to join and norm into ``out`` and leaves h alone.
    y [T, H] in the activations' type or float; None: only shift and norm.
    ``conv`` = (w, state, slots, positions), as ``short_conv`` takes them, for a step in which every
    row is a request of its own that brings one token: the normed rows then pass the short
    convolution in the same kernel (``branch_join_takes_conv`` says for which sizes)."""
    _dev(h, y, branch_weight, shift, next_weight, out, rows)
    _f32(branch_weight, shift, next_weight)
    cw = cstate = cslots = cpos = None
    taps = 1
    if conv is not None:
        cw, cstate, cslots, cpos = conv
        _dev(cw, cstate, cslots, cpos)
        _f32(cw)
        taps = cw.shape[1]
        if not branch_join_takes_conv(h.shape[1]) or rows is not None or next_weight is None or \
                tuple(cw.shape) != (h.shape[1], taps) or cslots.numel() != h.shape[0] or cpos.numel() != h.shape[0] or \
                (taps > 1 and (cstate is None or cstate.dtype != out.dtype or tuple(cstate.shape[1:]) != (taps - 1, h.shape[1]))):
            raise KernelError("branch_join: the convolution's operands do not fit the step")
    T, H = h.shape
    n = T if rows is None else rows.numel()
    if h.dtype != torch.float32 or (y is not None and (tuple(y.shape) != (T, H) or branch_weight is None or
                                                       branch_weight.numel() != H)):
        raise KernelError(f"branch_join: h {tuple(h.shape)} {h.dtype}, y {None if y is None else tuple(y.shape)}")
    if (shift is not None and shift.numel() != H) or (next_weight is not None and next_weight.numel() != H):
        raise KernelError("branch_join: shift and the following norm's weights have one value per feature")
    if (next_weight is not None and out is None) or (out is not None and tuple(out.shape) != (n, H)):
        raise KernelError("branch_join: the following norm needs an output of one row per joined row")
    if rows is not None and (rows.dtype != torch.int32 or out is None):
        raise KernelError("branch_join: rows are int32 and only picked for an output")
    lib = core()
    _check(lib.lyp_branch_join(_p(h), _p(y), _code(y.dtype) if y is not None else 0, _p(branch_weight), float(mult),
                               _p(shift), _p(next_weight), _p(out), _code(out.dtype) if out is not None else 0,
                               _p(rows), n, H, float(eps_branch), float(eps_next), _p(cw), _p(cstate), _p(cslots),
                               _p(cpos), taps, _stream()), lib)
    return out


def branch_join_takes_conv(H: int) -> bool:
    """Whether ``branch_join`` can carry the short convolution of a decode step's rows of H values."""
    return H % 4 == 0 and H <= 16384


def add_row(h: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """h[t, :] += v for every row of the float residual stream."""
    _dev(h, v)
    _f32(h, v)
    if v.numel() != h.shape[1]:
        raise KernelError(f"add_row: {v.numel()} values for rows of {h.shape[1]}")
    lib = core()
    _check(lib.lyp_add_row(_p(h), _p(v), h.shape[0], h.shape[1], _stream()), lib)
    return h


def _rows_view(t: torch.Tensor, what: str) -> None:
    """A 2-d GPU tensor whose rows' values are neighbours (a column range of a wider tensor is fine)."""
    if t is None or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1 or t.stride(0) < t.shape[1]:
        raise KernelError(f"{what}: a 2-d GPU tensor whose rows' values are neighbours, not "
                          f"{None if t is None else (tuple(t.shape), t.stride(), str(t.device))}")


def short_conv(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor | None, q_start: torch.Tensor,
               positions: torch.Tensor, slots: torch.Tensor, out: torch.Tensor, B: int, residual: bool = True,
               silu: bool = False, bias: torch.Tensor | None = None):
    """out = (x +) the causal filter of x over time, channel by channel, request by request:
    w float [C, taps]; ``state`` [slots, taps - 1, C] of x's type holds every request's last inputs
    from earlier steps (not read for a request at position 0) and is brought up to date.  x may be a
    column range of a wider tensor; ``bias`` (float [C]) is added to the filter's sum; ``silu``: the
    result passes x * sigmoid(x)."""
    _rows_view(x, "short_conv")
    _dev(w, state, q_start, positions, slots, out, bias)
    _f32(w, bias)
    if bias is not None and bias.numel() != x.shape[1]:
        raise KernelError(f"short_conv: a bias of {bias.numel()} values for {x.shape[1]} channels")
    T, C = x.shape
    taps = w.shape[1]
    if tuple(w.shape) != (C, taps) or out.shape != x.shape or out.dtype != x.dtype or out.data_ptr() == x.data_ptr():
        raise KernelError(f"short_conv: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} {out.dtype}")
    if taps > 1 and (state is None or state.dtype != x.dtype or tuple(state.shape[1:]) != (taps - 1, C)):
        raise KernelError(f"short_conv: state {None if state is None else tuple(state.shape)} for {taps} taps of {C}")
    if q_start.numel() != B + 1 or slots.numel() != B or positions.numel() != T:
        raise KernelError("short_conv: the step's tables do not fit its rows and requests")
    lib = core()
    _check(lib.lyp_short_conv(_p(x), _p(w), _p(state), _p(q_start), _p(positions), _p(slots), _p(out), _code(x.dtype),
                              T, B, C, taps, int(residual), x.stride(0), int(silu), _p(bias), _stream()), lib)
    return out


ACTIVATIONS = {"xielu": 0, "gelu_tanh": 1}


def activation(x: torch.Tensor, kind: str, params: torch.Tensor | None = None,
               out: torch.Tensor | None = None) -> torch.Tensor:
    """Elementwise activation in 32-bit: "xielu" (params: its two learned numbers, float) or
    "gelu_tanh".  In place unless ``out`` is given."""
    out = x if out is None else out
    _dev(x, params, out)
    _f32(params)
    if kind not in ACTIVATIONS or out.shape != x.shape or out.dtype != x.dtype or (kind == "xielu" and (
            params is None or params.numel() != 2)):
        raise KernelError(f"activation {kind!r} on {tuple(x.shape)} {x.dtype}")
    lib = core()
    _check(lib.lyp_activation(_p(x), _p(out), _code(x.dtype), x.numel(), ACTIVATIONS[kind], _p(params), _stream()), lib)
    return out


def mingru_scan(pre: torch.Tensor, bz: torch.Tensor, bx: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor,
                positions: torch.Tensor, slots: torch.Tensor, out: torch.Tensor, B: int,
                workspace: torch.Tensor | None = None) -> torch.Tensor:
    """The minGRU recurrence over the step's rows, request by request: pre float [T, 3 W] holds the
    update-gate, candidate and output-gate projections side by side; state float [slots, W].
    Without a workspace a thread walks all rows of its request and channel (steps of few rows per
    request); with one (``mingru_scan_workspace`` floats) the rows go in chunks of 32 that run side by
    side: a pass for every chunk's summary, a pass for the outputs (the recurrence is linear in the state)."""
    _dev(pre, bz, bx, state, q_start, positions, slots, out)
    _f32(pre, bz, bx, state)
    T, W = out.shape
    if tuple(pre.shape) != (T, 3 * W) or bz.numel() != W or bx.numel() != W or state.shape[1] != W or \
            q_start.numel() != B + 1 or slots.numel() != B or positions.numel() != T:
        raise KernelError(f"mingru_scan: pre {tuple(pre.shape)}, out {tuple(out.shape)}, state {tuple(state.shape)}")
    lib = core()
    if workspace is not None:
        _dev(workspace)
        _f32(workspace)
        if workspace.numel() < mingru_scan_workspace(T, B, W):
            raise KernelError("mingru_scan: workspace too small")
        _check(lib.lyp_mingru_scan_chunks(_p(pre), _p(bz), _p(bx), _p(state), _p(q_start), _p(positions), _p(slots),
                                          _p(out), _code(out.dtype), T, B, W, _p(workspace), workspace.numel(),
                                          _stream()), lib)
        return out
    _check(lib.lyp_mingru_scan(_p(pre), _p(bz), _p(bx), _p(state), _p(q_start), _p(positions), _p(slots), _p(out),
                               _code(out.dtype), B, W, _stream()), lib)
    return out


def mingru_scan_workspace(T: int, B: int, W: int) -> int:
    """Floats of the workspace with which ``mingru_scan`` walks a step's rows in chunks of 32."""
    return (2 * (-(-T // 32) + B) + B) * W


def latent_prep(d: torch.Tensor, wq: torch.Tensor, wkv: torch.Tensor, positions: torch.Tensor,
                table: torch.Tensor | None, slot_map: torch.Tensor, cq: torch.Tensor, pages: torch.Tensor, *,
                q_rank: int, kv_rank: int, rot_dim: int, eps: float) -> None:
    """From the down-projections of a step's rows (d [T, q_rank + kv_rank + rot_dim]): the normed
    query latent into cq, and the normed key/value latent with the position-rotated shared key part
    into each token's page slot (pages [pages, page size, kv_rank + rot_dim])."""
    _dev(d, wq, wkv, positions, table, slot_map, cq, pages)
    _f32(wq, wkv, table)
    T = d.shape[0]
    dims = 0 if table is None else table.shape[1]
    if d.shape[1] != q_rank + kv_rank + rot_dim or tuple(cq.shape) != (T, q_rank) or cq.dtype != d.dtype or \
            pages.dtype != d.dtype or pages.dim() != 3 or pages.shape[2] != kv_rank + rot_dim or \
            wq.numel() != q_rank or wkv.numel() != kv_rank or positions.numel() != T or slot_map.numel() != T:
        raise KernelError(f"latent_prep: d {tuple(d.shape)}, cq {tuple(cq.shape)}, pages {tuple(pages.shape)}")
    lib = core()
    _check(lib.lyp_latent_prep(_p(d), d.stride(0), _p(wq), _p(wkv), _p(positions), _p(table), dims, _p(slot_map),
                               _p(cq), _p(pages), _code(d.dtype), T, q_rank, kv_rank, rot_dim, float(eps),
                               _stream()), lib)


def latent_query_rotate(q: torch.Tensor, positions: torch.Tensor, table: torch.Tensor | None, qa: torch.Tensor, *,
                        num_heads: int, dim: int, rot_dim: int, kv_rank: int) -> None:
    """The rotated part of every query head (q [T, H (dim + rot_dim)], the last rot_dim of each head),
    turned by the token's position, into qa[:, head, kv_rank:] (qa [T, H, kv_rank + rot_dim])."""
    _dev(q, positions, table, qa)
    _f32(table)
    T = q.shape[0]
    dims = 0 if table is None else table.shape[1]
    if q.shape[1] != num_heads * (dim + rot_dim) or tuple(qa.shape) != (T, num_heads, kv_rank + rot_dim) or \
            qa.dtype != q.dtype or positions.numel() != T:
        raise KernelError(f"latent_query_rotate: q {tuple(q.shape)}, qa {tuple(qa.shape)}")
    lib = core()
    _check(lib.lyp_latent_query_rotate(_p(q), _p(positions), _p(table), dims, _p(qa), _code(q.dtype), T, num_heads,
                                       dim, rot_dim, kv_rank, _stream()), lib)


def latent_attn_rows(qa: torch.Tensor, pages: torch.Tensor, block_tables: torch.Tensor, q_start: torch.Tensor,
                     positions: torch.Tensor, ctx_len: torch.Tensor, sink: torch.Tensor, scale: float,
                     out: torch.Tensor, *, kv_rank: int, rot_dim: int) -> torch.Tensor:
    """Causal attention of every row over its request's latents in the pages, all heads sharing one
    key per token (the page row) whose first kv_rank values are also the value; the softmax's
    denominator holds exp(sink[head]) as well.  Any sizes; a workgroup per (row, head)."""
    _dev(qa, pages, block_tables, q_start, positions, ctx_len, sink, out)
    _f32(sink)
    T, H, Dk = qa.shape
    B = ctx_len.numel()
    if Dk != kv_rank + rot_dim or pages.dim() != 3 or pages.shape[2] != Dk or pages.dtype != qa.dtype or \
            tuple(out.shape) != (T, H, kv_rank) or out.dtype != qa.dtype or sink.numel() != H or \
            block_tables.dtype != torch.int32 or block_tables.dim() != 2 or block_tables.shape[0] != B or \
            q_start.numel() != B + 1 or positions.numel() != T:
        raise KernelError(f"latent_attn_rows: qa {tuple(qa.shape)}, pages {tuple(pages.shape)}, out {tuple(out.shape)}")
    lib = core()
    _check(lib.lyp_latent_attn_rows(_p(qa), _p(pages), _p(block_tables), block_tables.shape[1], pages.shape[1],
                                    _p(q_start), _p(positions), _p(ctx_len), B, _p(sink), float(scale), _p(out),
                                    _code(qa.dtype), T, H, kv_rank, rot_dim, _stream()), lib)
    return out


_latent: dict = {}


def latent_lib(kv_rank: int, rot_dim: int) -> ctypes.CDLL:
    lib = _latent.get((kv_rank, rot_dim))
    if lib is None:
        lib = _load(build.latent_attention_library(kv_rank, rot_dim))
        lib.lyp_last_error.restype = ctypes.c_char_p
        if (lib.lyp_latent_kv_rank(), lib.lyp_latent_rot_dim()) != (kv_rank, rot_dim):
            raise KernelError(f"latent attention library for sizes {kv_rank}, {rot_dim} reports others")
        lib.lyp_latent_plan.argtypes = [c_int, c_int, c_int]
        lib.lyp_latent_tile_keys.argtypes = [c_int]
        lib.lyp_latent_attn.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                        c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                        c_void_p, c_void_p, c_int, c_void_p]
        lib.lyp_latent_heads_out.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                             c_int, c_int, c_int, c_void_p]
        _latent[(kv_rank, rot_dim)] = lib
    return lib


def latent_attn_fits_matrix_cores(kv_rank: int, rot_dim: int) -> bool:
    return kv_rank % 16 == 0 and rot_dim % 16 == 0 and 16 <= kv_rank <= 512 and rot_dim <= 256


def latent_attn_launch(T: int, B: int, H: int, max_ctx: int, dtype: torch.dtype, kv_rank: int, rot_dim: int,
                       n_parts: int | None = None) -> dict:
    """The launch shape of ``latent_attn`` for a step of T rows of B requests with contexts of up
    to max_ctx: row groups, partitions of the keys, keys per partition, and the floats of the
    partitions' workspaces (host values only)."""
    lib = latent_lib(kv_rank, rot_dim)
    code = _code(dtype)
    row_groups = -(-T * H // 64) + B
    tile = lib.lyp_latent_tile_keys(code)
    if n_parts is None:
        n_parts = lib.lyp_latent_plan(row_groups, max_ctx, code)
    part_keys = max(tile, -(-(-(-max_ctx // n_parts)) // tile) * tile)
    n_parts = max(1, -(-max_ctx // part_keys))
    n = T * H * n_parts if n_parts > 1 else 0
    return dict(row_groups=row_groups, n_parts=n_parts, part_keys=part_keys, part_o=n * kv_rank, part_ml=n * 2)


def latent_attn(qa: torch.Tensor, pages: torch.Tensor, block_tables: torch.Tensor, q_start: torch.Tensor,
                positions: torch.Tensor, ctx_len: torch.Tensor, sink: torch.Tensor, scale: float, out: torch.Tensor,
                launch: dict, part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None, *,
                kv_rank: int, rot_dim: int, merge: bool = True) -> torch.Tensor:
    """``latent_attn_rows`` on the matrix cores (sizes in multiples of 16), a prompt's rows and
    single tokens alike; ``launch`` comes from ``latent_attn_launch`` for a bound on the step's
    contexts that the caller guarantees (keys beyond n_parts * part_keys would be left out).
    ``merge=False``: with several partitions ``out`` is left unwritten and the partitions' results
    stay in ``part_o`` / ``part_ml`` for ``latent_heads_out`` to merge."""
    _dev(qa, pages, block_tables, q_start, positions, ctx_len, sink, out, part_o, part_ml)
    _f32(sink, part_o, part_ml)
    T, H, Dk = qa.shape
    B = ctx_len.numel()
    if Dk != kv_rank + rot_dim or pages.dim() != 3 or pages.shape[2] != Dk or pages.dtype != qa.dtype or \
            tuple(out.shape) != (T, H, kv_rank) or out.dtype != qa.dtype or sink.numel() != H or \
            block_tables.dtype != torch.int32 or block_tables.dim() != 2 or block_tables.shape[0] != B or \
            q_start.numel() != B + 1 or positions.numel() != T or launch["row_groups"] < -(-T * H // 64) + B:
        raise KernelError(f"latent_attn: qa {tuple(qa.shape)}, pages {tuple(pages.shape)}, out {tuple(out.shape)}")
    if launch["n_parts"] > 1 and (part_o is None or part_ml is None or part_o.numel() < launch["part_o"]
                                  or part_ml.numel() < launch["part_ml"]):
        raise KernelError("latent_attn: the partitions' workspace is missing or too small")
    lib = latent_lib(kv_rank, rot_dim)
    _check(lib.lyp_latent_attn(_p(qa), _p(pages), _p(block_tables), block_tables.shape[1], pages.shape[1], _p(q_start),
                               _p(positions), _p(ctx_len), B, _p(sink), float(scale), _p(out), _code(qa.dtype), T, H,
                               launch["row_groups"], launch["n_parts"], launch["part_keys"], _p(part_o), _p(part_ml),
                               int(merge), _stream()), lib)
    return out


HEADS_OUT_MAX_ROWS = 512    # (token, head) rows up to which the merge and the value projection are one kernel


def latent_heads_out(w: torch.Tensor, out: torch.Tensor, *, kv_rank: int, rot_dim: int, mixed: torch.Tensor | None = None,
                     part_o: torch.Tensor | None = None, part_ml: torch.Tensor | None = None,
                     sink: torch.Tensor | None = None, n_parts: int = 1) -> torch.Tensor:
    """For a step of few rows: out[t, h, :] = w[h] @ (the latent sums of row (t, h)), w [H, vdim,
    kv_rank], the sums either merged here from the partitions ``latent_attn(..., merge=False)``
    left (with the sink), or read from ``mixed`` [T, H, kv_rank]."""
    _dev(w, out, mixed, part_o, part_ml, sink)
    _f32(part_o, part_ml, sink)
    T, H, vdim = out.shape
    if tuple(w.shape) != (H, vdim, kv_rank) or w.dtype != out.dtype or (mixed is None) == (part_o is None) or \
            (mixed is not None and (tuple(mixed.shape) != (T, H, kv_rank) or mixed.dtype != out.dtype)) or \
            (part_o is not None and (part_ml is None or sink is None or part_o.numel() < T * H * n_parts * kv_rank
                                     or part_ml.numel() < T * H * n_parts * 2 or sink.numel() != H)):
        raise KernelError(f"latent_heads_out: w {tuple(w.shape)}, out {tuple(out.shape)}")
    lib = latent_lib(kv_rank, rot_dim)
    _check(lib.lyp_latent_heads_out(_p(part_o), _p(part_ml), _p(sink), _p(mixed), _p(w), _p(out), _code(out.dtype),
                                    T * H, H, n_parts, vdim, _stream()), lib)
    return out


# ------------------------------------------------------------------- attention
def attn_decode_plan(n_seqs: int, max_ctx: int, num_heads: int, num_kv_heads: int, head_dim: int) -> int:
    """Keys per workgroup (the partition size) for a decode launch of this size."""
    return attention_lib(head_dim).lyp_attn_decode_plan(n_seqs, max_ctx, num_heads, num_kv_heads)


def attn_prefill_plan(n_tiles: int, max_keys: int, num_heads: int, num_kv_heads: int, head_dim: int,
                      dtype: torch.dtype, page_size: int) -> int:
    """Into how many runs a prefill launch had better cut every tile's keys
    (1: not at all) when one of its ``n_tiles`` tiles sees ``max_keys`` keys."""
    return attention_lib(head_dim).lyp_attn_prefill_plan(n_tiles, max_keys, num_heads, num_kv_heads, _code(dtype),
                                                         page_size)


def _sink_check(sink, num_heads: int) -> None:
    if sink is not None:
        _dev(sink)
        if sink.dtype != torch.float32 or sink.numel() != num_heads:
            raise KernelError(f"attention: the sinks are float, one per query head, not {tuple(sink.shape)} {sink.dtype}")


def _attn_check(q, out, kpool, vpool, block_tables, nh, nkv, hd):
    _dev(out, kpool, vpool, block_tables)
    n_pages, bs = kpool.shape[0], kpool.shape[2]
    if (tuple(kpool.shape) != (n_pages, nkv, bs, hd) or tuple(vpool.shape) != (n_pages, nkv, hd, bs)
            or kpool.dtype != q.dtype or vpool.dtype != q.dtype or out.dtype != q.dtype):
        raise KernelError(f"attention: pools {tuple(kpool.shape)} / {tuple(vpool.shape)} {kpool.dtype} do not fit "
                          f"{nkv} heads of {hd} and queries of {q.dtype}")
    if q.stride(1) != 1 or q.stride(0) < nh * hd or tuple(out.shape) != (q.shape[0], nh * hd):
        raise KernelError(f"attention: q {tuple(q.shape)} strides {q.stride()}, out {tuple(out.shape)}")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2:
        raise KernelError("attention: block tables must be a 2-d int32 tensor")
    return bs


def attn_prefill(q: torch.Tensor, out: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                 block_tables: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor, tile_seq: torch.Tensor,
                 tile_q0: torch.Tensor, n_tiles: int, *, num_heads: int, num_kv_heads: int, head_dim: int,
                 window: int = 0, scale: float | None = None, pair: bool | None = None,
                 split: bool = True, parts: int = 1, part_o: torch.Tensor | None = None,
                 part_ml: torch.Tensor | None = None, keep_first: int = 0,
                 sink: torch.Tensor | None = None, cap: float = 0.0,
                 slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of the step's new tokens over the paged cache (which already
    holds their own keys).  q is a view [T, >= nh * hd] whose first nh * hd
    columns are the query heads; a tile is 64 new tokens of one request, and
    the tiles are best listed in rising order of the keys they see.  ``pair``
    says whether the first tiles see far fewer keys than the last (then a
    workgroup may take one of each); None leaves it to the kernel's launcher.
    ``split=False`` keeps a small launch from sharing a tile's keys between
    two sets of waves (a different order of additions, for tests).  ``parts``
    > 1 (see ``attn_prefill_plan``) cuts every tile's keys into that many runs
    for workgroups of their own; it needs float workspaces ``part_o`` of
    n_tiles * 64 * heads * parts * head_dim and ``part_ml`` of n_tiles * 64 *
    heads * parts * 2 elements.  With a window, ``keep_first`` first tokens of a
    request stay visible whatever the distance; ``sink`` (float, one per query
    head) is a score without key or value that stands in the softmax's
    denominator once.  ``cap`` > 0 bends every score to cap * tanh(score / cap);
    ``slopes`` (float, one per query head) takes slopes[head] * (position - key)
    off the score of a key."""
    _sink_check(sink, num_heads)
    _sink_check(slopes, num_heads)
    _dev(slopes)
    if not q.is_cuda or q.dim() != 2:
        raise KernelError("attention: q must be a 2-d GPU tensor")
    bs = _attn_check(q, out, kpool, vpool, block_tables, num_heads, num_kv_heads, head_dim)
    _dev(q_start, ctx_len, tile_seq, tile_q0, part_o, part_ml)
    if parts > 1:
        need = n_tiles * 64 * num_heads * parts
        if part_o is None or part_ml is None or part_o.dtype != torch.float32 or part_ml.dtype != torch.float32 or \
                part_o.numel() < need * head_dim or part_ml.numel() < need * 2:
            raise KernelError("attention: the workspace for the parts of the keys is missing or too small")
    lib = attention_lib(head_dim)
    scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
    _check(lib.lyp_attn_prefill(_p(q), q.stride(0), _p(out), out.stride(0), _p(kpool), _p(vpool), _code(q.dtype),
                                _p(block_tables), block_tables.shape[1], _p(q_start), _p(ctx_len), _p(tile_seq),
                                _p(tile_q0), n_tiles, num_heads, num_kv_heads, bs, window, scale,
                                (1 if pair is None else int(bool(pair))) | (0 if split else 2), _p(part_o),
                                _p(part_ml), parts, int(keep_first), _p(sink), float(cap), _p(slopes), _stream()), lib)
    return out


def attn_decode(q: torch.Tensor, out: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                block_tables: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor,
                dec_seqs: torch.Tensor | None, n_seqs: int, part_o: torch.Tensor, part_ml: torch.Tensor,
                max_parts: int, part_keys: int, *, num_heads: int, num_kv_heads: int, head_dim: int, window: int = 0,
                scale: float | None = None, keep_first: int = 0, sink: torch.Tensor | None = None, cap: float = 0.0,
                slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of requests that bring one new token each, split over
    partitions of the context and merged.  ``part_keys`` comes from
    ``attn_decode_plan``; the caller guarantees that no request's context
    exceeds ``max_parts * part_keys`` (the contexts live on the device and are
    not read here: keys beyond that many partitions would silently be left
    out).  ``PagedAttention.decode_launch`` derives both from the step's bound.
    ``keep_first``, ``sink``, ``cap`` and ``slopes``: as for ``attn_prefill``."""
    _sink_check(sink, num_heads)
    _sink_check(slopes, num_heads)
    _dev(slopes)
    if not q.is_cuda or q.dim() != 2:
        raise KernelError("attention: q must be a 2-d GPU tensor")
    bs = _attn_check(q, out, kpool, vpool, block_tables, num_heads, num_kv_heads, head_dim)
    _dev(q_start, ctx_len, dec_seqs, part_o, part_ml)
    if part_o.dtype != torch.float32 or part_ml.dtype != torch.float32 or \
            part_o.numel() < n_seqs * num_heads * max_parts * head_dim or \
            part_ml.numel() < n_seqs * num_heads * max_parts * 2:
        raise KernelError("attention: partition workspace too small")
    lib = attention_lib(head_dim)
    scale = 1.0 / math.sqrt(head_dim) if scale is None else scale
    _check(lib.lyp_attn_decode(_p(q), q.stride(0), _p(out), out.stride(0), _p(kpool), _p(vpool), _code(q.dtype),
                               _p(block_tables), block_tables.shape[1], _p(q_start), _p(ctx_len), _p(dec_seqs),
                               n_seqs, _p(part_o), _p(part_ml), max_parts, part_keys, num_heads, num_kv_heads, bs,
                               window, scale, int(keep_first), _p(sink), float(cap), _p(slopes), _stream()), lib)
    return out


# ------------------------------- normed projections, windows with kept tokens, sinks
def qk_norm_rope_kv(qkv: torch.Tensor, q_norm: torch.Tensor | None, k_norm: torch.Tensor | None, eps: float,
                    positions: torch.Tensor, table: torch.Tensor | None, slots: torch.Tensor | None,
                    kpool: torch.Tensor | None, vpool: torch.Tensor | None, *, num_heads: int, num_kv_heads: int,
                    dim: int, vdim: int, page_size: int) -> None:
    """qkv [T, (H + G) dim + G vdim]: one RMS norm over each token's whole query projection and one
    over its whole key projection (``q_norm`` [H dim], ``k_norm`` [G dim], float; None: no norm),
    rotation of the pairs (2i, 2i+1) of the first ``table.shape[1]`` values of every query and key
    head by the token's position (table rows: cosines, then sines), queries back in place, keys and
    values into the tokens' page slots (keys [pages, G, page, dim], values [pages, G, vdim, page])."""
    _dev(qkv, q_norm, k_norm, positions, table, slots, kpool, vpool)
    _f32(q_norm, k_norm, table)
    T = qkv.shape[0]
    H, G = num_heads, num_kv_heads
    rot = 0 if table is None else table.shape[1]
    if qkv.shape[1] != (H + G) * dim + G * vdim or positions.numel() != T or positions.dtype != torch.int32 or \
            (q_norm is not None and q_norm.numel() != H * dim) or (k_norm is not None and k_norm.numel() != G * dim):
        raise KernelError(f"qk_norm_rope_kv: qkv {tuple(qkv.shape)} for {H}+{G} heads of {dim}/{vdim}")
    if slots is not None:
        n_pages = kpool.shape[0]
        if (slots.numel() != T or slots.dtype != torch.int32 or tuple(kpool.shape) != (n_pages, G, page_size, dim)
                or tuple(vpool.shape) != (n_pages, G, vdim, page_size) or kpool.dtype != qkv.dtype
                or vpool.dtype != qkv.dtype):
            raise KernelError(f"qk_norm_rope_kv: pools {tuple(kpool.shape)} / {tuple(vpool.shape)} {kpool.dtype} do "
                              f"not fit {G} heads of {dim}/{vdim}, pages of {page_size}, dtype {qkv.dtype}")
    lib = core()
    _check(lib.lyp_qk_norm_rope_kv(_p(qkv), qkv.stride(0), _code(qkv.dtype), _p(q_norm), _p(k_norm), float(eps),
                                   _p(positions), _p(table), rot, _p(slots), _p(kpool), _p(vpool), T, H, G, dim, vdim,
                                   page_size, _stream()), lib)


def attn_rows(q: torch.Tensor, out: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_tables: torch.Tensor,
              q_start: torch.Tensor, positions: torch.Tensor, ctx_len: torch.Tensor, *, num_heads: int,
              num_kv_heads: int, dim: int, vdim: int, scale: float, window: int = 0, keep_first: int = 0,
              sink: torch.Tensor | None = None, cap: float = 0.0, slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of every row of the step over its request's pages for any key and value size: q a
    view [T, >= H dim], out [T, H vdim].  A row at position p sees key j <= p when window == 0,
    p - j < window or j < keep_first.  ``cap`` > 0: scores become cap * tanh(score / cap);
    ``slopes`` (float [H]): key j's score loses slopes[head] * (p - j)."""
    _sink_check(sink, num_heads)
    _sink_check(slopes, num_heads)
    _dev(slopes)
    _dev(out, kpool, vpool, block_tables, q_start, positions, ctx_len)
    n_pages, bs = kpool.shape[0], kpool.shape[2]
    T = q.shape[0]
    if (not q.is_cuda or q.stride(1) != 1 or q.stride(0) < num_heads * dim
            or tuple(kpool.shape) != (n_pages, num_kv_heads, bs, dim) or tuple(vpool.shape) != (n_pages, num_kv_heads, vdim, bs)
            or tuple(out.shape) != (T, num_heads * vdim) or len({q.dtype, out.dtype, kpool.dtype, vpool.dtype}) != 1
            or block_tables.dtype != torch.int32 or block_tables.dim() != 2):
        raise KernelError(f"attn_rows: q {tuple(q.shape)}, out {tuple(out.shape)}, pools {tuple(kpool.shape)} / "
                          f"{tuple(vpool.shape)} for {num_heads}/{num_kv_heads} heads of {dim}/{vdim}")
    lib = core()
    _check(lib.lyp_attn_rows(_p(q), q.stride(0), _p(kpool), _p(vpool), _p(block_tables), block_tables.shape[1], bs,
                             _p(q_start), _p(positions), _p(ctx_len), q_start.numel() - 1, _p(sink), float(scale),
                             int(window), int(keep_first), _p(out), out.stride(0), _code(q.dtype), T, num_heads,
                             num_kv_heads, dim, vdim, float(cap), _p(slopes), _stream()), lib)
    return out


def stream_add(h: torch.Tensor, a, b: torch.Tensor | None = None) -> None:
    """h += a + b on the float residual stream: ``a`` what a layer left to be added (None, a tensor
    [T, H], float partial sums [S, T, H] or a product still to be run), ``b`` a float tensor [T, H]."""
    if isinstance(a, PendingLinear):
        a = a.run()
    _dev(h, a, b)
    parts = 0
    if a is not None:
        parts = a.shape[0] if a.dim() == 3 else 1
        if tuple(a.shape[-2:]) != tuple(h.shape) or (a.dim() == 3 and a.dtype != torch.float32):
            raise KernelError(f"stream_add: {tuple(a.shape)} {a.dtype} onto {tuple(h.shape)}")
    if h.dtype != torch.float32 or (b is not None and (b.dtype != torch.float32 or b.shape != h.shape)):
        raise KernelError("stream_add: the stream and what is added to it whole are float and of one shape")
    lib = core()
    _check(lib.lyp_stream_add(_p(h), _p(a), _code(a.dtype) if a is not None else 0, parts, _p(b), h.numel(),
                              _stream()), lib)


# ------------------------------------------------------------ routed feed-forward
def glu_clamped(gate_up: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """[T, 2 I] (gates first) -> [T, I]: g = min(gate, limit), u = clamp(up, -limit, limit);
    g * sigmoid(alpha * g) * (u + 1)."""
    _dev(gate_up)
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    lib = core()
    _check(lib.lyp_glu_clamped(_p(gate_up), _p(out), _code(gate_up.dtype), T, I, float(limit), float(alpha), _stream()), lib)
    return out


def moe_route(logits: torch.Tensor, bias: torch.Tensor | None, top: int, always: int = -1):
    """float router logits [T, E] (+ bias) -> (experts int32 [T, top], weights float [T, top]): the
    ``top`` largest (of equal ones the first) and the softmax over those alone.  ``always`` >= 0: one
    more pair a token, that expert with weight 1 (results are [T, top + 1])."""
    _dev(logits, bias)
    _f32(logits, bias)
    T, E = logits.shape
    per = top + (1 if always >= 0 else 0)
    idx = torch.empty((T, per), dtype=torch.int32, device=logits.device)
    wgt = torch.empty((T, per), dtype=torch.float32, device=logits.device)
    lib = core()
    _check(lib.lyp_moe_route(_p(logits), _p(bias), T, E, top, _p(idx), _p(wgt), int(always), _stream()), lib)
    return idx, wgt


ROUTE_SORT_MAX_ROWS = 64     # steps of up to this many rows choose and sort in one kernel


def moe_route_from(x: torch.Tensor, router: torch.Tensor, bias: torch.Tensor | None, top: int, always: int = -1,
                   sort_for: int = 0):
    """As ``moe_route`` from the router's input: x [T, K] activations, ``router`` [E, K] float; the
    logits x @ router.T are formed in 32-bit in the same kernel.  ``sort_for`` > 0 (the number of
    expert matrices, the always-used one included): also returns the ``MoePlan`` of the choices, as
    ``moe_sort`` makes it; with few rows the choice and the sort are one kernel."""
    _dev(x, router, bias)
    _f32(router, bias)
    T, K = x.shape
    E = router.shape[0]
    if router.shape[1] != K or x.stride(1) != 1:
        raise KernelError(f"moe_route_from: x {tuple(x.shape)}, router {tuple(router.shape)}")
    per = top + (1 if always >= 0 else 0)
    idx = torch.empty((T, per), dtype=torch.int32, device=x.device)
    wgt = torch.empty((T, per), dtype=torch.float32, device=x.device)
    lib = core()
    # few rows: several workgroups share the inner dimension and leave partial sums
    splits = lib.lyp_moe_route_splits(T, K)
    part = torch.empty((splits, T, E), dtype=torch.float32, device=x.device) if splits > 1 else None
    together = sort_for > 0 and splits > 1 and T <= ROUTE_SORT_MAX_ROWS
    _check(lib.lyp_moe_route_fused(_p(x), x.stride(0), _code(x.dtype), _p(router), _p(bias), T, E, K, top, _p(idx),
                                   _p(wgt), int(always), _p(part), splits, 0 if together else 1, _stream()), lib)
    if not sort_for:
        return idx, wgt
    return idx, wgt, MoePlan(idx, sort_for, route=(part, bias, top, always, wgt) if together else None)


class MoePlan:
    """Where the (token, choice) pairs of a step stand once sorted by expert, on the device."""

    def __init__(self, idx: torch.Tensor, E: int, route=None):
        """``route`` (partial sums [parts, T, experts], bias, top, always, weights): the choices are not
        made yet; the sort's kernel adds the router's partial sums up, chooses into ``idx`` and the
        weights, and sorts."""
        lib = core()
        self.pairs, self.top, self.E = idx.numel(), idx.shape[1], E
        self.tile_rows = lib.lyp_moe_tile_rows(self.pairs, E)
        self.most_tiles = lib.lyp_moe_most_tiles(self.pairs, E, self.tile_rows)
        # one allocation: expert offsets, pair at each place, place of each pair, tiles, their count
        sizes = (E + 1, self.pairs, self.pairs, self.most_tiles, self.most_tiles, 1)
        buf = torch.empty(sum(sizes), dtype=torch.int32, device=idx.device)
        views, at = [], 0
        for n in sizes:
            views.append(buf[at:at + n])
            at += n
        self.expert_off, self.sorted_pair, self.place_of, self.tile_expert, self.tile_row0, self.n_tiles = views
        if route is not None:
            part, bias, top, always, wgt = route
            _check(lib.lyp_moe_route_sort(_p(part), part.shape[0], _p(bias), part.shape[1], part.shape[2], top, always,
                                          _p(idx), _p(wgt), E, self.tile_rows, _p(self.expert_off), _p(self.sorted_pair),
                                          _p(self.place_of), _p(self.tile_expert), _p(self.tile_row0), _p(self.n_tiles),
                                          _stream()), lib)
            return
        _check(lib.lyp_moe_sort(_p(idx), self.pairs, E, self.tile_rows, _p(self.expert_off), _p(self.sorted_pair),
                                _p(self.place_of), _p(self.tile_expert), _p(self.tile_row0), _p(self.n_tiles),
                                _stream()), lib)


def moe_sort(idx: torch.Tensor, num_experts: int) -> MoePlan:
    _dev(idx)
    if idx.dtype != torch.int32 or idx.dim() != 2:
        raise KernelError("moe_sort: the chosen experts are int32 [tokens, top]")
    return MoePlan(idx, num_experts)


def moe_gemm(a: torch.Tensor, w: torch.Tensor, plan: MoePlan, *, gated: bool, limit: float = 0.0,
             alpha: float = 0.0, gather: bool = False, relu2: bool = False) -> torch.Tensor:
    """One product per expert over the rows sorted to it.  gated: a [T, K] (rows gathered by token),
    w [E, 2 N, K] (an expert's gate rows, then its up rows) -> [pairs, N], the gated activation of
    ``glu_clamped`` applied.  Otherwise a [pairs, K] in sorted order, w [E, N, K] -> [pairs, N]; with
    ``gather`` a is [T, K] and gathered by token as for a gated product, with ``relu2`` the result
    is max(y, 0)^2."""
    _dev(a, w)
    E, rows, K = w.shape
    N = rows // 2 if gated else rows
    if a.dtype != w.dtype or a.shape[1] != K or E != plan.E or (not gated and not gather and a.shape[0] != plan.pairs) \
            or (gated and (gather or relu2)):
        raise KernelError(f"moe_gemm: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} {w.dtype}, {plan.pairs} pairs")
    out = torch.empty((plan.pairs, N), dtype=a.dtype, device=a.device)
    lib = core()
    _check(lib.lyp_moe_gemm(_p(a), a.stride(0), _p(w), w.stride(0), w.stride(1), _p(out), out.stride(0), _code(a.dtype),
                            int(gated), _p(plan.tile_expert), _p(plan.tile_row0), _p(plan.n_tiles), plan.most_tiles,
                            plan.tile_rows, _p(plan.expert_off), _p(plan.sorted_pair), plan.top, N, K, float(limit),
                            float(alpha), int(gather) | 2 * int(relu2), _stream()), lib)
    return out


def moe_combine(y: torch.Tensor, plan: MoePlan, weights: torch.Tensor, rows: int, addend: torch.Tensor | None = None,
                shared: torch.Tensor | None = None) -> torch.Tensor:
    """float [1, rows, H]: addend + shared + sum over a token's choices of weight * y[place of the
    pair], added up in 32-bit in the order of the choices (one slice of partial sums, which a norm
    adds to the residual stream)."""
    _dev(y, weights, addend, shared)
    H = y.shape[1]
    for t in (addend, shared):
        if t is not None and (tuple(t.shape) != (rows, H) or t.dtype != y.dtype):
            raise KernelError(f"moe_combine: {tuple(t.shape)} {t.dtype} beside [{rows}, {H}] {y.dtype}")
    if weights.dtype != torch.float32 or weights.numel() != plan.pairs or rows * plan.top != plan.pairs:
        raise KernelError("moe_combine: weights do not fit the pairs")
    out = torch.empty((1, rows, H), dtype=torch.float32, device=y.device)
    lib = core()
    _check(lib.lyp_moe_combine(_p(y), _p(plan.place_of), _p(weights), plan.top, _p(addend), _p(shared), _p(out),
                               _code(y.dtype), rows, H, _stream()), lib)
    return out


def moe_route_grouped(x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor | None, top: int, groups: int,
                      keep: int, scale: float, on_matrix_cores: bool = True):
    """Sigmoid scores s = sigmoid(x @ router.T) in 32-bit (x [T, K] activations, router [E, K] float); the
    choice goes by s + correction among the experts of the ``keep`` best of ``groups`` equal groups of
    neighbours (a group's score: the sum of its two largest choice scores), the weights are the chosen
    experts' s over their sum, times ``scale``.  -> (experts int32 [T, top], weights float [T, top]).
    The logits come from the router's product kernel on the float matrix instruction (workgroups share
    the inner dimension and leave partial sums, which the choice's kernel adds up in their order);
    ``on_matrix_cores=False``: product and choice in one kernel of plain float sums, a wave a row."""
    _rows_view(x, "moe_route_grouped")
    _dev(router, correction)
    _f32(router, correction)
    T, K = x.shape
    E = router.shape[0]
    if router.shape[1] != K or (correction is not None and correction.numel() != E):
        raise KernelError(f"moe_route_grouped: x {tuple(x.shape)}, router {tuple(router.shape)}")
    idx = torch.empty((T, top), dtype=torch.int32, device=x.device)
    wgt = torch.empty((T, top), dtype=torch.float32, device=x.device)
    lib = core()
    if not on_matrix_cores:
        _check(lib.lyp_moe_route_grouped(_p(x), x.stride(0), _code(x.dtype), _p(router), _p(correction), T, E, K, top,
                                         int(groups), int(keep), float(scale), _p(idx), _p(wgt), _stream()), lib)
        return idx, wgt
    splits = max(2, lib.lyp_moe_route_splits(T, K))      # two shares at the least: the product then leaves its sums
    part = torch.empty((splits, T, E), dtype=torch.float32, device=x.device)
    _check(lib.lyp_moe_route_fused(_p(x), x.stride(0), _code(x.dtype), _p(router), None, T, E, K, top, _p(idx), _p(wgt), -1,
                                   _p(part), splits, 0, _stream()), lib)
    _check(lib.lyp_moe_choose_grouped(_p(part), splits, _p(correction), T, E, top, int(groups), int(keep), float(scale),
                                      _p(idx), _p(wgt), _stream()), lib)
    return idx, wgt


# ------------------------------------- grouped norms, scaled branches, gates, recurrences
class ScaledBranch:
    """A branch's output that joins the residual stream times a vector: h += y * scale.  ``y`` is
    [T, H] in the activations' type or float, or float partial sums [S, T, H]; ``scale`` float [H].
    A norm with ``takes_scaled`` does the sum in its own kernel; ``join(h)`` does it alone."""

    def __init__(self, y: torch.Tensor, scale: torch.Tensor):
        if isinstance(y, PendingLinear):
            y = y.run()
        self.y, self.scale = y, scale
        self.shape = y.shape

    def join(self, h: torch.Tensor) -> None:
        """Carry the sum out on h; nothing is left to add (returns None)."""
        group_rmsnorm(h, None, 1, 0.0, None, delta=self.y, scale=self.scale)
        return None


def group_rmsnorm(h: torch.Tensor, weight: torch.Tensor | None, groups: int, eps: float, out: torch.Tensor | None,
                  delta: torch.Tensor | None = None, scale: torch.Tensor | None = None,
                  rows: torch.Tensor | None = None):
    """h += scale * delta on the float residual stream (``delta`` [T, H] in the activations' type or
    float, or float partial sums [S, T, H]; ``scale`` float [H] or None), then out = every one of
    ``groups`` equal consecutive parts of a row over its own root mean square, the row times
    ``weight`` (float).  ``rows`` picks the rows to norm and leaves h alone; out None: the sum only."""
    _dev(h, weight, out, delta, scale, rows)
    _f32(h, weight, scale)
    T, H = h.shape
    n = T if rows is None else rows.numel()
    parts, stride = 0, 0
    if delta is not None:
        if delta.dim() == 3:
            if delta.dtype != torch.float32 or tuple(delta.shape[1:]) != (T, H):
                raise KernelError(f"group_rmsnorm: partial sums {tuple(delta.shape)} {delta.dtype} against h {tuple(h.shape)}")
            parts, stride = delta.shape[0], T * H
        elif tuple(delta.shape) != (T, H):
            raise KernelError(f"group_rmsnorm: delta {tuple(delta.shape)} against h {tuple(h.shape)}")
    if (scale is not None and scale.numel() != H) or (out is not None and (weight is None or weight.numel() != H or
                                                                           tuple(out.shape) != (n, H))):
        raise KernelError("group_rmsnorm: scale and weight have one value per feature, the output one row per normed row")
    if rows is not None and (rows.dtype != torch.int32 or out is None):
        raise KernelError("group_rmsnorm: rows are int32 and only picked for an output")
    lib = core()
    _check(lib.lyp_group_rmsnorm(_p(h), _p(delta), _code(delta.dtype) if delta is not None else 0, parts, stride,
                                 _p(scale), _p(weight), _p(out), _code(out.dtype) if out is not None else 0, _p(rows), n,
                                 H, int(groups), float(eps), _stream()), lib)
    return out


def add_sinusoid(h: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """h[t, 2i] += sin(p_t * base^(-2i/H)), h[t, 2i+1] += cos(the same) on a float tensor [T, H]."""
    _dev(h, positions)
    _f32(h)
    if positions.dtype != torch.int32 or positions.numel() != h.shape[0]:
        raise KernelError("add_sinusoid: one int32 position per row")
    lib = core()
    _check(lib.lyp_add_sinusoid(_p(h), _p(positions), h.shape[0], h.shape[1], float(base), _stream()), lib)
    return h


GLU_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def glu_act(gate_up: torch.Tensor, activation: str) -> torch.Tensor:
    """[T, 2 I] (a row's gates, then its ups) -> act(gate) * up [T, I]."""
    _dev(gate_up)
    if activation not in GLU_ACTIVATIONS or gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError(f"glu_act: {activation!r} on {tuple(gate_up.shape)}")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    lib = core()
    _check(lib.lyp_glu_act(_p(gate_up), _p(out), _code(gate_up.dtype), T, I, GLU_ACTIVATIONS[activation], _stream()), lib)
    return out


GATES = {"sigmoid": 0, "silu": 1}


def gate_mul(x: torch.Tensor, gate: torch.Tensor, kind: str, per: int = 1) -> torch.Tensor:
    """x *= sigmoid(gate) or silu(gate), in place: x [T, N] activations, gate [T, N / per] float or of
    x's type, possibly a column range of a wider tensor; one gate value serves ``per`` neighbouring
    values of x (a head's)."""
    _dev(x)
    _rows_view(gate, "gate_mul")
    if kind not in GATES or per < 1 or x.dim() != 2 or tuple(gate.shape) != (x.shape[0], x.shape[1] // per) or \
            x.shape[1] % per or gate.dtype not in (torch.float32, x.dtype):
        raise KernelError(f"gate_mul: {kind!r}, x {tuple(x.shape)} {x.dtype}, gate {tuple(gate.shape)} {gate.dtype}")
    lib = core()
    _check(lib.lyp_gate_mul(_p(x), _code(x.dtype), _p(gate), gate.stride(0), _code(gate.dtype), x.shape[0], x.shape[1],
                            GATES[kind], int(per), _stream()), lib)
    return x


def weighted_sum(a: torch.Tensor, sa: float, b: torch.Tensor, sb: float, bias: torch.Tensor | None = None) -> torch.Tensor:
    """float [1, T, H] (one slice of partial sums for the residual stream) = sa * (a + bias) + sb * b."""
    _dev(a, b, bias)
    _f32(bias)
    if a.shape != b.shape or a.dim() != 2 or (bias is not None and bias.numel() != a.shape[1]):
        raise KernelError(f"weighted_sum: {tuple(a.shape)} and {tuple(b.shape)}")
    T, H = a.shape
    out = torch.empty((1, T, H), dtype=torch.float32, device=a.device)
    lib = core()
    _check(lib.lyp_weighted_sum(_p(a), _code(a.dtype), _p(bias), float(sa), _p(b), _code(b.dtype), float(sb), _p(out), T, H,
                                _stream()), lib)
    return out


def qkv_bias_temper_kv(pre: torch.Tensor, bias: torch.Tensor | None, positions: torch.Tensor, coef: float, every: int,
                       slots: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, dtype: torch.dtype, *,
                       num_heads: int, num_kv_heads: int, dim: int, vdim: int, page_size: int) -> torch.Tensor:
    """From a float projection pre [T, >= (H + G) dim + G vdim] (queries, keys, values side by side):
    bias added, queries times 1 + coef * ln(floor((p + 1) / every) + 1) returned as [T, H dim] of
    ``dtype``, keys and values into the tokens' page slots (keys [pages, G, page, dim], values
    [pages, G, vdim, page])."""
    _rows_view(pre, "qkv_bias_temper_kv")
    _dev(bias, positions, slots, kpool, vpool)
    _f32(pre, bias)
    T = pre.shape[0]
    H, G = num_heads, num_kv_heads
    n = (H + G) * dim + G * vdim
    n_pages = kpool.shape[0]
    if pre.shape[1] < n or (bias is not None and bias.numel() != n) or positions.numel() != T or slots.numel() != T or \
            positions.dtype != torch.int32 or slots.dtype != torch.int32 or every < 1 or \
            tuple(kpool.shape) != (n_pages, G, page_size, dim) or tuple(vpool.shape) != (n_pages, G, vdim, page_size) or \
            kpool.dtype != dtype or vpool.dtype != dtype:
        raise KernelError(f"qkv_bias_temper_kv: pre {tuple(pre.shape)}, pools {tuple(kpool.shape)} / {tuple(vpool.shape)} "
                          f"{kpool.dtype} for {H}+{G} heads of {dim}/{vdim}, pages of {page_size}, dtype {dtype}")
    q = torch.empty((T, H * dim), dtype=dtype, device=pre.device)
    lib = core()
    _check(lib.lyp_qkv_bias_temper_kv(_p(pre), pre.stride(0), _p(bias), _p(positions), float(coef), int(every), _p(slots),
                                      _p(q), _p(kpool), _p(vpool), _code(dtype), T, H, G, dim, vdim, page_size,
                                      _stream()), lib)
    return q


LINEAR_SCAN_MAX_DIM = 512    # key channels a head of ``linear_scan`` may have


def linear_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, z: torch.Tensor, zbias: torch.Tensor | None,
                coef: torch.Tensor, sign: float, state: torch.Tensor, q_start: torch.Tensor, positions: torch.Tensor,
                slots: torch.Tensor, out: torch.Tensor, B: int, *, num_heads: int, num_kv_heads: int, dim: int,
                vdim: int, beta: torch.Tensor | None = None, unit: bool = False, q_scale: float = 1.0,
                bonus: torch.Tensor | None = None, z_per_head: bool = False, key_step: bool = False) -> torch.Tensor:
    """The recurrence with a matrix state per head over the step's rows, request by request, in order:
    S <- diag(g) S (+ the delta rule's correction when ``beta`` is given) + k v^T, out = S^T q, with
    g = exp(-coef[head] * softplus(sign * (z + zbias))); sign 0: z holds the decays themselves.  q, k [T, G dim] and v [T, H vdim] are
    activations (column ranges of wider tensors are fine), z float [T, H dim], beta [T, H] activations
    (before its sigmoid), state float [slots, H, vdim, dim] (a head's matrix transposed), out float
    [T, H vdim].  ``unit``: q and k become unit vectors per head first; q is multiplied by ``q_scale``.
    ``bonus`` (float [H dim]): the output reads the state before the token's decay and write, plus the
    token's own outer product weighted by the bonus per key channel: out = (S + diag(bonus) k v^T)^T q,
    then S <- diag(g) S + k v^T.  ``z_per_head``: z is [T, H] (zbias [H]), one decay for all of a
    head's key channels; with ``key_step`` the softplus inside that decay also multiplies the key
    (a step size: S <- g S + step k v^T)."""
    for t, what in ((q, "q"), (k, "k"), (v, "v"), (z, "z")) + (((beta, "beta"),) if beta is not None else ()):
        _rows_view(t, f"linear_scan {what}")
    _dev(zbias, coef, state, q_start, positions, slots, out, bonus)
    _f32(z, zbias, coef, state, out, bonus)
    zw = num_heads if z_per_head else num_heads * dim
    if (bonus is not None and (bonus.numel() != num_heads * dim or beta is not None)) or (key_step and not z_per_head):
        raise KernelError("linear_scan: a bonus has one value per head and key channel and no delta rule; a step "
                          "size comes with one decay per head")
    T = out.shape[0]
    H, G = num_heads, num_kv_heads
    if q.dtype != k.dtype or q.dtype != v.dtype or (beta is not None and beta.dtype != q.dtype) or \
            q.shape[0] != T or k.shape[0] != T or v.shape[0] != T or z.shape[0] != T or \
            q.shape[1] != G * dim or k.shape[1] != G * dim or v.shape[1] != H * vdim or z.shape[1] != zw or \
            (beta is not None and tuple(beta.shape) != (T, H)) or tuple(out.shape) != (T, H * vdim) or \
            tuple(state.shape[1:]) != (H, vdim, dim) or coef.numel() != H or \
            (zbias is not None and zbias.numel() != zw) or q_start.numel() != B + 1 or slots.numel() != B or \
            positions.numel() != T:
        raise KernelError(f"linear_scan: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}, z {tuple(z.shape)}, "
                          f"state {tuple(state.shape)}, out {tuple(out.shape)} for {H}/{G} heads of {dim}/{vdim}")
    lib = core()
    _check(lib.lyp_linear_scan(_p(q), q.stride(0), _p(k), k.stride(0), _p(v), v.stride(0), _code(q.dtype), _p(z),
                               z.stride(0), _p(zbias), _p(coef), float(sign), _p(beta),
                               beta.stride(0) if beta is not None else 0, _p(state), _p(q_start), _p(positions), _p(slots),
                               _p(out), out.stride(0), T, B, H, G, dim, vdim, int(beta is not None), int(unit),
                               float(q_scale), _p(bonus), int(z_per_head), int(key_step), _stream()), lib)
    return out


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, kind: str, eps: float,
                   dtype: torch.dtype, *, num_heads: int, vdim: int) -> torch.Tensor:
    """o float [T, H vdim]: every head divided by its root mean square over vdim, times ``weight``
    (float [vdim], shared by the heads, or [H vdim], every head its own), times sigmoid or silu of ``gate`` [T, H vdim] (float or of
    ``dtype``, possibly a column range); -> [T, H vdim] of ``dtype``."""
    _dev(o, weight)
    _rows_view(gate, "head_norm_gate")
    _f32(o, weight)
    T = o.shape[0]
    if kind not in GATES or tuple(o.shape) != (T, num_heads * vdim) or gate.shape != o.shape or \
            weight.numel() not in (vdim, num_heads * vdim) or \
            gate.dtype not in (torch.float32, dtype):
        raise KernelError(f"head_norm_gate: o {tuple(o.shape)}, gate {tuple(gate.shape)} {gate.dtype}, {num_heads} heads of {vdim}")
    out = torch.empty((T, num_heads * vdim), dtype=dtype, device=o.device)
    lib = core()
    _check(lib.lyp_head_norm_gate(_p(o), _p(weight), _p(gate), gate.stride(0), _code(gate.dtype), _p(out), _code(dtype), T,
                                  num_heads, vdim, float(eps), GATES[kind],
                                  int(weight.numel() != vdim), _stream()), lib)
    return out


def lowrank_up(mid: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
               decay_coef: torch.Tensor | None = None, decay_sign: float = 1.0, mid_tanh: bool = False,
               double_exp: bool = False) -> torch.Tensor:
    """float [T, N] = mid @ w.T (+ bias) in 32-bit: mid [T, R] activations (a column range is fine), w float [N, R].
    With ``decay_coef`` (float, one value per head of N / len values) the result y becomes the decay
    exp(-coef[head] * softplus(decay_sign * y)) that ``linear_scan`` takes with sign 0.  ``mid_tanh``:
    the inner values pass tanh first; ``double_exp``: the result y becomes the decay exp(-exp(y))."""
    _rows_view(mid, "lowrank_up")
    _dev(w, bias, decay_coef)
    _f32(w, bias, decay_coef)
    T, R = mid.shape
    N = w.shape[0]
    if w.shape[1] != R or (bias is not None and bias.numel() != N):
        raise KernelError(f"lowrank_up: mid {tuple(mid.shape)}, w {tuple(w.shape)}")
    out = torch.empty((T, N), dtype=torch.float32, device=mid.device)
    lib = core()
    heads = decay_coef.numel() if decay_coef is not None else 1
    if N % heads:
        raise KernelError(f"lowrank_up: {N} values do not split over {heads} heads")
    _check(lib.lyp_lowrank_up(_p(mid), mid.stride(0), _code(mid.dtype), _p(w), _p(bias), _p(out), T, N, R, _p(decay_coef),
                              float(decay_sign), N // heads, int(mid_tanh), int(double_exp), _stream()), lib)
    return out


def qkv_prepare(pre: torch.Tensor, dtype: torch.dtype, *, num_heads: int, num_kv_heads: int, dim: int, vdim: int,
                slots: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, page_size: int,
                bias: torch.Tensor | None = None, norm: str = "none", q_weight: torch.Tensor | None = None,
                k_weight: torch.Tensor | None = None, eps: float = 0.0, positions: torch.Tensor | None = None,
                table: torch.Tensor | None = None, pairing: str = "neighbours", values_from_keys: bool = False,
                blend: torch.Tensor | None = None, other_values: torch.Tensor | None = None,
                keep_values: bool = False):
    """From a float projection pre [T, >= (H + G) dim (+ G vdim)] (queries, keys and, unless the values
    are the keys, values side by side) to queries [T, H dim] of ``dtype`` (returned) and keys and
    values in the tokens' page slots: bias added; values taken (the biased key projection itself with
    ``values_from_keys``), blended with ``other_values`` (float [T, G vdim]) by the number in ``blend``
    (a float on the device: v <- (1 - b) v + b other) and, with ``keep_values``, returned unblended as
    float [T, G vdim]; queries and keys RMS-normed per head (``norm`` "head"; weights [dim] shared by
    the heads, or none) or over the whole projection ("whole"; weights over all of it); the first
    table.shape[1] values of every head turned by the position, pairs (2i, 2i + 1) ("neighbours") or
    (i, i + half) ("halves").  -> (q, kept values or None)."""
    _rows_view(pre, "qkv_prepare")
    _dev(bias, q_weight, k_weight, positions, table, slots, kpool, vpool, blend, other_values)
    _f32(pre, bias, q_weight, k_weight, table, blend, other_values)
    T, H, G = pre.shape[0], num_heads, num_kv_heads
    n = (H + G) * dim + (0 if values_from_keys else G * vdim)
    modes = {"none": 0, "head": 1, "whole": 2}
    pairings = {"neighbours": 0, "halves": 1}
    rot = table.shape[1] if table is not None else 0
    n_pages = kpool.shape[0]
    want_w = {0: (0, 0), 1: (dim, dim), 2: (H * dim, G * dim)}.get(modes.get(norm, -1))
    if norm not in modes or pairing not in pairings or pre.shape[1] < n or (bias is not None and bias.numel() != n) or \
            slots.numel() != T or slots.dtype != torch.int32 or (values_from_keys and vdim != dim) or \
            (rot and (positions is None or positions.numel() != T or positions.dtype != torch.int32)) or \
            any(w is not None and w.numel() != k for w, k in zip((q_weight, k_weight), want_w)) or \
            (blend is not None and (other_values is None or tuple(other_values.shape) != (T, G * vdim) or
                                    other_values.stride(1) != 1)) or \
            tuple(kpool.shape) != (n_pages, G, page_size, dim) or tuple(vpool.shape) != (n_pages, G, vdim, page_size) or \
            kpool.dtype != dtype or vpool.dtype != dtype:
        raise KernelError(f"qkv_prepare: pre {tuple(pre.shape)}, pools {tuple(kpool.shape)} / {tuple(vpool.shape)} "
                          f"{kpool.dtype} for {H}+{G} heads of {dim}/{vdim}, norm {norm!r}, pairing {pairing!r}, dtype {dtype}")
    q = torch.empty((T, H * dim), dtype=dtype, device=pre.device)
    kept = torch.empty((T, G * vdim), dtype=torch.float32, device=pre.device) if keep_values else None
    lib = core()
    _check(lib.lyp_qkv_prepare(_p(pre), pre.stride(0), _p(bias), modes[norm], _p(q_weight), _p(k_weight), float(eps),
                               _p(positions), _p(table), rot, pairings[pairing], int(values_from_keys), _p(blend),
                               _p(other_values), other_values.stride(0) if other_values is not None else 0, _p(kept),
                               _p(slots), _p(q), _p(kpool), _p(vpool), _code(dtype), T, H, G, dim, vdim, page_size,
                               _stream()), lib)
    return q, kept


def shift_mix(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, positions: torch.Tensor,
              slots: torch.Tensor, B: int) -> torch.Tensor:
    """[n, T, C] of x's type: for every row of ``mu`` (float [n, C]) the blend x_t + (x_(t-1) - x_t) * mu
    of each row with the row before it in its request; the row before a step's first is the request's
    state slot (``state`` [slots, C] of x's type; zeros for a request at position 0), which then takes
    the request's last row of this step."""
    _rows_view(x, "shift_mix")
    _dev(mu, state, q_start, positions, slots)
    _f32(mu)
    T, C = x.shape
    if mu.dim() != 2 or mu.shape[1] != C or state.dtype != x.dtype or tuple(state.shape[1:]) != (C,) or \
            q_start.numel() != B + 1 or slots.numel() != B or positions.numel() != T:
        raise KernelError(f"shift_mix: x {tuple(x.shape)}, mu {tuple(mu.shape)}, state {tuple(state.shape)} {state.dtype}")
    out = torch.empty((mu.shape[0], T, C), dtype=x.dtype, device=x.device)
    lib = core()
    _check(lib.lyp_shift_mix(_p(x), x.stride(0), _p(mu), mu.shape[0], _p(state), _p(q_start), _p(positions), _p(slots),
                             _p(out), _code(x.dtype), T, B, C, _stream()), lib)
    return out


def skip_gate_group_norm(o: torch.Tensor, x: torch.Tensor, skip: torch.Tensor, z: torch.Tensor, weight: torch.Tensor,
                         groups: int, eps: float, *, vdim: int) -> torch.Tensor:
    """[T, N] of x's type: y = (o + skip[head] * x) * silu(z), then every one of ``groups`` equal
    consecutive parts of y over its root mean square, times ``weight``.  o float [T, N]; x and z
    activations [T, N] (column ranges are fine); skip float [N / vdim]; weight float [N]."""
    _rows_view(x, "skip_gate_group_norm x")
    _rows_view(z, "skip_gate_group_norm z")
    _dev(o, skip, weight)
    _f32(o, skip, weight)
    T, N = o.shape
    if tuple(x.shape) != (T, N) or tuple(z.shape) != (T, N) or x.dtype != z.dtype or N % vdim or skip.numel() != N // vdim or \
            weight.numel() != N or groups < 1 or N % groups or not o.is_contiguous():
        raise KernelError(f"skip_gate_group_norm: o {tuple(o.shape)}, x {tuple(x.shape)}, z {tuple(z.shape)}, {groups} groups")
    out = torch.empty((T, N), dtype=x.dtype, device=x.device)
    lib = core()
    _check(lib.lyp_skip_gate_group_norm(_p(o), _p(x), x.stride(0), _p(skip), _p(z), z.stride(0), _p(weight), _p(out),
                                        _code(x.dtype), T, N, vdim, groups, float(eps), _stream()), lib)
    return out


def gather_gelu_mul(p: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """[T, N] of the table's type: gelu_tanh(p[t]) * table[tokens[t]], with p [T, N] float or of the
    table's type and table [vocab, N] (a column range of a wider table is fine)."""
    _rows_view(p, "gather_gelu_mul p")
    _rows_view(table, "gather_gelu_mul table")
    _dev(tokens)
    T, N = p.shape
    if table.shape[1] != N or tokens.numel() != T or tokens.dtype != torch.int32 or p.dtype not in (torch.float32, table.dtype):
        raise KernelError(f"gather_gelu_mul: p {tuple(p.shape)} {p.dtype}, table {tuple(table.shape)} {table.dtype}")
    out = torch.empty((T, N), dtype=table.dtype, device=p.device)
    lib = core()
    _check(lib.lyp_gather_gelu_mul(_p(p), p.stride(0), _code(p.dtype), _p(tokens), _p(table), table.stride(0),
                                   table.shape[0], _p(out), _code(table.dtype), T, N, _stream()), lib)
    return out



# -------------------------------------------------------------------- sampling
def sample_workspace(rows: int, device) -> torch.Tensor:
    return torch.empty(max(1, core().lyp_sample_workspace(rows)), dtype=torch.uint8, device=device)


def _pinned(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    if t.is_cuda or not t.is_pinned() or t.dtype != dtype or not t.is_contiguous():
        raise KernelError(f"{what} must be a contiguous pinned host tensor of {dtype}")


def table_load(src: torch.Tensor, dst: torch.Tensor, patch: torch.Tensor | None = None, patch_at: int = 0) -> None:
    """dst (int32, device) = the first dst.numel() words of src (int32, pinned
    host memory, read by the kernel itself: no copy engine, no second launch);
    ``patch`` (int32, device) replaces the words from ``patch_at`` on."""
    _pinned(src, torch.int32, "table_load: the source")
    _dev(dst, patch)
    if dst.dtype != torch.int32 or dst.numel() > src.numel() or not dst.is_contiguous():
        raise KernelError("table_load: the destination must be a contiguous int32 tensor no longer than the source")
    n_patch = 0
    if patch is not None:
        n_patch = patch.numel()
        if patch.dtype != torch.int32 or not patch.is_contiguous() or patch_at < 0 or patch_at + n_patch > dst.numel():
            raise KernelError("table_load: the patch does not fit")
    lib = core()
    _check(lib.lyp_table_load(src.data_ptr(), _p(dst), dst.numel(), _p(patch), patch_at, n_patch, _stream()), lib)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor | None = None,
           mirror: torch.Tensor | None = None, row_maxima: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row of logits.  With a ``workspace`` (``sample_workspace``)
    the search for each row's maximum is spread over the chip; with
    ``row_maxima`` (what ``lm_head`` returns beside these very logits) there is
    no search.  ``mirror``: pinned host memory (int32, a row each) that receives
    the tokens as well, readable once the work on the stream up to here is done."""
    _dev(temperature, top_k, top_p, uniform, out, workspace)
    if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be a 2-d GPU tensor whose rows are contiguous")
    if mirror is not None:
        _pinned(mirror, torch.int32, "sample: the mirror")
        if mirror.numel() != out.numel():
            raise KernelError("sample: one mirrored token per row")
    R, V = logits.shape
    if logits.dtype != torch.float32 or temperature.dtype != torch.float32 or top_k.dtype != torch.int32 or \
            top_p.dtype != torch.float32 or uniform.dtype != torch.float32 or out.dtype != torch.int32:
        raise KernelError("sample: logits, temperature, top_p, uniform float32; top_k, out int32")
    if any(t.numel() != R for t in (temperature, top_k, top_p, uniform, out)):
        raise KernelError("sample: one parameter per row")
    lib = core()
    cand = row_maxima
    if cand is not None:   # the head's kernel left the row maxima in pieces: no pass over the row for them
        if cand.dtype != torch.int32 or cand.dim() != 3 or cand.shape[0] < R or cand.shape[2] != 2 or \
                not cand.is_contiguous() or cand.device != logits.device:
            raise KernelError("sample: the row maxima must be a contiguous int32 tensor [rows, pieces, 2]")
        _check(lib.lyp_sample_cand(_p(logits), logits.stride(0), R, V, _p(temperature), _p(top_k), _p(top_p),
                                   _p(uniform), _p(cand), cand.shape[1], _p(out),
                                   mirror.data_ptr() if mirror is not None else None, _stream()), lib)
        return out
    if workspace is not None and workspace.numel() < lib.lyp_sample_workspace(R):
        raise KernelError("sample: workspace too small")
    _check(lib.lyp_sample(_p(logits), logits.stride(0), R, V, _p(temperature), _p(top_k), _p(top_p), _p(uniform),
                          _p(workspace), _p(out), mirror.data_ptr() if mirror is not None else None, _stream()), lib)
    return out
