"""ctypes binding of ``libjaxpp_amd.so`` (the C ABI in include/jaxpp_amd.h).

This is the host side for a process that has no GPU runtime of its own: it
owns device buffers through the library's allocation helpers and drives the
stage executor.  There is no CPU fallback: without the built library or
without a GPU every call raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Iterable

import numpy as np

from jaxpp_amd.types import TaskType

# JAXPP_AMD_LIB names another build of the library (A/B runs of two builds on one machine)
_LIB_PATH = os.environ.get("JAXPP_AMD_LIB") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "lib", "libjaxpp_amd.so")
_lib = None


class JppError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, code: int, msg: str):
        super().__init__(f"jaxpp_amd error {code}: {msg}")
        self.code = code


class GemmArgs(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("c", C.c_void_p), ("c2", C.c_void_p),
                ("bias", C.c_void_p), ("resid", C.c_void_p), ("aux", C.c_void_p),
                ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
                ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
                ("ldc2", C.c_int64), ("ldresid", C.c_int64), ("ldaux", C.c_int64),
                ("trans_a", C.c_int), ("trans_b", C.c_int), ("epilogue", C.c_int),
                ("gelu_tanh", C.c_int), ("tile", C.c_int),
                ("seg", C.c_void_p), ("n_seg", C.c_int), ("group_mode", C.c_int),
                ("stride_b", C.c_int64), ("stride_c", C.c_int64), ("group_rows", C.c_int64),
                ("seg_rows", C.c_void_p),
                ("a_more", C.c_void_p * 3), ("b_more", C.c_void_p * 3), ("k_parts", C.c_int),
                ("seg_more", C.c_void_p * 3), ("seg_rows_more", C.c_void_p * 3),
                ("rope_cos", C.c_void_p), ("rope_sin", C.c_void_p), ("rope_cols", C.c_int64),
                ("rope_seq", C.c_int), ("rope_head_dim", C.c_int)]


class AttnArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
                ("lse", C.c_void_p), ("d_o", C.c_void_p), ("dq", C.c_void_p),
                ("dk", C.c_void_p), ("dv", C.c_void_p), ("delta", C.c_void_p),
                ("ldq", C.c_int64), ("ldk", C.c_int64), ("ldv", C.c_int64), ("ldo", C.c_int64),
                ("lddo", C.c_int64), ("lddq", C.c_int64), ("lddk", C.c_int64),
                ("lddv", C.c_int64),
                ("batch", C.c_int), ("seq", C.c_int), ("n_heads", C.c_int),
                ("n_kv_heads", C.c_int), ("head_dim", C.c_int), ("causal", C.c_int),
                ("rope_cos", C.c_void_p), ("rope_sin", C.c_void_p)]


class NormArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("gamma", C.c_void_p), ("beta", C.c_void_p),
                ("y", C.c_void_p), ("mean", C.c_void_p), ("rstd", C.c_void_p),
                ("dy", C.c_void_p), ("resid", C.c_void_p), ("dx", C.c_void_p),
                ("dgamma", C.c_void_p), ("dbeta", C.c_void_p), ("partial", C.c_void_p),
                ("rows", C.c_int64), ("cols", C.c_int64), ("eps", C.c_float)]


class MoeArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("wr", C.c_void_p), ("ids", C.c_void_p), ("gates", C.c_void_p),
                ("row_of", C.c_void_p), ("tok_of", C.c_void_p), ("gate_of", C.c_void_p),
                ("seg", C.c_void_p), ("work", C.c_void_p), ("tokens", C.c_int64),
                ("hidden", C.c_int64), ("n_experts", C.c_int), ("top_k", C.c_int),
                ("dtype", C.c_int)]


class AdamArgs(C.Structure):
    _fields_ = [("count", C.c_int64), ("grad", C.c_void_p), ("master", C.c_void_p),
                ("param", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p), ("step", C.c_int64),
                ("lr", C.c_double), ("beta1", C.c_double), ("beta2", C.c_double),
                ("eps", C.c_double), ("grad_scale", C.c_double), ("zero_grad", C.c_int)]


class ColsumItem(C.Structure):
    _fields_ = [("x", C.c_void_p), ("ld", C.c_int64), ("cols", C.c_int64), ("acc", C.c_void_p)]


class StageDesc(C.Structure):
    _fields_ = [("family", C.c_int), ("hidden", C.c_int), ("n_heads", C.c_int),
                ("n_kv_heads", C.c_int), ("head_dim", C.c_int), ("ffn", C.c_int),
                ("seq", C.c_int), ("batch", C.c_int), ("causal", C.c_int),
                ("rope_theta", C.c_float), ("eps", C.c_float), ("gelu_tanh", C.c_int),
                ("n_experts", C.c_int), ("top_k", C.c_int), ("n_chunks", C.c_int),
                ("layers_per_chunk", C.c_int), ("max_live", C.c_int),
                ("split_backward", C.c_int), ("fused_wgrad_accum", C.c_int),
                ("two_streams", C.c_int), ("dtype", C.c_int), ("wgrad_group", C.c_int)]


EPI_BF16, EPI_GELU, EPI_DGELU, EPI_ACC_F32, EPI_F32, EPI_SWIGLU, EPI_DSWIGLU = range(7)
NORM_PARTIALS = 256
FAMILY = {"bert": 0, "llama": 1, "mixtral": 2, "decoder": 3}
DTYPE = {"bf16": 0, "f32": 1}

# every symbol include/jaxpp_amd.h declares
EXPORTS = [
    "jpp_last_error", "jpp_version", "jpp_device_count", "jpp_set_device", "jpp_malloc",
    "jpp_free", "jpp_memcpy_h2d", "jpp_memcpy_d2h", "jpp_memcpy_d2d_async", "jpp_fill_u32",
    "jpp_stream_create", "jpp_stream_destroy", "jpp_stream_sync", "jpp_stream_wait_event",
    "jpp_device_sync",
    "jpp_event_create", "jpp_event_destroy", "jpp_event_record", "jpp_event_sync",
    "jpp_event_elapsed_ms", "jpp_mem_info", "jpp_workspace_bytes", "jpp_graph_begin", "jpp_graph_end", "jpp_graph_launch",
    "jpp_graph_destroy", "jpp_probe_begin", "jpp_probe_end", "jpp_probe_class",
    "jpp_gemm_bf16", "jpp_gemm_bf16_multi", "jpp_attn_fwd", "jpp_attn_bwd",
    "jpp_gemm_f32", "jpp_attn_fwd_f32", "jpp_attn_bwd_f32", "jpp_norm_fwd_f32", "jpp_norm_bwd_f32",
    "jpp_colsum_accum_f32", "jpp_mse_loss_f32", "jpp_rope_f32",
    "jpp_norm_fwd", "jpp_norm_bwd", "jpp_norm_bwd_static", "jpp_swiglu_fwd", "jpp_swiglu_bwd", "jpp_rope",
    "jpp_grad_accum_f32", "jpp_sum_accum_f32", "jpp_colsum_accum", "jpp_colsum_accum_multi", "jpp_mse_loss", "jpp_moe_capacity", "jpp_moe_route",
    "jpp_moe_gather", "jpp_moe_combine_fwd", "jpp_moe_bwd_prepare", "jpp_moe_combine_bwd",
    "jpp_moe_router_wgrad", "jpp_cast_f32_to_bf16", "jpp_cast_bf16_to_f32", "jpp_adam_step",
    "jpp_stage_optimizer_init", "jpp_stage_opt_ptr", "jpp_stage_adam_step",
    "jpp_stage_create", "jpp_stage_destroy", "jpp_stage_n_params", "jpp_stage_param_info",
    "jpp_stage_param_ptr", "jpp_stage_grad_ptr", "jpp_stage_zero_grads", "jpp_stage_join",
    "jpp_stage_quiesce",
    "jpp_stage_bytes",
    "jpp_stage_run_task", "jpp_stage_live_slots", "jpp_stage_routing",
]


def lib_path() -> str:
    return _LIB_PATH


_diag = None


def load_diag():
    """The measurement aids (libjaxpp_amd_diag.so, next to the product library)."""
    global _diag
    if _diag is None:
        load()                                        # its error reporting lives there
        path = os.path.join(os.path.dirname(_LIB_PATH), "libjaxpp_amd_diag.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python -m jaxpp_amd.build`")
        _diag = C.CDLL(path)
        _diag.jpp_mfma_rate.argtypes = [C.c_int, C.c_int, C.c_int64, C.POINTER(C.c_double)]
        _diag.jpp_lds_read_rate.argtypes = [C.POINTER(C.c_uint32), C.c_int, C.POINTER(C.c_double)]
    return _diag


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python -m jaxpp_amd.build` "
            "(there is no fallback path)")
    lib = C.CDLL(_LIB_PATH)
    lib.jpp_last_error.restype = C.c_char_p
    lib.jpp_workspace_bytes.restype = C.c_size_t
    lib.jpp_workspace_bytes.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int64]
    lib.jpp_stage_bytes.restype = C.c_size_t
    lib.jpp_stage_bytes.argtypes = [C.c_void_p]
    lib.jpp_malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    lib.jpp_free.argtypes = [C.c_void_p]
    lib.jpp_memcpy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    lib.jpp_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    lib.jpp_memcpy_d2d_async.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
    lib.jpp_fill_u32.argtypes = [C.c_void_p, C.c_uint32, C.c_size_t, C.c_void_p]
    lib.jpp_stream_create.argtypes = [C.POINTER(C.c_void_p)]
    lib.jpp_stream_wait_event.argtypes = [C.c_void_p, C.c_void_p]
    lib.jpp_stream_destroy.argtypes = [C.c_void_p]
    lib.jpp_stream_sync.argtypes = [C.c_void_p]
    lib.jpp_event_create.argtypes = [C.POINTER(C.c_void_p)]
    lib.jpp_event_destroy.argtypes = [C.c_void_p]
    lib.jpp_event_record.argtypes = [C.c_void_p, C.c_void_p]
    lib.jpp_event_sync.argtypes = [C.c_void_p]
    lib.jpp_event_elapsed_ms.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]
    lib.jpp_mem_info.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    lib.jpp_graph_begin.argtypes = [C.c_void_p]
    lib.jpp_graph_end.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    lib.jpp_graph_launch.argtypes = [C.c_void_p, C.c_void_p]
    lib.jpp_graph_destroy.argtypes = [C.c_void_p]
    lib.jpp_probe_begin.argtypes = [C.c_char_p]
    lib.jpp_probe_end.argtypes = [C.POINTER(C.c_int64), C.POINTER(C.c_double),
                                  C.POINTER(C.c_double), C.POINTER(C.c_double)]
    lib.jpp_probe_class.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_int64),
                                    C.POINTER(C.c_double), C.POINTER(C.c_double),
                                    C.POINTER(C.c_double)]
    lib.jpp_gemm_bf16.argtypes = [C.c_void_p, C.POINTER(GemmArgs)]
    lib.jpp_gemm_bf16_multi.argtypes = [C.c_void_p, C.POINTER(GemmArgs), C.c_int]
    lib.jpp_attn_fwd.argtypes = [C.c_void_p, C.POINTER(AttnArgs)]
    lib.jpp_attn_bwd.argtypes = [C.c_void_p, C.POINTER(AttnArgs)]
    lib.jpp_norm_fwd.argtypes = [C.c_void_p, C.POINTER(NormArgs)]
    lib.jpp_norm_bwd.argtypes = [C.c_void_p, C.POINTER(NormArgs)]
    lib.jpp_norm_bwd_static.argtypes = [C.c_void_p, C.POINTER(NormArgs)]
    lib.jpp_gemm_f32.argtypes = [C.c_void_p, C.POINTER(GemmArgs)]
    lib.jpp_attn_fwd_f32.argtypes = [C.c_void_p, C.POINTER(AttnArgs)]
    lib.jpp_attn_bwd_f32.argtypes = [C.c_void_p, C.POINTER(AttnArgs)]
    lib.jpp_norm_fwd_f32.argtypes = [C.c_void_p, C.POINTER(NormArgs)]
    lib.jpp_norm_bwd_f32.argtypes = [C.c_void_p, C.POINTER(NormArgs)]
    lib.jpp_colsum_accum_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                         C.c_void_p]
    lib.jpp_rope_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int,
                                 C.c_int, C.c_int, C.c_int, C.c_int]
    lib.jpp_mse_loss_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_float,
                                     C.c_void_p, C.c_void_p]
    lib.jpp_swiglu_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                   C.c_int]
    lib.jpp_swiglu_bwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                   C.c_int64, C.c_int]
    lib.jpp_rope.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int,
                             C.c_int, C.c_int, C.c_int, C.c_int]
    lib.jpp_grad_accum_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
    lib.jpp_colsum_accum.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                     C.c_void_p, C.c_void_p]
    lib.jpp_sum_accum_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64]
    lib.jpp_colsum_accum_multi.argtypes = [C.c_void_p, C.c_int, C.POINTER(ColsumItem), C.c_int64,
                                           C.c_void_p]
    lib.jpp_mse_loss.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_float,
                                 C.c_void_p, C.c_void_p, C.c_void_p]
    lib.jpp_moe_capacity.restype = C.c_int64
    lib.jpp_moe_capacity.argtypes = [C.c_int64, C.c_int, C.c_int]
    lib.jpp_moe_route.argtypes = [C.c_void_p, C.POINTER(MoeArgs)]
    lib.jpp_moe_gather.argtypes = [C.c_void_p, C.POINTER(MoeArgs), C.c_void_p, C.c_void_p]
    lib.jpp_moe_combine_fwd.argtypes = [C.c_void_p, C.POINTER(MoeArgs), C.c_void_p, C.c_void_p,
                                        C.c_void_p]
    lib.jpp_moe_bwd_prepare.argtypes = [C.c_void_p, C.POINTER(MoeArgs), C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_void_p]
    lib.jpp_moe_combine_bwd.argtypes = [C.c_void_p, C.POINTER(MoeArgs), C.c_void_p, C.c_void_p,
                                        C.c_void_p]
    lib.jpp_moe_router_wgrad.argtypes = [C.c_void_p, C.POINTER(MoeArgs), C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_void_p]
    lib.jpp_cast_f32_to_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64]
    lib.jpp_cast_bf16_to_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64]
    lib.jpp_stage_create.argtypes = [C.POINTER(StageDesc), C.POINTER(C.c_void_p)]
    lib.jpp_stage_destroy.argtypes = [C.c_void_p]
    lib.jpp_stage_n_params.argtypes = [C.c_void_p]
    lib.jpp_stage_param_info.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_char_p),
                                         C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    lib.jpp_stage_param_ptr.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int,
                                        C.POINTER(C.c_void_p)]
    lib.jpp_stage_grad_ptr.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int,
                                       C.POINTER(C.c_void_p)]
    lib.jpp_stage_zero_grads.argtypes = [C.c_void_p, C.c_void_p]
    lib.jpp_stage_join.argtypes = [C.c_void_p, C.c_void_p]
    lib.jpp_stage_quiesce.argtypes = [C.c_void_p]
    lib.jpp_stage_run_task.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                       C.c_void_p, C.c_void_p]
    lib.jpp_stage_live_slots.argtypes = [C.c_void_p]
    lib.jpp_stage_routing.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                      C.c_void_p]
    lib.jpp_adam_step.argtypes = [C.c_void_p, C.POINTER(AdamArgs)]
    lib.jpp_stage_optimizer_init.argtypes = [C.c_void_p, C.c_void_p]
    lib.jpp_stage_opt_ptr.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                      C.POINTER(C.c_void_p)]
    lib.jpp_stage_adam_step.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_double,
                                        C.c_double, C.c_double, C.c_double, C.c_double]
    _lib = lib
    return lib


def check(rc: int):
    if rc != 0:
        raise JppError(rc, load().jpp_last_error().decode(errors="replace"))


def device_count() -> int:
    n = C.c_int(0)
    rc = load().jpp_device_count(C.byref(n))
    return n.value if rc == 0 else 0


def require_gpu():
    if device_count() < 1:
        raise RuntimeError("jaxpp_amd needs a GPU: no HIP device is visible")


# ---------------------------------------------------------------------------
# bf16 <-> float32 on the host (round to nearest even), numpy only
# ---------------------------------------------------------------------------
def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    return r.astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(
        np.float32)


class DeviceBuffer:
    """A device allocation owned by this object."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(load().jpp_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value or 0

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        buf.upload(a)
        return buf

    @classmethod
    def from_f32_as_bf16(cls, a: np.ndarray) -> "DeviceBuffer":
        return cls.from_numpy(to_bf16_bits(a))

    def upload(self, a: np.ndarray, offset: int = 0):
        a = np.ascontiguousarray(a)
        assert offset + a.nbytes <= self.nbytes
        check(load().jpp_memcpy_h2d(self.ptr + offset, a.ctypes.data, a.nbytes))

    def download(self, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        check(load().jpp_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes))
        return out

    def download_bf16(self, shape) -> np.ndarray:
        return from_bf16_bits(self.download(np.uint16, shape))

    def zero(self, stream=None):
        check(load().jpp_fill_u32(self.ptr, 0, self.nbytes // 4, stream))

    def free(self):
        if self.ptr:
            load().jpp_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def upload_ptr(ptr: int, a: np.ndarray):
    a = np.ascontiguousarray(a)
    check(load().jpp_memcpy_h2d(ptr, a.ctypes.data, a.nbytes))


def download_ptr(ptr: int, dtype, shape) -> np.ndarray:
    out = np.empty(shape, dtype=dtype)
    check(load().jpp_memcpy_d2h(out.ctypes.data, ptr, out.nbytes))
    return out


def sync():
    check(load().jpp_device_sync())


class Stream:
    """A HIP stream of default priority that does not synchronise with the null stream."""

    def __init__(self):
        p = C.c_void_p()
        check(load().jpp_stream_create(C.byref(p)))
        self.ptr = p.value

    def wait(self, event: "Event"):
        check(load().jpp_stream_wait_event(self.ptr, event.ptr))

    def sync(self):
        check(load().jpp_stream_sync(self.ptr))

    def __del__(self):
        try:
            if self.ptr:
                load().jpp_stream_destroy(self.ptr)
        except Exception:
            pass


class Graph:
    """A recorded sequence of calls on `stream` (see jpp_graph_begin in the header)::

        g = Graph(stream)
        with g:                 # record
            loop.run(io, stream=stream.ptr); executor.join(stream.ptr)
        g.launch()              # replay, as often as wanted
    """

    def __init__(self, stream: Stream):
        self.stream, self.exec = stream, None

    def __enter__(self):
        check(load().jpp_graph_begin(self.stream.ptr))
        return self

    def __exit__(self, exc_type, exc, tb):
        p = C.c_void_p()
        rc = load().jpp_graph_end(self.stream.ptr, C.byref(p))
        if exc_type is None:
            check(rc)
            self.exec = p.value
        return False

    def launch(self, stream=None):
        check(load().jpp_graph_launch(self.exec, stream if stream is not None else self.stream.ptr))

    def __del__(self):
        try:
            if self.exec:
                load().jpp_graph_destroy(self.exec)
        except Exception:
            pass


def stream_wait(stream, event: "Event"):
    """Work queued on `stream` (None: the null stream) after this call waits for `event`."""
    check(load().jpp_stream_wait_event(stream, event.ptr))


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(load().jpp_event_create(C.byref(p)))
        self.ptr = p.value

    def record(self, stream=None):
        check(load().jpp_event_record(self.ptr, stream))

    def sync(self):
        check(load().jpp_event_sync(self.ptr))

    def elapsed_ms(self, later: "Event") -> float:
        ms = C.c_float()
        check(load().jpp_event_elapsed_ms(self.ptr, later.ptr, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                load().jpp_event_destroy(self.ptr)
        except Exception:
            pass


class probe:
    """Times every launch of one kernel class with HIP events on the launch
    stream (reference: ``collect_task_times_ms``,
    src/jaxpp/jax_primitives.py:742-773).  After the ``with`` block:
    ``launches``, ``total_ms``, ``flops``, ``bytes``."""

    def __init__(self, kernel_class: str):
        self.kernel_class = kernel_class
        self.launches, self.total_ms, self.flops, self.bytes = 0, 0.0, 0.0, 0.0

    def __enter__(self):
        check(load().jpp_probe_begin(self.kernel_class.encode()))
        return self

    def __exit__(self, *exc):
        n, ms, fl, by = C.c_int64(), C.c_double(), C.c_double(), C.c_double()
        check(load().jpp_probe_end(C.byref(n), C.byref(ms), C.byref(fl), C.byref(by)))
        self.launches, self.total_ms, self.flops, self.bytes = n.value, ms.value, fl.value, by.value
        # per class: {name: (launches, total ms, flops, bytes)}; one entry unless the class is "*"
        self.classes = {}
        i = 0
        while True:
            name = C.c_char_p()
            if load().jpp_probe_class(i, C.byref(name), C.byref(n), C.byref(ms), C.byref(fl),
                                      C.byref(by)) != 0:
                break
            self.classes[name.value.decode()] = (n.value, ms.value, fl.value, by.value)
            i += 1
        return False


# ---------------------------------------------------------------------------
# kernel wrappers (thin: arguments are device pointers)
# ---------------------------------------------------------------------------
def gemm(a, b, c, m, n, k, lda, ldb, ldc, trans_a, trans_b, epilogue=EPI_BF16, bias=None,
         resid=None, ldresid=0, aux=None, ldaux=0, c2=None, ldc2=0, gelu_tanh=0, tile=0,
         stream=None, seg=None, n_seg=0, group_mode=0, stride_b=0, stride_c=0, group_rows=0,
         seg_rows=None, f32=False, more=(), more_seg=(), rope=None):
    """`more`: further (a, b) operand pairs the contraction continues over (k elements each);
    `more_seg`: for a grouped contraction, the (seg, seg_rows) row groups of those pairs;
    `rope`: (cos, sin, cols, seq, head_dim) - rotary embedding of columns [0, cols) in the
    epilogue of a forward product."""
    g = GemmArgs(a, b, c, c2, bias, resid, aux, m, n, k, lda, ldb, ldc, ldc2, ldresid, ldaux,
                 int(trans_a), int(trans_b), epilogue, gelu_tanh, tile, seg, n_seg, group_mode,
                 stride_b, stride_c, group_rows, seg_rows)
    if more:
        g.a_more = (C.c_void_p * 3)(*([pa for pa, _ in more] + [None] * (3 - len(more))))
        g.b_more = (C.c_void_p * 3)(*([pb for _, pb in more] + [None] * (3 - len(more))))
        g.k_parts = 1 + len(more)
    if more_seg:
        g.seg_more = (C.c_void_p * 3)(*([sg for sg, _ in more_seg] + [None] * (3 - len(more_seg))))
        g.seg_rows_more = (C.c_void_p * 3)(*([sr for _, sr in more_seg] + [None] * (3 - len(more_seg))))
    if rope:
        g.rope_cos, g.rope_sin, g.rope_cols, g.rope_seq, g.rope_head_dim = rope
    check((load().jpp_gemm_f32 if f32 else load().jpp_gemm_bf16)(stream, C.byref(g)))


def gemm_multi(problems, stream=None):
    """Up to four accumulated weight gradients as one launch (jpp_gemm_bf16_multi).  Each
    problem is a dict: a, b, c (device pointers), m, n, k, lda, ldb, ldc and optionally
    `more` = further (a, b) operand pairs."""
    arr = (GemmArgs * len(problems))()
    for i, q in enumerate(problems):
        g = GemmArgs(q["a"], q["b"], q["c"], None, None, None, None, q["m"], q["n"], q["k"],
                     q["lda"], q["ldb"], q["ldc"], 0, 0, 0, 1, 1, q.get("epilogue", EPI_ACC_F32),
                     0, q.get("tile", 0), None, 0, 0, 0, 0, 0, None)
        more = q.get("more", ())
        if more:
            g.a_more = (C.c_void_p * 3)(*([pa for pa, _ in more] + [None] * (3 - len(more))))
            g.b_more = (C.c_void_p * 3)(*([pb for _, pb in more] + [None] * (3 - len(more))))
            g.k_parts = 1 + len(more)
        arr[i] = g
    check(load().jpp_gemm_bf16_multi(stream, arr, len(problems)))


def mfma_rate(shape: int, random_operands: bool, iters: int = 100000) -> float:
    """TFLOP/s of a register-only MFMA loop on every SIMD (see jpp_mfma_rate)."""
    out = C.c_double(0.0)
    check(load_diag().jpp_mfma_rate(shape, int(random_operands), iters, C.byref(out)))
    return out.value


def lds_read_rate(lane_offsets, transposing: bool) -> float:
    """Shader clocks per wave-level LDS read of 8 waves reading with these 64 per-lane byte
    offsets (see jpp_lds_read_rate)."""
    if len(lane_offsets) != 64:
        raise ValueError("one byte offset per lane of a wave: 64 of them")
    arr = (C.c_uint32 * 64)(*[int(o) for o in lane_offsets])
    out = C.c_double(0.0)
    check(load_diag().jpp_lds_read_rate(arr, int(transposing), C.byref(out)))
    return out.value


def adam_step(count, grad, m, v, step, master=None, param=None, lr=1e-3, b1=0.9, b2=0.999,
              eps=1e-8, grad_scale=1.0, zero_grad=False, stream=None):
    """`optax.adam` + `apply_updates` on flat device tensors (device pointers)."""
    a = AdamArgs(count, grad, master, param, m, v, step, lr, b1, b2, eps, grad_scale,
                 int(zero_grad))
    check(load().jpp_adam_step(stream, C.byref(a)))


class StageExecutor:
    """One pipeline rank on one GPU: parameters, fp32 gradient accumulators,
    residual slots, and the FWD / BWD / BWD_I / BWD_W tasks."""

    def __init__(self, spec, n_chunks: int, layers_per_chunk: int, max_live: int,
                 split_backward: bool = False, fused_wgrad_accum: bool = True,
                 two_streams: bool = False, wgrad_group: int = 0):
        require_gpu()
        self.spec = spec
        self.dtype = getattr(spec, "dtype", "bf16")
        self.n_chunks, self.layers_per_chunk = n_chunks, layers_per_chunk
        d = StageDesc(FAMILY[spec.family], spec.hidden, spec.n_heads, spec.kvh, spec.d, spec.ffn,
                      spec.seq, spec.batch, int(spec.causal), spec.rope_theta, spec.eps,
                      int(spec.gelu_tanh), spec.n_experts, spec.top_k, n_chunks,
                      layers_per_chunk, max_live, int(split_backward), int(fused_wgrad_accum),
                      int(two_streams), DTYPE[self.dtype], int(wgrad_group))
        h = C.c_void_p()
        check(load().jpp_stage_create(C.byref(d), C.byref(h)))
        self.handle = h.value
        self.params = []
        for i in range(load().jpp_stage_n_params(self.handle)):
            name, r, c = C.c_char_p(), C.c_int64(), C.c_int64()
            check(load().jpp_stage_param_info(self.handle, i, C.byref(name), C.byref(r),
                                              C.byref(c)))
            self.params.append((name.value.decode(), r.value, c.value))
        self.index = {n: i for i, (n, _, _) in enumerate(self.params)}

    @property
    def nbytes(self) -> int:
        return load().jpp_stage_bytes(self.handle)

    def _ptr(self, fn, chunk, layer, name):
        p = C.c_void_p()
        check(fn(self.handle, chunk, layer, self.index[name], C.byref(p)))
        return p.value

    def _device_columns(self, name: str, cols: int):
        """Column order of a parameter in device memory, or None when it is the host's.  The
        Llama and Mixtral layers keep ``Wgu = [gate | up]`` with the two projections interleaved in blocks
        of 32 columns (device column 64q+w = gate feature 32q+w for w < 32, up feature 32q+w-32
        otherwise), which lets the GEMM epilogue apply SwiGLU (JPP_EPI_SWIGLU)."""
        if self.spec.family not in ("llama", "mixtral") or name != "Wgu":
            return None
        f = cols // 2
        c = np.arange(cols)
        q, w = c // 64, c % 64
        return np.where(w < 32, 32 * q + w, f + 32 * q + w - 32)

    def set_params(self, chunk: int, layer: int, params: dict):
        """Upload float32 host arrays as device parameters (bf16, or f32 for an f32 stage)."""
        for name, rows, cols in self.params:
            a = np.asarray(params[name], dtype=np.float32)
            assert a.size == rows * cols, (name, a.shape, rows, cols)
            order = self._device_columns(name, cols)
            if order is not None:
                a = np.ascontiguousarray(a.reshape(rows, cols)[:, order])
            upload_ptr(self._ptr(load().jpp_stage_param_ptr, chunk, layer, name),
                       a if self.dtype == "f32" else to_bf16_bits(a))

    def get_params(self, chunk: int, layer: int) -> dict:
        """The device parameters as float32 host arrays."""
        self.join()
        out = {}
        for name, rows, cols in self.params:
            shape = (cols,) if rows == 1 and not name.startswith("W") else (rows, cols)
            ptr = self._ptr(load().jpp_stage_param_ptr, chunk, layer, name)
            if self.dtype == "f32":
                a = download_ptr(ptr, np.float32, shape)
            else:
                a = from_bf16_bits(download_ptr(ptr, np.uint16, shape))
            order = self._device_columns(name, cols)
            if order is not None:
                host = np.empty_like(a)
                host[:, order] = a
                a = host
            out[name] = a
        return out

    def get_grads(self, chunk: int, layer: int) -> dict:
        self.join()          # the copies below run on the null stream
        out = {}
        for name, rows, cols in self.params:
            shape = (cols,) if rows == 1 and not name.startswith("W") else (rows, cols)
            g = download_ptr(self._ptr(load().jpp_stage_grad_ptr, chunk, layer, name),
                             np.float32, shape)
            order = self._device_columns(name, cols)
            if order is not None:
                host = np.empty_like(g)
                host[:, order] = g
                g = host
            out[name] = g
        return out

    def upload_activation(self, a: np.ndarray) -> "DeviceBuffer":
        """A float32 host array as a device tensor of the stage's element type."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        return DeviceBuffer.from_numpy(a if self.dtype == "f32" else to_bf16_bits(a))

    def new_activation(self) -> "DeviceBuffer":
        return DeviceBuffer(self.spec.tokens * self.spec.hidden * (4 if self.dtype == "f32" else 2))

    def download_activation(self, buf: "DeviceBuffer", shape) -> np.ndarray:
        if self.dtype == "f32":
            return buf.download(np.float32, shape)
        return buf.download_bf16(shape)

    def zero_grads(self, stream=None):
        check(load().jpp_stage_zero_grads(self.handle, stream))

    def optimizer_init(self, stream=None):
        """Allocates (first call) and resets the optimizer state: f32 weights cast up from
        the bf16 parameters as they are now, zero moments."""
        check(load().jpp_stage_optimizer_init(self.handle, stream))

    def adam_step(self, step: int, lr: float = 1e-3, b1: float = 0.9, b2: float = 0.999,
                  eps: float = 1e-8, grad_scale: float = 1.0, stream=None):
        """The update after the loop (README.md:90-93 with `optax.adam`, whose defaults these
        are): one launch over every parameter of the stage; rewrites the bf16 parameters and
        clears the gradient accumulators.  `step` counts from 1."""
        check(load().jpp_stage_adam_step(self.handle, stream, step, lr, b1, b2, eps, grad_scale))

    def get_opt_state(self, chunk: int, layer: int) -> dict:
        """name -> (f32 weights, m, v) in the host's column order."""
        self.join()
        out = {}
        for name, rows, cols in self.params:
            shape = (cols,) if rows == 1 and not name.startswith("W") else (rows, cols)
            order = self._device_columns(name, cols)
            trio = []
            for which in range(3):
                p = C.c_void_p()
                check(load().jpp_stage_opt_ptr(self.handle, which, chunk, layer, self.index[name],
                                               C.byref(p)))
                a = download_ptr(p.value, np.float32, shape)
                if order is not None:
                    host = np.empty_like(a)
                    host[:, order] = a
                    a = host
                trio.append(a)
            out[name] = tuple(trio)
        return out

    def join(self, stream=None):
        """Orders `stream` behind the weight-gradient work on the stage's own stream."""
        check(load().jpp_stage_join(self.handle, stream))

    def quiesce(self):
        """Waits (on the host) for the stage's own stream; call before recording a graph."""
        check(load().jpp_stage_quiesce(self.handle))

    def run_task(self, kind: TaskType, chunk: int, mubatch: int, inp=None, out=None,
                 stream=None):
        check(load().jpp_stage_run_task(self.handle, kind.value, chunk, mubatch,
                                        inp, out, stream))

    def live_slots(self) -> int:
        return load().jpp_stage_live_slots(self.handle)

    def routing(self, chunk: int, mubatch: int, layer: int):
        """(expert ids [tokens, top_k] int32, gates [tokens, top_k] f32) a forward task of a
        mixture-of-experts stage chose, while that microbatch's residuals are live."""
        n = self.spec.tokens * self.spec.top_k
        ids, gates = DeviceBuffer(4 * n), DeviceBuffer(4 * n)
        check(load().jpp_stage_routing(self.handle, chunk, mubatch, layer, ids.ptr, gates.ptr, None))
        sync()
        shape = (self.spec.tokens, self.spec.top_k)
        return ids.download(np.int32, shape), gates.download(np.float32, shape)

    def close(self):
        if getattr(self, "handle", None):
            load().jpp_stage_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
