"""Loads ``libcswap_hip.so`` and declares its C ABI for ctypes.

There is no fallback: if the library is missing or fails to load, importing the
functions raises, so nothing can silently run on a CPU path.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcswap_hip.so")


class CswapError(RuntimeError):
    def __init__(self, code: int, what: str):
        self.code = code
        super().__init__(f"{what}: {lib().cswap_strerror(code).decode()} (code {code}, "
                         f"hipError {lib().cswap_last_hip_error()})")


_lib = None

vp, sz, pd, u, i32 = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint, C.c_int


class Costs(C.Structure):
    _fields_ = [("bw_d2h_gbs", C.c_double), ("bw_h2d_gbs", C.c_double), ("copy_latency_us", C.c_double),
                ("kernel_latency_us", C.c_double), ("zfp_latency_us", C.c_double), ("zvc_compress_gbs", C.c_double),
                ("zvc_expand_gbs", C.c_double), ("zfp_compress_gbs", C.c_double),
                ("zfp_decompress_gbs", C.c_double), ("sparse_max_ratio", C.c_double), ("lossy_min_gain", C.c_double),
                ("probe_latency_us", C.c_double), ("probe_gbs", C.c_double), ("min_gain", C.c_double),
                ("d2h_hidden", C.c_int),
                ("size_floor_bytes", C.c_size_t), ("allow_lossy", C.c_int), ("process", C.c_int)]


class Choice(C.Structure):
    _fields_ = [("policy", C.c_int), ("bytes_out", C.c_size_t), ("ratio", C.c_double),
                ("t_none_us", C.c_double), ("t_sparse_us", C.c_double), ("t_zfp_us", C.c_double)]


class EngineConfig(C.Structure):
    _fields_ = [("pinned_pool_bytes", C.c_size_t), ("device_pool_bytes", C.c_size_t), ("process", C.c_int),
                ("zfp_maxbits", C.c_uint), ("max_tickets", C.c_int), ("costs", Costs), ("timing", C.c_int)]


class TicketInfo(C.Structure):
    _fields_ = [("policy", C.c_int), ("n", C.c_size_t), ("nnz", C.c_size_t), ("bytes_in", C.c_size_t),
                ("bytes_out", C.c_size_t), ("state", C.c_int)]


class TicketTiming(C.Structure):
    _fields_ = [("compress_us", C.c_double), ("copy_out_us", C.c_double), ("copy_in_us", C.c_double),
                ("decompress_us", C.c_double)]


class PlanSummary(C.Structure):
    _fields_ = [("time_us", C.c_double), ("base_time_us", C.c_double), ("bytes_total", C.c_size_t),
                ("bytes_target", C.c_size_t), ("bytes_moved", C.c_size_t), ("bytes_on_link", C.c_size_t),
                ("n_selected", C.c_int), ("target_met", C.c_int)]


class ZfpBitstream(C.Structure):
    _fields_ = [("bits", C.c_uint), ("buffer", C.c_uint64), ("ptr", C.c_void_p), ("begin", C.c_void_p),
                ("end", C.c_void_p)]


class ZfpStream(C.Structure):
    _fields_ = [("minbits", C.c_uint), ("maxbits", C.c_uint), ("maxprec", C.c_uint), ("minexp", C.c_int),
                ("stream", C.POINTER(ZfpBitstream)), ("exec_policy", C.c_int), ("omp_threads", C.c_uint),
                ("omp_chunk", C.c_uint)]


class ZfpField(C.Structure):
    _fields_ = [("type", C.c_int), ("nx", C.c_size_t), ("ny", C.c_size_t), ("nz", C.c_size_t),
                ("nw", C.c_size_t), ("sx", C.c_ssize_t), ("sy", C.c_ssize_t), ("sz", C.c_ssize_t),
                ("sw", C.c_ssize_t), ("data", C.c_void_p)]


_SIGNATURES = {
    "cswap_strerror": (C.c_char_p, [i32]),
    "cswap_last_hip_error": (i32, []),
    "cswap_abi_version": (i32, []),
    "cswap_zfp_stream_bytes": (sz, [sz, sz, sz, u]),
    "cswap_zfp_stream_capacity": (sz, [sz, sz, sz, u]),
    "cswap_zfp_compress_f32": (i32, [vp, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_decompress_f32": (i32, [vp, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_stream_capacity_nd": (sz, [i32, sz, sz, sz, u]),
    "cswap_zfp_stream_bytes_nd": (sz, [i32, sz, sz, sz, u]),
    "cswap_zfp_compress_f32_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_decompress_f32_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_compress_i32_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_decompress_i32_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_compress_f64_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_decompress_f64_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_compress_i64_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_decompress_i64_nd": (i32, [vp, i32, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_set_pair_bytes": (None, [sz, sz, C.POINTER(sz)]),
    "cswap_zvc_chunk_elems": (i32, [i32, i32]),
    "cswap_zvc_chunk_words": (i32, [i32, i32]),
    "cswap_zvc_active_chunks": (i32, [i32, i32]),
    "cswap_zvc_mask_bytes": (sz, [i32, i32]),
    "cswap_zvc_pick_process": (i32, [sz]),
    "cswap_zvc_set_staged_compact_bytes": (sz, [sz]),
    "cswap_zvc_set_single_pass_bytes": (sz, [sz]),
    "cswap_zvc_takes_single_pass": (i32, [i32, i32]),
    "cswap_zvc_count": (i32, [vp, i32, i32, vp, vp]),
    "cswap_zvc_scan": (i32, [vp, i32, vp, vp]),
    "cswap_zvc_compact": (i32, [vp, i32, i32, vp, vp, vp, vp]),
    "cswap_zvc_expand": (i32, [vp, vp, vp, i32, i32, vp, vp]),
    "cswap_zvc_compress": (i32, [vp, i32, i32, vp, vp, vp, vp, vp]),
    "cswap_zvc_workspace_bytes": (sz, [i32]),
    "cswap_zvc_compress_fused": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp]),
    "cswap_zvc_workspace_clear": (i32, [vp, i32, vp]),
    "cswap_zvc_debug_set_lookback": (None, [u, u]),        # include/cswap_test_hooks.h
    "cswap_test_zvc_stream_groups": (i32, [i32, i32]),      # include/cswap_test_hooks.h
    "cswap_zvc_compress_fused_static": (i32, [vp, i32, i32, vp, vp, vp, vp, vp]),
    "cswap_probe_nnz": (i32, [vp, sz, vp, vp]),
    "cswap_costs_default": (None, [C.POINTER(Costs)]),
    "cswap_policy_bytes": (sz, [i32, sz, sz, u, i32, sz, sz, sz]),
    "cswap_select": (i32, [sz, sz, u, C.POINTER(Costs), C.POINTER(Choice)]),
    "cswap_select_field": (i32, [sz, sz, sz, sz, u, C.POINTER(Costs), C.POINTER(Choice)]),
    "cswap_engine_config_default": (None, [C.POINTER(EngineConfig)]),
    "cswap_engine_create": (i32, [C.POINTER(vp), C.POINTER(EngineConfig)]),
    "cswap_engine_destroy": (None, [vp]),
    "cswap_swap_out": (i32, [vp, vp, sz, sz, sz, i32, vp, C.POINTER(i32)]),
    "cswap_swap_wait": (i32, [vp, i32]),
    "cswap_swap_in": (i32, [vp, i32, vp, vp]),
    "cswap_swap_prefetch": (i32, [vp, i32]),
    "cswap_swap_release": (i32, [vp, i32]),
    "cswap_swap_info": (i32, [vp, i32, C.POINTER(TicketInfo)]),
    "cswap_swap_timing": (i32, [vp, i32, C.POINTER(TicketTiming)]),
    "cswap_engine_set_zfp_maxbits": (i32, [vp, C.c_uint]),
    "cswap_engine_probe_count": (C.c_ulonglong, [vp]),
    "cswap_engine_calibrate": (i32, [vp, C.POINTER(Costs)]),
    "cswap_engine_copy_stream": (vp, [vp]),
    "cswap_engine_tune": (i32, [vp, sz, C.POINTER(i32)]),
    "cswap_engine_process_for": (i32, [vp, sz]),
    "cswap_planner_create": (vp, [C.POINTER(Costs), u]),
    "cswap_planner_destroy": (None, [vp]),
    "cswap_planner_reset": (i32, [vp]),
    "cswap_planner_set_backward_factor": (i32, [vp, C.c_double]),
    "cswap_planner_add_comptime": (i32, [vp, C.c_double]),
    "cswap_planner_add_tensor": (i32, [vp, i32, sz]),
    "cswap_planner_add_stepdep": (i32, [vp, i32, i32]),
    "cswap_planner_add_omitid": (i32, [vp, i32]),
    "cswap_planner_set_field": (i32, [vp, i32, sz, sz, sz]),
    "cswap_planner_set_nnz": (i32, [vp, i32, sz]),
    "cswap_planner_init": (i32, [vp, C.c_double]),
    "cswap_planner_make_policy": (i32, [vp, C.POINTER(i32), C.POINTER(i32), i32, C.POINTER(PlanSummary)]),
    "cswap_planner_capuchin": (i32, [vp, C.POINTER(i32), C.POINTER(i32), i32, C.POINTER(PlanSummary)]),
    # the reference's own entry-point names (include/cswap_compat.h)
    "PreGPUcompression": (None, [i32, i32, vp, vp, i32, i32, vp]),
    "PreAcc": (None, [vp, i32, vp, i32, i32, vp]),
    "GPUcompression": (None, [i32, i32, vp, vp, vp, vp, i32, i32, vp]),
    "GPUdecompression": (None, [vp, vp, i32, i32, vp, vp, i32, i32]),
    "cuda_compress": (sz, [C.POINTER(ZfpStream), C.POINTER(ZfpField)]),
    "cuda_decompress": (None, [C.POINTER(ZfpStream), C.POINTER(ZfpField)]),
    "setRatio": (None, [i32]),
    "compress": (vp, [vp, C.c_longlong, C.POINTER(sz)]),
    "decompress": (i32, [vp, C.c_longlong, vp]),
    "cswap_set_allocator": (None, [vp, vp]),
    "cswap_compat_set_field": (None, [sz, sz]),
}


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m cswap_amd.build` "
                "(there is no CPU fallback)")
        # torch ships its own copy of the HIP runtime; if this library (linked against the
        # system's) is the first to bring a runtime into the process and initialise it, torch
        # afterwards reports no GPU.  Importing torch first makes both use the one torch loads.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            f = getattr(L, name)  # AttributeError if the symbol is not exported
            f.restype = res
            f.argtypes = args
        _lib = L
    return _lib


def declared_symbols():
    return sorted(_SIGNATURES)


def check(code: int, what: str) -> None:
    if code != 0:
        raise CswapError(code, what)
