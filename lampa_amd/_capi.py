"""ctypes binding of ``liblampa_amd.so`` -- the only route from Python to the gfx950 kernels.

There is no CPU fallback: if the library has not been built the import of any operator raises.
Every entry point takes raw device pointers, sizes and a HIP stream, and returns 0 or a negative error code.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblampa_amd.so")

_ERRORS = {
    -1: "invalid argument",
    -2: "workspace missing or too small",
    -3: "HIP launch error",
    -4: "unsupported shape or dtype",
}

_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float

_SIGNATURES = {
    "lampa_lsh_bucket_workspace_bytes": (_i64, [_i64, _i32, _i32]),
    "lampa_lsh_bucket_keys": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _i32, _i32, _f32, _vp, _vp, _vp, _vp, _i64, _vp]),
    "lampa_lsh_bucket_sort_workspace_bytes": (_i64, [_i64, _i32, _i32]),
    "lampa_lsh_bucket_sort": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _i32, _i32, _f32, _vp, _vp, _vp, _vp, _vp, _i64,
                                     _vp, _i32, _vp, _i64, _vp]),
    "lampa_lsh_bucket_sort_batch_workspace_bytes": (_i64, [_i32, _i64, _i32, _i32]),
    "lampa_lsh_bucket_sort_batch": (_i32, [_vp, _i32, _i64, _vp, _i32, _vp, _vp, _i32, _i32, _f32, _vp, _vp, _vp, _vp,
                                           _vp, _i64, _vp, _i32, _vp, _i64, _vp]),
    "lampa_lsh_one_launch_config": (_i32, [_i32, _i64]),
    "lampa_lsh_project_f32": (_i32, [_vp, _i32, _i64, _i32, _vp, _i32, _vp, _i64, _i64, _i64, _vp]),
    "lampa_lsh_ordering_keys": (_i32, [_vp, _i64, _i32, _vp, _i32, _vp, _vp, _vp]),
    "lampa_row_minmax_f32": (_i32, [_vp, _i32, _i64, _vp, _vp]),
    "lampa_sort_workspace_bytes": (_i64, [_i32, _i64]),
    "lampa_sort_pairs": (_i32, [_vp, _i32, _vp, _i32, _i64, _i32, _vp, _i32, _i32, _vp, _vp, _i64, _vp]),
    "lampa_sort_pairs_static_max_bytes": (_i64, []),
    "lampa_sort_pairs_static": (_i32, [_vp, _i32, _vp, _i32, _i64, _i32, _vp, _i32, _i32, _vp, _vp]),
    "lampa_gather_rows": (_i32, [_vp, _i32, _i64, _vp, _i32, _i32, _i64, _i64, _vp, _vp]),
    "lampa_scatter_rows": (_i32, [_vp, _vp, _i32, _i32, _i64, _i64, _vp, _vp]),
    "lampa_invert_perm": (_i32, [_vp, _i32, _i32, _i64, _vp, _vp]),
    "lampa_quantile_regions": (_i32, [_vp, _i32, _i64, _vp, _i32, _vp, _vp]),
    "lampa_geo_shift": (_i32, [_vp, _vp, _vp, _vp, _i32, _i64, _vp, _vp]),
    "lampa_hept_sort_keys": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _vp]),
    "lampa_hept_prep_qk": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp]),
    "lampa_causal_conv1d_fwd": (_i32, [_vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _vp, _i32, _i64, _i32, _i32, _vp,
                                       _i64, _i32, _i64, _vp]),
    "lampa_proj_conv_fwd": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _i32, _vp, _vp, _i32, _i32, _vp, _i32, _vp, _i32, _vp, _i32,
                                   _vp]),
    "lampa_norm_proj_fwd": (_i32, [_vp, _vp, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _f32, _vp, _vp, _vp, _f32, _vp, _i32,
                                   _vp]),
    "lampa_rms_norm_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _f32, _i32, _i32, _i32, _i32, _i64,
                                  _vp]),
    "lampa_gdr_gates_fwd": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _i32, _f32, _i32, _vp, _vp, _vp]),
    "lampa_gdr_recurrent_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32,
                                       _i32, _i32, _f32, _i32, _vp]),
    "lampa_gdr_recurrent_headwise_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32,
                                                _i32, _i32, _i32, _f32, _i32, _vp]),
    "lampa_gdr_recurrent_segmented_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32]),
    "lampa_gdr_recurrent_segmented_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                                 _i32, _i32, _i32, _i32, _f32, _i32, _vp, _i64, _vp]),
    "lampa_gdr_bwd_workspace_bytes": (_i64, [_i64, _i32, _i32, _i32, _i32, _i32]),
    "lampa_gdr_bwd": (_i32, [_vp] * 18 + [_i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _i64, _vp]),
    "lampa_gdr_bwd_chunk_plan_size": (_i64, [_vp, _i32]),
    "lampa_gdr_bwd_chunk_plan_fill": (_i32, [_vp, _i32, _vp]),
    "lampa_gdr_bwd_chunk_workspace_bytes": (_i64, [_vp, _i32]),
    "lampa_gdr_bwd_chunk": (_i32, [_vp] * 16 + [_i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _i64, _vp]),
    "lampa_profile_begin": (_i32, []),
    "lampa_profile_end": (_i32, [_i32, _vp, _vp]),
    "lampa_gdr_traffic_probe": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "lampa_gdr_traffic_probe_walk": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "lampa_gdr_plan_size": (_i64, [_vp, _i32, _i32]),
    "lampa_gdr_plan_fill": (_i32, [_vp, _i32, _i32, _vp]),
    "lampa_gdr_plan_size_balanced": (_i64, [_vp, _i32, _i32]),
    "lampa_gdr_plan_fill_balanced": (_i32, [_vp, _i32, _i32, _vp]),
    "lampa_gdr_plan_size_lengths": (_i64, [_vp, _i32, _vp, _i32]),
    "lampa_gdr_plan_fill_lengths": (_i32, [_vp, _i32, _vp, _i32, _vp]),
    "lampa_gdr_chunk_workspace_bytes": (_i64, [_i64, _i64, _i32, _i32, _i32]),
    "lampa_gdr_chunk_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                   _f32, _i32, _vp, _i64, _vp]),
    "lampa_gdr_chunk_config": (_i32, [_i32]),
    "lampa_hgdn_chunk_workspace_bytes": (_i64, [_i64, _i64, _i32, _i32, _i32]),
    "lampa_hgdn_chunk_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _f32, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32,
                                    _i32, _i32, _f32, _i32, _vp, _i64, _vp]),
    "lampa_hgdn_step": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _f32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32,
                               _i32, _i32, _f32, _i32, _vp]),
}

_lib = None


class LampaError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built (``python -m lampa_amd.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP library first (python -m lampa_amd.build). "
                "lampa_amd has no CPU or PyTorch fallback.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def profile_begin():
    """Start timing every kernel launched by the library (HIP events on the launch stream)."""
    check(lib().lampa_profile_begin(), "lampa_profile_begin")


def profile_end(max_entries: int = 256):
    """Stop timing; returns [(kernel name, milliseconds), ...] in launch order."""
    ms = (ctypes.c_float * max_entries)()
    names = (ctypes.c_char_p * max_entries)()
    n = check(lib().lampa_profile_end(max_entries, ms, names), "lampa_profile_end")
    return [(names[i].decode(), float(ms[i])) for i in range(n)]


def exported_symbols():
    return sorted(_SIGNATURES)


def check(code: int, what: str):
    if code < 0:
        raise LampaError(f"{what} failed: {_ERRORS.get(int(code), 'error')} ({int(code)})")
    return code


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def stream_of(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise LampaError("lampa_amd operators run on the GPU only: got a CPU tensor (there is no CPU fallback)")
