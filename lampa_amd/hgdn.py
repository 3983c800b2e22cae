"""Hierarchical (level-weighted) gated-delta forward on the GPU behind the reference's operator signature.

``chunk_h_gated_delta_rule`` (reference ``models/hattention/gated_delta_rule_apis.py:21-134``): same argument names,
order, defaults and checks. The reference's own chunk pipeline for this operator does not run as shipped
(``chunkwise_hgdn.py:661`` unpacks the single tensor ``chunk_scaled_dot_kkt_fwd`` returns into two), so the function
implemented is its specification, ``hattention_recurrent`` (``recurrent.py:169-216``), reached the way the operator
reaches it: q l2-normalised and scaled, k l2-normalised (``kernel.py:100-101``), lambda divided by ``scale``
(``gated_delta_rule_apis.py:68-70``; the kernel does it, with the rounding of a division in lambda's dtype), weak
hierarchy, base 2.

Differences a caller can observe: forward only; ``output_final_state=True`` (the prefill and single-step branches,
``gated_delta_rule_apis.py:92-128``) raises ``NotImplementedError``; head sizes K = 64 and V in {64, 128} only.
"""
import ctypes
import warnings
from typing import Optional

import torch

from . import _capi
from . import gated_delta as _gd
from ._capi import check, ptr, require_cuda, stream_of

SCALE_LAMBDA = True  # gated_delta_rule_apis.py:17

# Chunks per segment of the split-sequence walk (a power of two); None picks it from the sequence length.
CHUNKS_PER_SEGMENT: Optional[int] = None

_plan_cache = {}


def num_levels(length: int, chunk: int = 64) -> int:
    """Levels a sequence of ``length`` tokens needs: ``get_num_levels`` (``base.py:36-37``) of the chunk plus the
    number of chunk-index bits (``chunkwise_hgdn.py:716-720``)."""
    nt = (length + chunk - 1) // chunk
    return (chunk - 1).bit_length() + 1 + (max(nt, 1) - 1).bit_length()


def _plan(B: int, T: int, device, n_value_heads: int, n_slabs: int):
    nt = (T + 63) // 64
    cps = CHUNKS_PER_SEGMENT
    if not cps:
        # a compute unit holds one workgroup of the walk (segment, head, 32 value columns): the shortest segments that
        # still run in one round; the scan in between is serial in the segments of a sequence
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        cps = 1 << max(nt - 1, 1).bit_length()  # one segment per sequence
        while cps > 8 and B * ((nt + cps // 2 - 1) // (cps // 2)) * n_value_heads * n_slabs <= cus:
            cps //= 2
    key = (B, T, cps, str(device))
    hit = _plan_cache.get(key)
    if hit is not None:
        return hit
    lib = _capi.lib()
    cu_host = [i * T for i in range(B + 1)]
    cu = (ctypes.c_int64 * len(cu_host))(*cu_host)
    size = check(lib.lampa_gdr_plan_size(cu, B, cps), "lampa_gdr_plan_size")
    host = torch.empty(size, dtype=torch.int32)
    check(lib.lampa_gdr_plan_fill(cu, B, cps, ctypes.c_void_p(host.data_ptr())), "lampa_gdr_plan_fill")
    dev = host.to(device)
    if len(_plan_cache) > 64:
        _plan_cache.clear()
    _plan_cache[key] = (host, dev)
    return host, dev


class _ForwardOnly(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, g, lam, beta, scale, lam_div):
        require_cuda(q, k, v, g, lam, beta)
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        g, beta = g.to(torch.float32).contiguous(), beta.to(torch.float32).contiguous()
        if lam.dtype not in _gd._DTYPES:
            lam = lam.to(torch.float32)
        lam = lam.contiguous()
        B, T, H, K = q.shape
        HV, V, L = v.shape[2], v.shape[3], lam.shape[-1]
        plan_host, plan_dev = _plan(B, T, q.device, HV, V // 32)
        chunks, segs = int(plan_host[1]), int(plan_host[2])
        lib = _capi.lib()
        ws_bytes = check(lib.lampa_hgdn_chunk_workspace_bytes(chunks, segs, HV, K, V), "lampa_hgdn_chunk_workspace_bytes")
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        o = torch.empty_like(v)
        check(lib.lampa_hgdn_chunk_fwd(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(lam), _gd._DTYPES[lam.dtype],
                                       float(lam_div), ptr(o),
                                       ctypes.c_void_p(plan_host.data_ptr()), ptr(plan_dev), H, HV, K, V, L,
                                       _gd._DTYPES[q.dtype], float(scale), _gd.L2_CHUNK, ptr(ws), ws_bytes, stream_of(q)),
              "lampa_hgdn_chunk_fwd")
        return o

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("lampa_amd gated-delta operators are forward-only")


def chunk_h_gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, l: torch.Tensor,
                             beta: torch.Tensor, scale: float = None, initial_state=None,
                             output_final_state: bool = False, cu_seqlens: Optional[torch.LongTensor] = None,
                             head_first: bool = False, use_qk_l2norm_in_kernel: bool = False):
    """``gated_delta_rule_apis.py:21-134``. q, k ``[B,T,H,K]``, v ``[B,T,HV,V]``, g, beta ``[B,T,HV]``, l
    ``[B,T,HV,L]`` with ``L >= num_levels(T)``; T a multiple of 64. Returns ``(o, None)``."""
    assert q.dtype == k.dtype == v.dtype
    assert q.dtype != torch.float32, "ChunkGatedDeltaRuleFunction does not support float32. Please use bfloat16."
    assert len(beta.shape) == 3, "beta must be of shape [B, T, H] if head_first=False, or [B, H, T] otherwise."
    assert cu_seqlens is None
    assert use_qk_l2norm_in_kernel is True
    if head_first:
        raise DeprecationWarning(
            "head_first is deprecated and will be removed in a future version. "
            "Please use head_first=False for now instead.")
    if q.shape[1] < q.shape[2]:
        warnings.warn(
            f"Input tensor shape suggests potential format mismatch: seq_len ({q.shape[1]}) < num_heads ({q.shape[2]}). "
            "This may indicate the inputs were passed in head-first format [B, H, T, ...] "
            "when head_first=False was specified. "
            "Please verify your input tensor format matches the expected shape [B, T, H, ...].")
    if scale is None:
        scale = k.shape[-1] ** -0.5
    lam_div = scale if SCALE_LAMBDA else 1.0  # l = l / scale (gated_delta_rule_apis.py:68-70), done by the kernel
    if output_final_state or initial_state is not None:
        raise NotImplementedError("hierarchical final / initial states are not built")
    B, T, H, K = q.shape
    if T % 64 != 0:  # chunkwise_hgdn.py:598-601
        raise ValueError(f"T={T} and BT=64")
    if K != 64 or v.shape[-1] not in (64, 128):
        raise NotImplementedError("hierarchical forward: K = 64 and V in {64, 128} only")
    if num_levels(T) > l.shape[-1]:  # chunkwise_hgdn.py:718-721
        raise ValueError
    if (T // 64) > 4096:
        raise NotImplementedError("hierarchical forward: at most 4096 chunks per sequence")
    o = _ForwardOnly.apply(q, k, v, g, l, beta, scale, lam_div)
    return o, None
