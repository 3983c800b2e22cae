"""Hierarchical (level-weighted) gated-delta forward on the GPU behind the reference's operator signature.

``chunk_h_gated_delta_rule`` (reference ``models/hattention/gated_delta_rule_apis.py:21-134``): same argument names,
order, defaults and checks. The reference evaluates it with Triton kernels (``chunkwise_hgdn.py:565-791``), which
cannot run here, so the function implemented is the token loop the reference keeps as its specification,
``hattention_recurrent`` (``recurrent.py:169-216``). The reference's chunk pipeline is the same function for g <= 0:
its two inverses ``Aw = (I + tril(beta K K^T))^-1`` and ``Au = (I + tril(beta K K^T . e^{gamma_i - gamma_j}))^-1``
(``fla_future/chunk_scaled_dot_kkt.py:62-77``, ``chunkwise_hgdn.py:651-676``) are related by
``Au = diag(e^gamma) Aw diag(e^-gamma)``, so its ``w_new = e^gamma (Aw beta K)`` (``fla_future/chunk_delta_h.py:449-453``)
equals ``Au diag(beta e^gamma) K``, the W of the one-inverse form used here, and its per-level state passes
(``chunkwise_hgdn.py:725-760``: sources masked where the level's bit of the chunk index is set, state reset at the end
of each period) hold exactly the buckets of the token loop's level states. The operator is reached the way the
reference reaches it: q l2-normalised and scaled, k l2-normalised (``kernel.py:100-101``), lambda divided by ``scale``
(``gated_delta_rule_apis.py:68-70``; the kernel does it, with the rounding of a division in lambda's dtype), weak
hierarchy, base 2.

All three branches of the operator are here: outputs only (``hattention_kernel``), prefill returning the level
states (``hattention_prefill``, ``kernel.py:467-575``: the whole chunks through the chunk kernels, the remaining
tokens one by one) and the single-token step on an ``HState`` (``hattention_step``, ``kernel.py:577-633``).

Differences a caller can observe: forward only; the chunk kernels are built for K = 64 and V in {64, 128}, smaller
heads are zero-padded to those, larger ones are refused (the single-token step takes any K and V, up to 32 levels); ``HState.counts`` lives on the host (the reference keeps it on the device and synchronises
on every comparison, ``recurrent.py:44-56``); the step computes its output from the fp32 states, the reference rounds
them to the output type first (``kernel.py:628-631``).
"""
import ctypes
import enum
import warnings
from typing import Optional, Tuple

import torch

from . import _capi
from . import gated_delta as _gd
from ._capi import check, ptr, require_cuda, stream_of

SCALE_LAMBDA = True  # gated_delta_rule_apis.py:17

# Chunks per segment of the split-sequence walk (a power of two); None picks it from the sequence length.
CHUNKS_PER_SEGMENT: Optional[int] = None

_plan_cache = {}


class HType(enum.Enum):  # base.py:12-14
    WEAK = 0
    STRONG = 1


class HStruct(enum.Enum):  # base.py:17-19
    MAMBA2 = 0
    GDELTA = 1


class HState(object):
    """Level states of one batch: ``recurrent.py:9-132``. ``states`` fp32 ``[B, HV, K, V, L]``, ``counts`` int32
    ``[L]`` (tokens per level). The cascade, the gate and the insert run inside the step kernel; the bookkeeping of
    the counts (``cascade_weak``, ``recurrent.py:44-56``) is replayed on host integers."""

    def __init__(self, base: int, htype: HType, hstruct: HStruct, shape: Tuple[int, ...], dtype: torch.dtype,
                 device: torch.device) -> None:
        if htype != HType.WEAK or base != 2 or hstruct != HStruct.GDELTA:
            raise NotImplementedError
        self.base, self.htype, self.hstruct = base, htype, hstruct
        self.shape, self.dtype, self.device = tuple(shape), dtype, device
        self.max_num_levels = self.shape[-1]
        self.states = torch.zeros(self.shape, dtype=self.dtype, device=self.device)
        self._counts = [0] * self.max_num_levels  # host integers; ``counts`` shows them as the reference's tensor

    @property
    def counts(self) -> torch.Tensor:
        return torch.tensor(self._counts, dtype=torch.int32)

    @counts.setter
    def counts(self, value) -> None:
        self._counts = [int(c) for c in value]

    @property
    def tokens_seen(self) -> int:
        return sum(self._counts)

    def cascade_weak(self) -> int:
        """Replays ``recurrent.py:44-56`` on the counts; returns the level that received the full ones (0: none)."""
        z, counts = 0, self._counts
        for level in range(self.max_num_levels):
            capacity = self.base ** level
            if counts[level] == capacity:
                if level + 1 >= self.max_num_levels:
                    raise ValueError("the state has no level left for this many tokens")
                counts[level + 1] += counts[level]
                counts[level] = 0
                z = level + 1
            elif counts[level] < capacity:
                break
            else:
                raise ValueError
        return z

    def reset_states(self) -> None:
        self.states = torch.zeros_like(self.states)

    def replace(self, other: "HState") -> None:
        if not all([tuple(self.shape) == tuple(other.shape), self.base == other.base, self.htype == other.htype,
                    self.dtype == other.dtype, self.device == other.device]):
            raise ValueError("Shape, dtype or device mismatch")
        self.states = other.states

    def to(self, dtype: Optional[torch.dtype] = None, device: Optional[torch.device] = None) -> "HState":
        new_state = HState(self.base, self.htype, self.hstruct, self.shape, dtype or self.dtype, device or self.device)
        new_state.states = self.states.to(dtype=new_state.dtype, device=new_state.device)
        new_state._counts = list(self._counts)
        return new_state


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
    def forward(ctx, q, k, v, g, lam, beta, scale, lam_div, level_states=None):
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
                                       float(lam_div), ptr(o), ptr(level_states),
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
    ``[B,T,HV,L]`` with ``L >= num_levels(T)``. ``output_final_state=False``: T a multiple of 64, returns ``(o, None)``;
    ``output_final_state=True``: any T, returns ``(o, HState)``; with ``initial_state`` (an ``HState``) and T = 1: one
    step, returns ``(o, initial_state)`` updated in place."""
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
    B, T, H, K = q.shape
    HV, V, L = v.shape[2], v.shape[3], l.shape[-1]
    if output_final_state is False:
        if initial_state is not None:
            raise NotImplementedError
        _check_chunk_shapes(T, K, V, L)
        if T % 64 != 0:  # chunkwise_hgdn.py:598-601
            raise ValueError(f"T={T} and BT=64")
        pq, pk, pv = _pad_heads(q, k, v)
        return _ForwardOnly.apply(pq, pk, pv, g, l, beta, scale, lam_div)[..., :V].contiguous(), None
    if initial_state is None:  # hattention_prefill, kernel.py:467-575
        require_cuda(q, k, v, g, l, beta)
        hstate = HState(2, HType.WEAK, HStruct.GDELTA, (B, HV, K, V, L), torch.float32, q.device)
        T0 = T - T % 64
        o = torch.empty_like(v)
        if T0:
            _check_chunk_shapes(T0, K, V, L)
            cut = lambda x: x[:, :T0]
            pq, pk, pv = _pad_heads(cut(q), cut(k), cut(v))
            padded = pq.shape[-1] != K or pv.shape[-1] != V
            states = (torch.zeros(B, HV, pq.shape[-1], pv.shape[-1], L, dtype=torch.float32, device=q.device)
                      if padded else hstate.states)
            o[:, :T0] = _ForwardOnly.apply(pq, pk, pv, cut(g), cut(l), cut(beta), scale, lam_div, states)[..., :V]
            if padded:  # (the padded rows and columns of the states are zero)
                hstate.states = states[:, :, :K, :V].contiguous()
            # counts after T0 tokens (kernel.py:451-462): the last token alone in level 0, level l > 0 holds 2^(l-1)
            # tokens iff that bit of T0 - 1 is set
            hstate._counts[0] = 1
            for level in range(1, L):
                hstate._counts[level] = (1 << (level - 1)) if ((T0 - 1) >> (level - 1)) & 1 else 0
        for t in range(T0, T):
            o[:, t] = _step(hstate, q[:, t], k[:, t], v[:, t], g[:, t], l[:, t], beta[:, t], scale, lam_div)
        return o, hstate
    if not all([q.ndim == 4, q.shape[1] == 1, k.ndim == 4, k.shape[1] == 1, v.ndim == 4, v.shape[1] == 1,
                beta.ndim == 3, beta.shape[1] == 1, g.ndim == 3, g.shape[1] == 1, l.ndim == 4, l.shape[1] == 1]):
        raise ValueError
    return _step(initial_state, q, k, v, g, l, beta, scale, lam_div, token_dim=True), initial_state


def _pad_heads(q, k, v):
    """The chunk kernels are built for K = 64 and V in {64, 128}; smaller heads are zero-padded along the head
    dimension: zero columns of k and q add nothing to k k^T, q k^T, q S or the norms, zero columns of v give zero
    columns of every level state and of o, so the padded problem contains the original one exactly (`scale` is fixed
    from the original K by the caller)."""
    K, V = q.shape[-1], v.shape[-1]
    Kp, Vp = 64, (64 if V <= 64 else 128)
    pad = torch.nn.functional.pad
    return (q if K == Kp else pad(q, (0, Kp - K)), k if K == Kp else pad(k, (0, Kp - K)),
            v if V == Vp else pad(v, (0, Vp - V)))


def _check_chunk_shapes(T: int, K: int, V: int, L: int) -> None:
    if K > 64 or V > 128:
        raise NotImplementedError("hierarchical chunk kernels: K <= 64 and V <= 128 only")
    if num_levels(T) > L:  # chunkwise_hgdn.py:718-721
        raise ValueError
    if (T // 64) > 4096:
        raise NotImplementedError("hierarchical chunk kernels: at most 4096 chunks per sequence")


def _step(hstate: HState, q, k, v, g, l, beta, scale, lam_div, token_dim: bool = False) -> torch.Tensor:
    """``hattention_step`` (``kernel.py:577-633``) on ``[B, H, K]`` / ``[B, HV, V]`` / ``[B, HV]`` / ``[B, HV, L]``
    slices -- or, with ``token_dim``, on the operator's own ``[B, 1, ...]`` tensors, which are the same memory when
    contiguous (no slicing on the way to the kernel); updates ``hstate`` in place and returns ``o`` shaped like ``v``."""
    t = 1 if token_dim else 0
    if not all([q.ndim == 3 + t, k.ndim == 3 + t, v.ndim == 3 + t, beta.ndim == 2 + t, g.ndim == 2 + t, l.ndim == 3 + t,
                hstate.dtype == torch.float32, q.dtype == k.dtype == v.dtype, hstate.base == 2,
                hstate.htype == HType.WEAK, hstate.hstruct == HStruct.GDELTA]):
        raise TypeError
    require_cuda(q, k, v, g, l, beta, hstate.states)
    B, H, K = q.shape[0], q.shape[-2], q.shape[-1]
    HV, V, L = v.shape[-2], v.shape[-1], l.shape[-1]
    if tuple(hstate.shape) != (B, HV, K, V, L):
        raise ValueError("Shape, dtype or device mismatch")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    g, beta = g.to(torch.float32).contiguous(), beta.to(torch.float32).contiguous()
    if l.dtype not in _gd._DTYPES:
        l = l.to(torch.float32)
    l = l.contiguous()
    if not hstate.states.is_contiguous():
        hstate.states = hstate.states.contiguous()
    z = hstate.cascade_weak()
    o = torch.empty_like(v)
    check(_capi.lib().lampa_hgdn_step(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(l), _gd._DTYPES[l.dtype],
                                      float(lam_div), ptr(hstate.states), ptr(o), B, H, HV, K, V, L, z,
                                      _gd._DTYPES[q.dtype], float(scale), _gd.L2_CHUNK, stream_of(q)), "lampa_hgdn_step")
    hstate._counts[0] += 1
    return o
