"""Gated-delta-rule forward on the GPU behind the reference's operator signatures.

``chunk_gated_delta_rule`` (reference ``models/hattention/gated_delta_rule_ori.py:236-357``) and
``fused_recurrent_gated_delta_rule`` (``gated_delta_rule_ori.py:565-667``): same argument names, order,
defaults, checks and return tuples.  The arithmetic runs in hand-written gfx950 kernels reached through the
C ABI of ``liblampa_amd.so``; there is no Triton, no PyTorch fallback and no CPU path.

Differences that a caller can observe, all additive:
* ``chunk_gated_delta_rule`` is differentiable (``lampa_gdr_bwd``: fp32, token-serial inside parallel segments);
  ``fused_recurrent_gated_delta_rule``'s backward raises ``NotImplementedError`` as the reference's does;
* ``allow_fp32=True`` lets ``chunk_gated_delta_rule`` accept float32 q/k/v (the reference rejects them); they
  are evaluated by the token-serial fp32 kernel (long sequences cut into segments that run in parallel);
* head sizes up to 128 other than the built ones (K, V in {64, 128} and 32 x 32) are zero-padded along the head
  dimension to the next built shape and run on the same chunk kernels; larger heads take the token-serial kernel.
"""
import ctypes
import math
import warnings
from typing import Optional

import torch

from . import _capi
from ._capi import check, ptr, require_cuda, stream_of

L2_NONE, L2_CHUNK, L2_RECURRENT = 0, 1, 2
_DTYPES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

# Number of 64-token chunks per segment of the split-sequence scan; None picks it from the sequence lengths.
CHUNKS_PER_SEGMENT: Optional[int] = None

_plan_cache = {}


def _sequence_bounds(cu_seqlens, B: int, T: int):
    """Token boundaries of the sequences as a Python list. ``cu_seqlens`` must start at 0, never decrease and end at
    the number of tokens that were passed (B * T): the kernels index q, k, v and the outputs with these numbers, so a
    boundary beyond the tensors would be an out-of-range access on the GPU, and tokens outside every sequence would
    keep uninitialised outputs and gradients."""
    if cu_seqlens is None:
        return [i * T for i in range(B + 1)]
    # Reading a device tensor on the host drains the stream, so the validated list is remembered for the tensor OBJECT it
    # was read from (and the version counter that in-place writes bump), as the reference's `tensor_cache` does for its
    # `prepare_chunk_indices` (models/hattention/fla_utils.py:88-125, index.py:69-83): a loop that passes the same `cu_seqlens`
    # tensor every step pays the copy once.
    for ref, version, key, cached in _bounds_cache:
        if ref is cu_seqlens and version == cu_seqlens._version and key == (B, T):
            return cached
    cu = [int(c) for c in cu_seqlens.tolist()]
    if len(cu) < 2:
        raise ValueError(f"cu_seqlens must hold at least two entries (one sequence), got {len(cu)}")
    if cu[0] != 0 or cu[-1] != B * T or any(b < a for a, b in zip(cu[:-1], cu[1:])):
        raise ValueError(f"cu_seqlens must start at 0, be non-decreasing and end at the number of tokens ({B * T}); "
                         f"got first = {cu[0]}, last = {cu[-1]}"
                         + ("" if all(b >= a for a, b in zip(cu[:-1], cu[1:])) else ", not monotone"))
    _bounds_cache.insert(0, (cu_seqlens, cu_seqlens._version, (B, T), cu))
    del _bounds_cache[4:]
    return cu


_bounds_cache = []  # (tensor, its version when read, (B, T), validated list), most recent first


def _default_chunks_per_segment(chunks_per_seq, n_value_heads: int, slots: int) -> int:
    """Segment length of the split-sequence scan. One workgroup walks one (segment, head) chunk by chunk, so the two
    segment kernels take (chunks per segment) chunk periods as long as all workgroups are resident at once
    (``slots`` = workgroups the chip holds), and the scan in between is serial in the segments per sequence:
    the shortest segments that still fit are best."""
    cps = 4
    while cps < MAX_CHUNKS_PER_SEGMENT and sum((n + cps - 1) // cps for n in chunks_per_seq) * n_value_heads > slots:
        cps += 1
    return cps


MAX_CHUNKS_PER_SEGMENT = 64


LONG_SEGMENT_FACTOR = 1.17


def _default_segmentation(chunks_per_seq, n_value_heads: int, slots: int, per_cu: int = 1):
    """How the sequences are cut into segments: ("cps", chunks per segment), ("balanced", total segments) or
    ("lengths", [chunks of every segment, sequence after sequence]).

    * One round of workgroups, two per CU (heads up to 64 x 64): the workgroups with the lowest indices start first, one
      per CU, and keep the larger share of their CU when the second one arrives; the plan orders the segments by length,
      so the first half of every sequence's segments is made LONG_SEGMENT_FACTOR times the average and the second half
      (which also walks more composites before its first chunk) correspondingly shorter. Measured against segments of one
      length, bf16, K = V = 64: 60 000 tokens x 8 heads 124.1 -> 120.9 us, 30 016 x 8 80.0 -> 75.8 us, 120 000 x 8
      255.1 -> 250.7 us, 60 000 x 4 82.4 -> 80.1 us (factors 1.1 / 1.17 / 1.23 / 1.3 at 60 000 x 8: 122.0 / 120.9 / 120.7 /
      123.3 us).
    * When even segments of MAX_CHUNKS_PER_SEGMENT chunks give more workgroups than the chip holds, they run in rounds,
      and with one fixed length the last round is partly empty while every round lasts a full segment (config 4: 1 064
      workgroups on 256 slots = 4.2 rounds that take the time of 5). The plan then deals out a whole number of rounds of
      segments of nearly equal length instead (4 rounds of 51-68 chunks there)."""
    cps = _default_chunks_per_segment(chunks_per_seq, n_value_heads, slots)
    if sum(max(1, (n + cps - 1) // cps) for n in chunks_per_seq) * n_value_heads > slots:
        work = sum(chunks_per_seq) * n_value_heads
        rounds = (work + slots * MAX_CHUNKS_PER_SEGMENT - 1) // (slots * MAX_CHUNKS_PER_SEGMENT)
        return "balanced", max(1, rounds * slots // n_value_heads)
    total = slots // n_value_heads
    if per_cu != 2 or cps <= 4 or total < 2 * len(chunks_per_seq):
        return "cps", cps
    # segments per sequence as the balanced plan deals them (the longest segments as short as possible) ...
    ns = [1] * len(chunks_per_seq)
    for _ in range(total - len(ns)):
        best = max(range(len(ns)), key=lambda i: (chunks_per_seq[i] / ns[i], -i))
        if chunks_per_seq[best] <= ns[best]:
            break
        ns[best] += 1
    # ... and within a sequence the first half long, the rest evenly over what is left
    lens = []
    for n, k in zip(chunks_per_seq, ns):
        n_long = k // 2
        l_long = int(round(LONG_SEGMENT_FACTOR * n / k)) if n_long else 0
        rest, n_short = n - n_long * l_long, k - n_long
        if n_long and rest < n_short:  # too few chunks for that: equal lengths
            n_long, rest, n_short = 0, n, k
        lo, longer = divmod(rest, n_short)
        lens += [l_long] * n_long + [lo + (1 if i < longer else 0) for i in range(n_short)]
    return "lengths", lens


def _plan(cu_host, device, n_value_heads: int, head_dims):
    """Host + device copies of the chunk/segment tables for these sequence boundaries (cached)."""
    kind, arg = "cps", CHUNKS_PER_SEGMENT
    if not arg:
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        per_cu = 2 if max(head_dims) <= 64 else 1  # workgroups of the segment kernels a CU holds (LDS, registers)
        chunks_per_seq = [(b - a + 63) // 64 for a, b in zip(cu_host[:-1], cu_host[1:])]
        kind, arg = _default_segmentation(chunks_per_seq, n_value_heads, per_cu * cus, per_cu)
    key = (tuple(cu_host), kind, tuple(arg) if kind == "lengths" else arg, str(device))
    hit = _plan_cache.get(key)
    if hit is not None:
        return hit
    lib = _capi.lib()
    cu = (ctypes.c_int64 * len(cu_host))(*cu_host)
    n_seq = len(cu_host) - 1
    if kind == "lengths":
        arr = (ctypes.c_int32 * len(arg))(*arg)
        size = check(lib.lampa_gdr_plan_size_lengths(cu, n_seq, arr, len(arg)), "lampa_gdr_plan_size_lengths")
        host = torch.empty(size, dtype=torch.int32)
        check(lib.lampa_gdr_plan_fill_lengths(cu, n_seq, arr, len(arg), ctypes.c_void_p(host.data_ptr())),
              "lampa_gdr_plan_fill_lengths")
    else:
        size_fn, fill_fn = ((lib.lampa_gdr_plan_size_balanced, lib.lampa_gdr_plan_fill_balanced) if kind == "balanced"
                            else (lib.lampa_gdr_plan_size, lib.lampa_gdr_plan_fill))
        size = check(size_fn(cu, n_seq, arg), "lampa_gdr_plan_size")
        host = torch.empty(size, dtype=torch.int32)
        check(fill_fn(cu, n_seq, arg, ctypes.c_void_p(host.data_ptr())), "lampa_gdr_plan_fill")
    dev = host.to(device)
    if len(_plan_cache) > 64:
        _plan_cache.clear()
    _plan_cache[key] = (host, dev)
    return host, dev


def output_pass_config(narrow: int = 1) -> None:
    """Process-wide form of the chunk forward's output pass (``lampa_gdr_chunk_config``): 0 = 32 value columns per
    recurrence wave everywhere, 1 = 16 columns ("narrow" waves on the 16x16x32 MFMA) for heads wider than 64 x 64, where
    it is the faster form (the default), 2 = narrow wherever it is built (K >= 64). For A/B measurements and tests."""
    check(_capi.lib().lampa_gdr_chunk_config(int(narrow)), "lampa_gdr_chunk_config")


# Token-serial operator: sequences at least this long are cut into segments that run in parallel when the launch
# would otherwise occupy less than a quarter of the chip (None: never).
SEGMENT_MIN_TOKENS: Optional[int] = 512

_segment_cache = {}


def _segment_tables(cu_host, seg_len: int, device):
    """Device tables of ``lampa_gdr_recurrent_segmented_fwd``: every sequence cut into segments of ``seg_len`` tokens
    (an empty sequence keeps one empty segment, so that its final state is still written)."""
    key = (tuple(cu_host), seg_len, str(device))
    hit = _segment_cache.get(key)
    if hit is not None:
        return hit
    cu_seg, seq_seg0, seg_out = [], [], []
    for s, (a, b) in enumerate(zip(cu_host[:-1], cu_host[1:])):
        seq_seg0.append(len(cu_seg))
        starts = list(range(a, b, seg_len)) or [a]
        cu_seg.extend(starts)
        seg_out.extend([-1] * (len(starts) - 1) + [s])
    seq_seg0.append(len(cu_seg))
    cu_seg.append(cu_host[-1])
    tables = (torch.tensor(cu_seg, dtype=torch.int64).to(device), torch.tensor(seq_seg0, dtype=torch.int32).to(device),
              torch.tensor(seg_out, dtype=torch.int32).to(device), len(seg_out))
    if len(_segment_cache) > 64:
        _segment_cache.clear()
    _segment_cache[key] = tables
    return tables


def _recurrent_segmented_launch(q, k, v, g, beta, scale, initial_state, output_final_state, cu_host, seg_len, l2norm):
    H, K = q.shape[2], q.shape[3]
    HV, V = v.shape[2], v.shape[3]
    n_seq = len(cu_host) - 1
    cu_seg, seq_seg0, seg_out, n_seg = _segment_tables(cu_host, seg_len, q.device)
    lib = _capi.lib()
    ws_bytes = check(lib.lampa_gdr_recurrent_segmented_workspace_bytes(n_seg, HV, K, V),
                     "lampa_gdr_recurrent_segmented_workspace_bytes")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    o = torch.empty_like(v)
    ht = torch.empty((n_seq, HV, K, V), dtype=torch.float32, device=q.device) if output_final_state else None
    h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
    check(lib.lampa_gdr_recurrent_segmented_fwd(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(o), ptr(h0), ptr(ht),
                                                ptr(cu_seg), ptr(seq_seg0), ptr(seg_out), n_seq, n_seg, H, HV, K, V,
                                                _DTYPES[q.dtype], float(scale), l2norm, ptr(ws), ws_bytes,
                                                stream_of(q)), "lampa_gdr_recurrent_segmented_fwd")
    return o, ht


def _recurrent_launch(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm):
    B, T, H, K = q.shape
    HV, V = v.shape[2], v.shape[3]
    n_seq = B if cu_seqlens is None else len(cu_seqlens) - 1
    slabs = (V + 31) // 32
    headwise = beta.dim() == 4  # one beta per value column (the reference's IS_BETA_HEADWISE)
    if (not headwise and SEGMENT_MIN_TOKENS and K % 4 == 0 and V % 4 == 0 and K <= 128 and n_seq * HV * slabs <= 256
            and q.shape[0] * T >= SEGMENT_MIN_TOKENS and q.data_ptr() % 16 == 0 and k.data_ptr() % 16 == 0):
        # a few long sequences: one or two waves each would leave most of the chip idle
        cu_host = _sequence_bounds(cu_seqlens, B, T)
        if max(b - a for a, b in zip(cu_host[:-1], cu_host[1:])) >= SEGMENT_MIN_TOKENS:
            want = max(1, 1024 // (HV * slabs))  # segments for about one wave per SIMD in the output pass (the scan
            # between the passes is serial in the groups of segments: no more of them than fill the chip)
            seg_len = max(64, -(-(cu_host[-1] // want) // 64) * 64)
            return _recurrent_segmented_launch(q, k, v, g, beta, scale, initial_state, output_final_state, cu_host,
                                               seg_len, l2norm)
    if cu_seqlens is not None:
        _sequence_bounds(cu_seqlens, B, T)
    o = torch.empty_like(v)
    ht = torch.empty((n_seq, HV, K, V), dtype=torch.float32, device=q.device) if output_final_state else None
    cu = None if cu_seqlens is None else cu_seqlens.to(device=q.device, dtype=torch.int64).contiguous()
    h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
    fn = _capi.lib().lampa_gdr_recurrent_headwise_fwd if headwise else _capi.lib().lampa_gdr_recurrent_fwd
    check(fn(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(o), ptr(h0), ptr(ht), ptr(cu), n_seq, T, H, HV, K, V,
             _DTYPES[q.dtype], float(scale), l2norm, stream_of(q)), "lampa_gdr_recurrent_fwd")
    return o, ht


def _chunk_launch(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm):
    B, T, H, K = q.shape
    HV, V = v.shape[2], v.shape[3]
    cu_host = _sequence_bounds(cu_seqlens, B, T)
    n_seq = len(cu_host) - 1
    plan_host, plan_dev = _plan(cu_host, q.device, HV, (K, V))
    chunks, segs = int(plan_host[1]), int(plan_host[2])
    lib = _capi.lib()
    ws_bytes = check(lib.lampa_gdr_chunk_workspace_bytes(chunks, segs, HV, K, V), "lampa_gdr_chunk_workspace_bytes")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    o = torch.empty_like(v)
    ht = torch.empty((n_seq, HV, K, V), dtype=torch.float32, device=q.device) if output_final_state else None
    h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
    check(lib.lampa_gdr_chunk_fwd(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(o), ptr(h0), ptr(ht),
                                  ctypes.c_void_p(plan_host.data_ptr()), ptr(plan_dev), H, HV, K, V, _DTYPES[q.dtype],
                                  float(scale), l2norm, ptr(ws), ws_bytes, stream_of(q)), "lampa_gdr_chunk_fwd")
    return o, ht


def _chunk_path_supported(q, v) -> bool:
    return q.dtype in (torch.bfloat16, torch.float16) and q.shape[-1] <= 128 and v.shape[-1] <= 128


def _chunk_head_sizes(K: int, V: int):
    """The chunk kernels are built for K, V in {64, 128} and for K = V = 32; other head sizes run as the next larger
    built shape."""
    if K <= 32 and V <= 32:
        return 32, 32
    return (64 if K <= 64 else 128), (64 if V <= 64 else 128)


def _chunk_launch_any_head(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm):
    """Head sizes that are not built (the reference's layer uses d_k = 16, d_v = 32,
    ``modeling_gated_deltaproduct.py:583-587``): q, k and v are zero-padded along the head dimension. Zero columns
    of k and q add nothing to k k^T, q k^T, q S or the norms, zero columns of v give zero columns of the state and
    of o, so the padded problem contains the original one exactly; `scale` was fixed from the original K."""
    K, V = q.shape[-1], v.shape[-1]
    Kp, Vp = _chunk_head_sizes(K, V)
    if (Kp, Vp) == (K, V):
        return _chunk_launch(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm)
    pad = torch.nn.functional.pad
    h0 = None if initial_state is None else pad(initial_state.to(torch.float32), (0, Vp - V, 0, Kp - K))
    o, ht = _chunk_launch(pad(q, (0, Kp - K)), pad(k, (0, Kp - K)), pad(v, (0, Vp - V)), g, beta, scale, h0,
                          output_final_state, cu_seqlens, l2norm)
    return o[..., :V].contiguous(), None if ht is None else ht[..., :K, :V].contiguous()


# Backward pass: about this many (segment, value head, 16-column slab) units, one wavefront each.
BACKWARD_UNITS = 2048

_backward_tables_cache = {}


def _backward_tables(cu_host, seg_len: int, device):
    """The segment tables of ``lampa_gdr_bwd``: those of the segmented forward plus, for the pass that runs backwards,
    one extra row per sequence (``seq_seg0_rev``) and every segment's row counted from its sequence's end."""
    key = (tuple(cu_host), seg_len, str(device))
    hit = _backward_tables_cache.get(key)
    if hit is not None:
        return hit
    cu_seg, seq_seg0, _, n_seg = _segment_tables(cu_host, seg_len, device)
    first = seq_seg0.tolist()
    rev0 = [p + s for s, p in enumerate(first)]
    seg_rev = []
    for s in range(len(first) - 1):
        seg_rev.extend(rev0[s] + (first[s + 1] - 1) - p for p in range(first[s], first[s + 1]))
    tables = (cu_seg, seq_seg0, torch.tensor(rev0, dtype=torch.int32).to(device),
              torch.tensor(seg_rev, dtype=torch.int32).to(device), n_seg)
    if len(_backward_tables_cache) > 64:
        _backward_tables_cache.clear()
    _backward_tables_cache[key] = tables
    return tables


# Backward pass in the chunked form on the matrix cores (``lampa_gdr_bwd_chunk``) where it is built: 16-bit inputs,
# K = V = 64, one value head per q/k head. False sends everything to the fp32 token-serial form (``lampa_gdr_bwd``).
CHUNKED_BACKWARD = True

_backward_plan_cache = {}


def _backward_chunk_plan(cu_host, device):
    """Host + device copies of the chunk tables of ``lampa_gdr_bwd_chunk`` for these sequence boundaries (cached)."""
    key = (tuple(cu_host), str(device))
    hit = _backward_plan_cache.get(key)
    if hit is not None:
        return hit
    lib = _capi.lib()
    cu = (ctypes.c_int64 * len(cu_host))(*cu_host)
    n_seq = len(cu_host) - 1
    size = check(lib.lampa_gdr_bwd_chunk_plan_size(cu, n_seq), "lampa_gdr_bwd_chunk_plan_size")
    host = torch.empty(size, dtype=torch.int32)
    check(lib.lampa_gdr_bwd_chunk_plan_fill(cu, n_seq, ctypes.c_void_p(host.data_ptr())), "lampa_gdr_bwd_chunk_plan_fill")
    dev = host.to(device)
    if len(_backward_plan_cache) > 64:
        _backward_plan_cache.clear()
    _backward_plan_cache[key] = (host, dev)
    return host, dev


def _backward_chunk_supported(q, v) -> bool:
    """16-bit inputs with K, V <= 64: smaller heads are zero-padded to 64 x 64 (as in the forward pass: zero columns of
    q, k and v change neither the function nor the other columns' gradients), and grouped value heads (HV > H) run with
    q and k repeated per value head, their gradients summed over each group afterwards."""
    return (CHUNKED_BACKWARD and q.dtype in (torch.bfloat16, torch.float16) and q.shape[-1] <= 64 and v.shape[-1] <= 64
            and q.data_ptr() % 16 == 0)


def _backward_chunk_launch(q, k, v, g, beta, scale, initial_state, cu_seqlens, l2norm, do, dht):
    """Gradients (dq, dk, dv, dg, dbeta, dh0) through ``lampa_gdr_bwd_chunk`` (built for K = V = 64, HV = H)."""
    B, T, H, K = q.shape
    HV, V = v.shape[2], v.shape[3]
    pad = torch.nn.functional.pad
    if K < 64:
        q, k = pad(q, (0, 64 - K)), pad(k, (0, 64 - K))
    if V < 64:
        v, do = pad(v, (0, 64 - V)), pad(do, (0, 64 - V))
    if (K, V) != (64, 64):
        initial_state = None if initial_state is None else pad(initial_state.to(torch.float32), (0, 64 - V, 0, 64 - K))
        dht = None if dht is None else pad(dht.to(torch.float32), (0, 64 - V, 0, 64 - K))
    rep = HV // H
    if rep > 1:
        q, k = q.repeat_interleave(rep, dim=2), k.repeat_interleave(rep, dim=2)
    q, k, v, do = q.contiguous(), k.contiguous(), v.contiguous(), do.contiguous()
    cu_host = _sequence_bounds(cu_seqlens, B, T)
    plan_host, plan_dev = _backward_chunk_plan(cu_host, q.device)
    lib = _capi.lib()
    ws_bytes = check(lib.lampa_gdr_bwd_chunk_workspace_bytes(ctypes.c_void_p(plan_host.data_ptr()), HV),
                     "lampa_gdr_bwd_chunk_workspace_bytes")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dg, dbeta = torch.empty_like(g), torch.empty_like(beta)
    h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
    dht = None if dht is None else dht.to(torch.float32).contiguous()
    dh0 = None if h0 is None else torch.empty_like(h0)
    check(lib.lampa_gdr_bwd_chunk(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(h0), ptr(do), ptr(dht), ptr(dq), ptr(dk),
                                  ptr(dv), ptr(dg), ptr(dbeta), ptr(dh0), ctypes.c_void_p(plan_host.data_ptr()),
                                  ptr(plan_dev), HV, HV, 64, 64, _DTYPES[q.dtype], float(scale), l2norm, ptr(ws), ws_bytes,
                                  stream_of(q)), "lampa_gdr_bwd_chunk")
    if rep > 1:  # the value heads of a group share their q / k head
        dq = dq.view(B, T, H, rep, 64).float().sum(3).to(q.dtype)
        dk = dk.view(B, T, H, rep, 64).float().sum(3).to(k.dtype)
    if (K, V) != (64, 64):
        dq, dk, dv = dq[..., :K].contiguous(), dk[..., :K].contiguous(), dv[..., :V].contiguous()
        dh0 = None if dh0 is None else dh0[..., :K, :V].contiguous()
    return dq, dk, dv, dg, dbeta, dh0


def _backward_launch(q, k, v, g, beta, scale, initial_state, cu_seqlens, l2norm, do, dht):
    """Gradients (dq, dk, dv, dg, dbeta, dh0) through ``lampa_gdr_bwd``. Head sizes that are not multiples of 4 are
    zero-padded (zero columns of q, k and v change neither the function nor the other columns' gradients)."""
    if _backward_chunk_supported(q, v) and q.shape[0] * q.shape[1] > 0:
        return _backward_chunk_launch(q, k, v, g, beta, scale, initial_state, cu_seqlens, l2norm, do, dht)
    B, T, H, K = q.shape
    HV, V = v.shape[2], v.shape[3]
    if K > 128:
        raise NotImplementedError(f"backward of the gated-delta operators is built for K <= 128, got K = {K}")
    Kp, Vp = -(-K // 4) * 4, -(-V // 4) * 4
    pad = torch.nn.functional.pad
    if (Kp, Vp) != (K, V):
        q, k, v, do = pad(q, (0, Kp - K)), pad(k, (0, Kp - K)), pad(v, (0, Vp - V)), pad(do, (0, Vp - V))
        initial_state = None if initial_state is None else pad(initial_state, (0, Vp - V, 0, Kp - K))
        dht = None if dht is None else pad(dht, (0, Vp - V, 0, Kp - K))
    q, k, v, do = q.contiguous(), k.contiguous(), v.contiguous(), do.contiguous()
    cu_host = _sequence_bounds(cu_seqlens, B, T)
    n_seq, total = len(cu_host) - 1, B * T
    slabs = (Vp + 15) // 16
    want = max(1, BACKWARD_UNITS // (HV * slabs))
    seg_len = max(64, -(-(total // want) // 64) * 64)
    cu_seg, seq_seg0, seq_seg0_rev, seg_rev, n_seg = _backward_tables(cu_host, seg_len, q.device)
    lib = _capi.lib()
    ws_bytes = check(lib.lampa_gdr_bwd_workspace_bytes(total, n_seq, n_seg, HV, Kp, Vp), "lampa_gdr_bwd_workspace_bytes")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dg, dbeta = torch.empty_like(g), torch.empty_like(beta)
    h0 = None if initial_state is None else initial_state.to(torch.float32).contiguous()
    dht = None if dht is None else dht.to(torch.float32).contiguous()
    dh0 = None if h0 is None else torch.empty_like(h0)
    check(lib.lampa_gdr_bwd(ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(h0), ptr(do), ptr(dht), ptr(dq), ptr(dk),
                            ptr(dv), ptr(dg), ptr(dbeta), ptr(dh0), ptr(cu_seg), ptr(seq_seg0), ptr(seq_seg0_rev),
                            ptr(seg_rev), total, n_seq, n_seg, H, HV, Kp, Vp, _DTYPES[q.dtype], float(scale), l2norm,
                            ptr(ws), ws_bytes, stream_of(q)), "lampa_gdr_bwd")
    if (Kp, Vp) != (K, V):
        dq, dk, dv = dq[..., :K].contiguous(), dk[..., :K].contiguous(), dv[..., :V].contiguous()
        dh0 = None if dh0 is None else dh0[..., :K, :V].contiguous()
    return dq, dk, dv, dg, dbeta, dh0


class _GatedDelta(torch.autograd.Function):
    """Forward through ``launcher``; backward through ``lampa_gdr_bwd`` (``ChunkGatedDeltaRuleFunction``,
    ``gated_delta_rule_ori.py:163-233``). ``differentiable=False`` keeps the reference's behaviour for the fused
    recurrent operator, whose backward raises (``gated_delta_rule_ori.py:555-562``)."""

    @staticmethod
    def forward(ctx, launcher, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm,
                differentiable):
        require_cuda(q, k, v, g, beta, initial_state)
        ctx.g_dtype, ctx.beta_dtype = g.dtype, beta.dtype
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        g, beta = g.to(torch.float32).contiguous(), beta.to(torch.float32).contiguous()
        ctx.differentiable = differentiable
        if differentiable:
            ctx.save_for_backward(q, k, v, g, beta, initial_state, cu_seqlens)
            ctx.scale, ctx.l2norm = scale, l2norm
        o, ht = launcher(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, l2norm)
        ctx.o_shape, ctx.o_dtype = o.shape, o.dtype
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        if not ctx.differentiable:
            raise NotImplementedError(
                "Backward pass is not implemented yet and we do not have plans to implement it "
                "because we haven't figured out how to compute dg without materializing the full "
                "hidden states for all time steps.")
        q, k, v, g, beta, initial_state, cu_seqlens = ctx.saved_tensors
        if bool((g > 0).any()):
            # the forward masks decay ratios with a positive exponent (safe_exp); the gradients here are those of the
            # unmasked recurrence, which is the same function only for g <= 0
            raise ValueError("chunk_gated_delta_rule backward: g has positive entries; the gradients are defined for "
                             "log-decays g <= 0 only (the forward masks decay ratios with positive exponents, the "
                             "backward pass differentiates the unmasked recurrence)")
        if do is None:
            do = torch.zeros(ctx.o_shape, dtype=ctx.o_dtype, device=q.device)
        dq, dk, dv, dg, dbeta, dh0 = _backward_launch(q, k, v, g, beta, ctx.scale, initial_state, cu_seqlens,
                                                      ctx.l2norm, do.to(v.dtype), dht)
        if dh0 is not None:
            dh0 = dh0.to(initial_state.dtype)
        return (None, dq, dk, dv, dg.to(ctx.g_dtype), dbeta.to(ctx.beta_dtype), None, dh0, None, None, None, None)


def _check_shapes(q, k, v, g, beta, what, headwise_beta_ok=False):
    """g and beta are per (token, value head): [B, T, HV]. The reference's token-serial kernel also takes a headwise
    beta [B, T, HV, V] (``gated_delta_rule_ori.py:444-447,515``), and so does ``fused_recurrent_gated_delta_rule`` here;
    the chunk operator has no such form (the reference asserts ``len(beta.shape) == 3`` there)."""
    if q.dim() != 4 or k.shape != q.shape or v.dim() != 4 or v.shape[:2] != q.shape[:2]:
        raise ValueError(f"{what}: expected q, k [B, T, H, K] and v [B, T, HV, V], got {tuple(q.shape)}, "
                         f"{tuple(k.shape)}, {tuple(v.shape)}")
    if v.shape[2] % q.shape[2] != 0:
        raise ValueError(f"{what}: the number of value heads ({v.shape[2]}) must be a multiple of the number of "
                         f"q/k heads ({q.shape[2]})")
    beta_shapes = [tuple(v.shape[:3])] + ([tuple(v.shape)] if headwise_beta_ok else [])
    if tuple(g.shape) != tuple(v.shape[:3]) or tuple(beta.shape) not in beta_shapes:
        raise ValueError(f"{what}: g must have shape {tuple(v.shape[:3])} (= v.shape[:3]) and beta that shape"
                         + (f" or {tuple(v.shape)} (one value per value column)" if headwise_beta_ok else "")
                         + f", got {tuple(g.shape)} and {tuple(beta.shape)}")


def _check_varlen(q, initial_state, cu_seqlens):
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f"The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`."
                f"Please flatten variable-length inputs before processing.")
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f"The number of initial states is expected to be equal to the number of input sequences, "
                f"i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.")


def chunk_gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, beta: torch.Tensor,
                           scale: float = None, initial_state: torch.Tensor = None, output_final_state: bool = False,
                           cu_seqlens: Optional[torch.LongTensor] = None, head_first: bool = False,
                           use_qk_l2norm_in_kernel: bool = False, *, allow_fp32: bool = False):
    """q, k [B,T,H,K]; v [B,T,H,V]; g (log-decay), beta [B,T,H]; returns (o [B,T,H,V] in q.dtype,
    final_state [N,H,K,V] fp32 or None). See ``gated_delta_rule_ori.py:236-357`` for the argument contract.
    g is meant to be <= 0; for positive entries the chunk kernels do what the reference's do: every ratio of
    cumulative decays inside a chunk goes through ``safe_exp`` (``fla_op.py:27-29``), i.e. it is dropped where its
    exponent is positive."""
    assert q.dtype == k.dtype == v.dtype
    if not allow_fp32:
        assert q.dtype != torch.float32, "ChunkGatedDeltaRuleFunction does not support float32. Please use bfloat16."
    assert len(beta.shape) == 3, "beta must be of shape [B, T, H] if head_first=False, or [B, H, T] otherwise."
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
    _check_shapes(q, k, v, g, beta, "chunk_gated_delta_rule")
    _check_varlen(q, initial_state, cu_seqlens)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    l2norm = L2_CHUNK if use_qk_l2norm_in_kernel else L2_NONE
    launcher = _chunk_launch_any_head if _chunk_path_supported(q, v) else _recurrent_launch
    o, final_state = _GatedDelta.apply(launcher, q, k, v, g, beta, scale, initial_state, output_final_state,
                                       cu_seqlens, l2norm, True)
    return o.to(q.dtype), final_state


def fused_recurrent_gated_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                                     beta: torch.Tensor = None, scale: float = None,
                                     initial_state: torch.Tensor = None, output_final_state: bool = False,
                                     cu_seqlens: Optional[torch.LongTensor] = None,
                                     use_qk_l2norm_in_kernel: bool = False):
    """q, k [B,T,H,K]; v [B,T,HV,V]; g [B,T,HV]; beta [B,T,HV] or, one value per value column, [B,T,HV,V]
    (``gated_delta_rule_ori.py:444-448,515``); grouped value heads when HV > H. Returns (o [B,T,HV,V],
    final_state [N,HV,K,V] fp32 or None). See ``gated_delta_rule_ori.py:565-667``."""
    _check_varlen(q, initial_state, cu_seqlens)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    else:
        assert scale > 0, "scale must be positive"
    if beta is None:
        beta = torch.ones_like(g)
    _check_shapes(q, k, v, g, beta, "fused_recurrent_gated_delta_rule", headwise_beta_ok=True)
    l2norm = L2_RECURRENT if use_qk_l2norm_in_kernel else L2_NONE
    return _GatedDelta.apply(_recurrent_launch, q, k, v, g, beta, scale, initial_state, output_final_state,
                             cu_seqlens, l2norm, False)
