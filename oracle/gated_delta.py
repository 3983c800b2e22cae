"""CPU oracle for the gated-delta-rule forward (TEST INFRASTRUCTURE ONLY).

Four independent statements of the same function, so that each pins the others:

* ``recurrent_delta``   token loop in the "delta" form of ``gated_delta_rule_ori.py:430-453``
                        (decay, d = beta (v - S^T k), S += k d^T, o = S^T q);
* ``recurrent_matrix``  token loop in the transition-matrix form of ``recurrent.py:134-155``
                        (S_t = a_t (I - b_t k_t k_t^T) S_{t-1} + b_t k_t v_t^T);
* ``chunk_form``        the chunkwise algorithm of ``gated_delta_rule_ori.py:29-80`` with its stages
                        ``cumsum.py:56-62``, ``chunk_scaled_dot_kkt.py:56-71``, ``solve_tril.py``,
                        ``wy_fast.py:168-189``, ``chunk_delta_h.py:109-189``, ``chunk_o.py:74-111``;
* ``recurrent_c``       the C restatement in ``gdr_oracle.c`` (fast enough for T = 60000).

``chunk_form(masked=True)`` adds the reference's ``safe_exp`` masking, which only matters for positive g; it is pinned in
``tests/test_oracle_gdr.py`` by the cases where the masking has a closed form (no effect for g <= 0; a positive g on the
first token of a chunk masks nothing; one large positive g inside the first chunk acts as a restart of the sequence
at that token) and by a scalar-loop restatement of the masked kernels.

Shapes follow the reference operators: q, k [B,T,H,K]; v [B,T,HV,V]; g, beta [B,T,HV]; states [N,HV,K,V].
"""
import ctypes

import numpy as np
import torch

from ._lib import lib, ptr

L2_NONE, L2_CHUNK, L2_RECURRENT = 0, 1, 2


def l2norm(x: torch.Tensor, mode: int) -> torch.Tensor:
    """``l2norm.py:100-101`` (mode 1: x / sqrt(sum x^2 + 1e-6)) and ``gated_delta_rule_ori.py:436-438``
    (mode 2: x / (sqrt(sum x^2) + 1e-6))."""
    if mode == L2_NONE:
        return x
    ss = (x * x).sum(-1, keepdim=True)
    if mode == L2_CHUNK:
        return x / torch.sqrt(ss + 1e-6)
    return x / (torch.sqrt(ss) + 1e-6)


def _segments(B, T, cu_seqlens):
    if cu_seqlens is None:
        return [(b, 0, T) for b in range(B)]
    cu = [int(c) for c in cu_seqlens]
    return [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def _prep(q, k, v, g, beta, scale, l2, dtype):
    q, k, v, g, beta = (x.detach().to("cpu", dtype) for x in (q, k, v, g, beta))
    if scale is None:
        scale = k.shape[-1] ** -0.5
    q, k = l2norm(q, l2), l2norm(k, l2)
    rep = v.shape[2] // q.shape[2]
    if rep > 1:
        q = q.repeat_interleave(rep, dim=2)
        k = k.repeat_interleave(rep, dim=2)
    return q, k, v, g, beta, scale


def recurrent_delta(q, k, v, g, beta, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE,
                    dtype=torch.float64):
    """Token loop, delta form. Returns (o [B,T,HV,V], final_state [N,HV,K,V]) in ``dtype``."""
    q, k, v, g, beta, scale = _prep(q, k, v, g, beta, scale, l2, dtype)
    B, T, HV, V = v.shape
    K = k.shape[-1]
    segs = _segments(B, T, cu_seqlens)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    final = torch.zeros(len(segs), HV, K, V, dtype=dtype)
    for n, (b, t0, t1) in enumerate(segs):
        S = torch.zeros(HV, K, V, dtype=dtype)
        if initial_state is not None:
            S = initial_state[n].detach().to("cpu", dtype).clone()
        for t in range(t0, t1):
            S = S * torch.exp(g[b, t])[:, None, None]
            d = beta[b, t][:, None] * (v[b, t] - torch.einsum("hkv,hk->hv", S, k[b, t]))
            S = S + torch.einsum("hk,hv->hkv", k[b, t], d)
            o[b, t] = torch.einsum("hkv,hk->hv", S, q[b, t] * scale)
        final[n] = S
    return o, final


def recurrent_matrix(q, k, v, g, beta, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE,
                     dtype=torch.float64):
    """Token loop, transition-matrix form of ``recurrent.py:141-155``."""
    q, k, v, g, beta, scale = _prep(q, k, v, g, beta, scale, l2, dtype)
    B, T, HV, V = v.shape
    K = k.shape[-1]
    segs = _segments(B, T, cu_seqlens)
    eye = torch.eye(K, dtype=dtype)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    final = torch.zeros(len(segs), HV, K, V, dtype=dtype)
    for n, (b, t0, t1) in enumerate(segs):
        S = torch.zeros(HV, K, V, dtype=dtype)
        if initial_state is not None:
            S = initial_state[n].detach().to("cpu", dtype).clone()
        for t in range(t0, t1):
            a = torch.exp(g[b, t])[:, None, None]
            bkk = beta[b, t][:, None, None] * torch.einsum("hm,hn->hmn", k[b, t], k[b, t])
            gate = a * (eye - bkk)
            value = beta[b, t][:, None, None] * torch.einsum("hk,hv->hkv", k[b, t], v[b, t])
            S = gate @ S + value
            o[b, t] = scale * torch.einsum("hk,hkv->hv", q[b, t], S)
        final[n] = S
    return o, final


def safe_exp(x: torch.Tensor) -> torch.Tensor:
    """``fla_op.py:27-29``: exp(x) where x <= 0, otherwise 0 (the exponent is replaced by -inf)."""
    return torch.exp(torch.where(x <= 0, x, torch.full_like(x, float("-inf"))))


def chunk_stage_one(k, v, g, beta, dtype=torch.float64, masked=False):
    """Intra-chunk quantities of ONE chunk of ONE head: k [C,K], v [C,V], g, beta [C] (already l2-normed k).

    Returns gamma (inclusive cumsum of g), A (strictly lower), Tm = (I + A)^-1, W, U. ``masked``: the decay ratio
    inside A goes through ``safe_exp`` as in ``chunk_scaled_dot_kkt.py:65-67`` (a no-op when g <= 0).
    """
    k, v, g, beta = (x.to(dtype) for x in (k, v, g, beta))
    C = k.shape[0]
    gamma = torch.cumsum(g, 0)
    diff = gamma[:, None] - gamma[None, :]
    lower = torch.tril(torch.ones(C, C, dtype=torch.bool), -1)
    ratio = safe_exp(diff) if masked else torch.exp(torch.where(lower, diff, 0.0))
    A = torch.where(lower, beta[:, None] * (k @ k.T) * ratio, 0.0)
    Tm = torch.linalg.solve_triangular(torch.eye(C, dtype=dtype) + A, torch.eye(C, dtype=dtype), upper=False)
    U = Tm @ (beta[:, None] * v)
    W = Tm @ ((beta * torch.exp(gamma))[:, None] * k)
    return gamma, A, Tm, W, U


def chunk_form(q, k, v, g, beta, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE, chunk=64,
               dtype=torch.float64, masked=False):
    """Chunkwise algorithm (chunks never straddle sequences, ``index.py:69-83``; a partial last chunk uses
    the gamma of its last valid row, ``chunk_delta_h.py:148``).

    ``masked=True`` is what the reference's kernels compute for ANY sign of g: the three decay RATIOS go through
    ``safe_exp`` -- inside A (``chunk_scaled_dot_kkt.py:67``), inside the intra-chunk attention matrix
    (``chunk_o.py:98``) and on the state update's e^{gamma_last - gamma_j} (``chunk_delta_h.py:152``) -- while
    e^{gamma_i} (``wy_fast.py:173``, ``chunk_o.py:97``) and e^{gamma_last} (``chunk_delta_h.py:153``) are plain
    exponentials. With g <= 0 no ratio's exponent is positive and both settings are the same function; with positive
    g the result depends on where the chunk boundaries fall (chunk = 64 in the reference)."""
    q, k, v, g, beta, scale = _prep(q, k, v, g, beta, scale, l2, dtype)
    B, T, HV, V = v.shape
    K = k.shape[-1]
    segs = _segments(B, T, cu_seqlens)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    final = torch.zeros(len(segs), HV, K, V, dtype=dtype)
    for n, (b, t0, t1) in enumerate(segs):
        for h in range(HV):
            S = torch.zeros(K, V, dtype=dtype)
            if initial_state is not None:
                S = initial_state[n, h].detach().to("cpu", dtype).clone()
            for c0 in range(t0, t1, chunk):
                c1 = min(c0 + chunk, t1)
                qc, kc, vc = q[b, c0:c1, h], k[b, c0:c1, h], v[b, c0:c1, h]
                gamma, _, _, W, U = chunk_stage_one(kc, vc, g[b, c0:c1, h], beta[b, c0:c1, h], dtype, masked)
                v_new = U - W @ S
                diff = gamma[:, None] - gamma[None, :]
                incl = torch.tril(torch.ones(c1 - c0, c1 - c0, dtype=torch.bool))
                ratio = safe_exp(diff) if masked else torch.exp(torch.where(incl, diff, 0.0))
                P = torch.where(incl, (qc @ kc.T) * ratio, 0.0)
                o[b, c0:c1, h] = scale * (torch.exp(gamma)[:, None] * (qc @ S) + P @ v_new)
                k_dec = kc * (safe_exp(gamma[-1] - gamma) if masked else torch.exp(gamma[-1] - gamma))[:, None]
                S = torch.exp(gamma[-1]) * S + k_dec.T @ v_new
            final[n, h] = S
    return o, final


def quadratic_form(q, k, v, g, beta, scale=None, l2=L2_NONE, dtype=torch.float64):
    """Materialised (whole sequence as one block) form with zero initial state, for short T
    (``base.py:384-420`` with all level weights equal to one): o = scale * tril(QK^T . Gamma) (I + A)^-1 (beta V)."""
    q, k, v, g, beta, scale = _prep(q, k, v, g, beta, scale, l2, dtype)
    B, T, HV, V = v.shape
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    for b in range(B):
        for h in range(HV):
            gamma, _, _, _, U = chunk_stage_one(k[b, :, h], v[b, :, h], g[b, :, h], beta[b, :, h], dtype)
            diff = gamma[:, None] - gamma[None, :]
            incl = torch.tril(torch.ones(T, T, dtype=torch.bool))
            P = torch.where(incl, (q[b, :, h] @ k[b, :, h].T) * torch.exp(torch.where(incl, diff, 0.0)), 0.0)
            o[b, :, h] = scale * (P @ U)
    return o


def recurrent_c(q, k, v, g, beta, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE,
                dtype=torch.float64):
    """``gdr_oracle.c`` through ctypes. Inputs are converted to fp32 arrays (exact for bf16/fp16/fp32 inputs);
    the state is carried in ``dtype`` (float64 or float32). Returns float32 tensors. ``beta`` is [B, T, HV] or, one
    value per value column, [B, T, HV, V] (``gated_delta_rule_ori.py:444-448``)."""
    B, T, H, K = q.shape
    HV, V = v.shape[2], v.shape[3]
    f = lambda x: np.ascontiguousarray(x.detach().to("cpu", torch.float32).numpy())
    qa, ka, va, ga, ba = f(q), f(k), f(v), f(g), f(beta)
    if scale is None:
        scale = K ** -0.5
    if cu_seqlens is None:
        cu = np.arange(B + 1, dtype=np.int64) * T
    else:
        assert B == 1
        cu = np.asarray([int(c) for c in cu_seqlens], dtype=np.int64)
    n_seq = len(cu) - 1
    h0 = None if initial_state is None else f(initial_state)
    o = np.empty((B, T, HV, V), np.float32)
    ht = np.empty((n_seq, HV, K, V), np.float32)
    fn = lib().oracle_gdr_recurrent_f64 if dtype == torch.float64 else lib().oracle_gdr_recurrent_f32
    fn(ptr(qa), ptr(ka), ptr(va), ptr(ga), ptr(ba), ptr(cu), n_seq, H, HV, K, V, ctypes.c_float(scale), l2,
       ptr(h0), ptr(o), ptr(ht), 1 if beta.dim() == 4 else 0)
    return torch.from_numpy(o), torch.from_numpy(ht)
