"""CPU oracle for the hierarchical (level-weighted) gated-delta forward (TEST INFRASTRUCTURE ONLY).

Three independent statements of ``chunk_h_gated_delta_rule`` (``gated_delta_rule_apis.py:21-134`` with
``HType.WEAK``, ``HStruct.GDELTA``, ``level_base=2``), whose specification is ``hattention_recurrent``
(``recurrent.py:169-216``):

* ``recurrent_states``  token loop over an explicit list of level states with the cascade of
                        ``recurrent.py:44-56`` and the insert of ``recurrent.py:84-97``;
* ``quadratic_form``    o_t = sum_s lambda_t[level(t, s)] * (q_t^T G_t ... G_{s+1} b_s k_s) v_s with the level of a
                        (target, source) pair from the recursion of ``base.py:41-46`` and lambda_t[0] on the diagonal
                        (``base.py:83-93``);
* ``recurrent_c``       the C restatement in ``hgdn_oracle.c`` (fast enough for tens of thousands of tokens).

q is l2-normalised and multiplied by ``scale``, k is l2-normalised (``kernel.py:100-101``); the caller of the
reference divides lambda by ``scale`` first (``gated_delta_rule_apis.py:68-70``), which the functions here leave to
their caller as well: they take the lambda that enters ``hattention_kernel``.

Shapes: q, k [B,T,H,K]; v [B,T,HV,V]; g, beta [B,T,HV]; lam [B,T,HV,L]; o [B,T,HV,V].
"""
import ctypes

import numpy as np
import torch

from ._lib import lib, ptr
from .gated_delta import L2_CHUNK, _prep


def level_index(t: int, s: int) -> int:
    """Level of source s < t for target t: the recursion of ``base.py:41-46`` (base 2), in integer arithmetic."""
    assert 0 <= s < t
    lg = t.bit_length() - 1  # floor(log2 t)
    v = 1 << lg
    if s < v:
        return lg + 1
    return level_index(t - v, s - v)


def num_levels(length: int) -> int:
    """``base.py:36-37``: ceil(log2(length)) + 1."""
    return (max(length, 1) - 1).bit_length() + 1


def recurrent_states(q, k, v, g, beta, lam, scale=None, l2=L2_CHUNK, dtype=torch.float64):
    """Token loop with explicit level states. Returns o [B,T,HV,V] in ``dtype``."""
    q, k, v, g, beta, scale = _prep(q, k, v, g, beta, scale, l2, dtype)
    lam = lam.detach().to("cpu", dtype)
    B, T, HV, V = v.shape
    K, L = k.shape[-1], lam.shape[-1]
    eye = torch.eye(K, dtype=dtype)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    for b in range(B):
        S = torch.zeros(L, HV, K, V, dtype=dtype)
        counts = [0] * L
        for t in range(T):
            for lvl in range(L):  # cascade_weak
                cap = 2 ** lvl
                if counts[lvl] == cap:
                    S[lvl + 1] = S[lvl + 1] + S[lvl]
                    counts[lvl + 1] += counts[lvl]
                    S[lvl] = 0
                    counts[lvl] = 0
                elif counts[lvl] < cap:
                    break
                else:
                    raise ValueError
            a = torch.exp(g[b, t])[:, None, None]
            bkk = beta[b, t][:, None, None] * torch.einsum("hm,hn->hmn", k[b, t], k[b, t])
            gate = a * (eye - bkk)
            S = torch.einsum("hmn,lhnv->lhmv", gate, S)
            S[0] = beta[b, t][:, None, None] * torch.einsum("hk,hv->hkv", k[b, t], v[b, t])
            counts[0] += 1
            Sl = torch.einsum("lhkv,hl->hkv", S, lam[b, t])
            o[b, t] = torch.einsum("hk,hkv->hv", q[b, t] * scale, Sl)
    return o


def quadratic_form(q, k, v, g, beta, lam, scale=None, l2=L2_CHUNK, dtype=torch.float64):
    """Materialised form for short T: the attention-like matrix of the gated delta rule, entry by entry from the
    products of the transition matrices, masked with lambda by level."""
    q, k, v, g, beta, scale = _prep(q, k, v, g, beta, scale, l2, dtype)
    lam = lam.detach().to("cpu", dtype)
    B, T, HV, V = v.shape
    K = k.shape[-1]
    eye = torch.eye(K, dtype=dtype)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    for b in range(B):
        for h in range(HV):
            G = [torch.exp(g[b, t, h]) * (eye - beta[b, t, h] * torch.outer(k[b, t, h], k[b, t, h])) for t in range(T)]
            for t in range(T):
                prod = eye.clone()  # G_t ... G_{s+1}
                for s in range(t, -1, -1):
                    w = lam[b, t, h, 0] if s == t else lam[b, t, h, level_index(t, s)]
                    a_ts = scale * (q[b, t, h] @ prod @ k[b, s, h]) * beta[b, s, h]
                    o[b, t, h] += w * a_ts * v[b, s, h]
                    prod = prod @ G[s]
    return o


def recurrent_c(q, k, v, g, beta, lam, scale=None, l2=L2_CHUNK):
    """``hgdn_oracle.c`` through ctypes (fp64 states). Inputs are converted to fp32 arrays (exact for bf16 / fp16 /
    fp32 inputs). Returns a float32 tensor."""
    B, T, H, K = q.shape
    HV, V, L = v.shape[2], v.shape[3], lam.shape[-1]
    f = lambda x: np.ascontiguousarray(x.detach().to("cpu", torch.float32).numpy())
    qa, ka, va, ga, ba, la = f(q), f(k), f(v), f(g), f(beta), f(lam)
    if scale is None:
        scale = K ** -0.5
    cu = np.arange(B + 1, dtype=np.int64) * T
    o = np.empty((B, T, HV, V), np.float32)
    lib().oracle_hgdn_recurrent_f64(ptr(qa), ptr(ka), ptr(va), ptr(ga), ptr(ba), ptr(la), ptr(cu), B, H, HV, K, V, L,
                                    ctypes.c_float(scale), l2, ptr(o))
    return torch.from_numpy(o)


def recurrent_c_state(q, k, v, g, beta, lam, scale=None, l2=L2_CHUNK, states=None, counts=None):
    """As ``recurrent_c``, carrying the level states: ``states`` [B,HV,K,V,L] and ``counts`` [L] (the ``HState`` of
    ``recurrent.py:9-40``) enter when given (zero otherwise); returns ``(o, states, counts)`` after the last token."""
    B, T, H, K = q.shape
    HV, V, L = v.shape[2], v.shape[3], lam.shape[-1]
    f = lambda x: np.ascontiguousarray(x.detach().to("cpu", torch.float32).numpy())
    qa, ka, va, ga, ba, la = f(q), f(k), f(v), f(g), f(beta), f(lam)
    if scale is None:
        scale = K ** -0.5
    cu = np.arange(B + 1, dtype=np.int64) * T
    o = np.empty((B, T, HV, V), np.float32)
    s_in = None if states is None else f(states)
    c_in = None if counts is None else np.ascontiguousarray(np.asarray(counts, dtype=np.int32))
    s_out = np.empty((B, HV, K, V, L), np.float32)
    c_out = np.empty((L,), np.int32)
    lib().oracle_hgdn_recurrent_state_f64(ptr(qa), ptr(ka), ptr(va), ptr(ga), ptr(ba), ptr(la), ptr(cu), B, H, HV, K, V,
                                          L, ctypes.c_float(scale), l2, ptr(s_in), ptr(c_in), ptr(o), ptr(s_out),
                                          ptr(c_out))
    return torch.from_numpy(o), torch.from_numpy(s_out), torch.from_numpy(c_out)
