"""CPU oracle for the gradients of the gated delta rule (TEST INFRASTRUCTURE ONLY).

The reference obtains them with ``chunk_gated_delta_rule_bwd`` (``gated_delta_rule_ori.py:83-160``) and
``l2norm_bwd`` (``gated_delta_rule_ori.py:205-233``): the gradients of ``chunk_gated_delta_rule``'s outputs (o, final
state) with respect to q, k, v, g, beta and the initial state. Two independent statements, so that each pins the other:

* ``backward_autograd``  torch.autograd through a float64 token loop in the transition-matrix form of
                         ``recurrent.py:141-155`` (``forward_differentiable``; its forward values are pinned against
                         ``oracle.gated_delta.recurrent_delta`` and the C oracle);
* ``backward_manual``    a hand-derived reverse token loop in the delta form of ``gated_delta_rule_ori.py:430-453``
                         (no autograd anywhere), which also is fast enough for a few thousand tokens.

``tests/test_oracle_gdr_bwd.py`` pins both against central finite differences of the forward oracle and against the
closed form of a single token.

Shapes: q, k [B,T,H,K]; v, do [B,T,HV,V]; g, beta [B,T,HV]; h0, dht [N,HV,K,V]. All results float64.
"""
import torch

from .gated_delta import L2_CHUNK, L2_NONE, _segments, l2norm


def forward_differentiable(q, k, v, g, beta, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE):
    """float64 token loop, transition-matrix form; every input may require grad. Returns (o, final_state)."""
    if scale is None:
        scale = k.shape[-1] ** -0.5
    qn, kn = l2norm(q, l2), l2norm(k, l2)
    B, T, HV, V = v.shape
    K = k.shape[-1]
    rep = HV // q.shape[2]
    if rep > 1:
        qn, kn = qn.repeat_interleave(rep, dim=2), kn.repeat_interleave(rep, dim=2)
    eye = torch.eye(K, dtype=torch.float64)
    rows = [[None] * T for _ in range(B)]
    finals = []
    for n, (b, t0, t1) in enumerate(_segments(B, T, cu_seqlens)):
        S = torch.zeros(HV, K, V, dtype=torch.float64) if initial_state is None else initial_state[n]
        for t in range(t0, t1):
            kk = torch.einsum("hm,hn->hmn", kn[b, t], kn[b, t])
            gate = torch.exp(g[b, t])[:, None, None] * (eye - beta[b, t][:, None, None] * kk)
            S = gate @ S + beta[b, t][:, None, None] * torch.einsum("hk,hv->hkv", kn[b, t], v[b, t])
            rows[b][t] = scale * torch.einsum("hk,hkv->hv", qn[b, t], S)
        finals.append(S)
    zero = torch.zeros(HV, V, dtype=torch.float64)
    o = torch.stack([torch.stack([r if r is not None else zero for r in row]) for row in rows])
    return o, torch.stack(finals)


def _as64(x, grad=False):
    return None if x is None else x.detach().to("cpu", torch.float64).clone().requires_grad_(grad)


def backward_autograd(q, k, v, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE):
    """Returns (dq, dk, dv, dg, dbeta, dh0); dh0 is None without an initial state."""
    q, k, v, g, beta = (_as64(x, True) for x in (q, k, v, g, beta))
    h0 = _as64(initial_state, True)
    o, final = forward_differentiable(q, k, v, g, beta, scale, h0, cu_seqlens, l2)
    loss = (o * _as64(do)).sum()
    if dht is not None:
        loss = loss + (final * _as64(dht)).sum()
    wrt = [q, k, v, g, beta] + ([h0] if h0 is not None else [])
    grads = list(torch.autograd.grad(loss, wrt, allow_unused=True))
    grads = [torch.zeros_like(w) if gr is None else gr for gr, w in zip(grads, wrt)]
    return tuple(grads) + ((None,) if h0 is None else ())


def _l2norm_backward(x, dy, mode):
    """Gradient of ``oracle.gated_delta.l2norm`` written out: y = x c with c = (|x|^2 + eps)^(-1/2) gives
    dx = c (dy - y (y . dy)); c = 1 / (|x| + eps) gives dx = c dy - y (y . dy) / |x|."""
    if mode == L2_NONE:
        return dy
    ss = (x * x).sum(-1, keepdim=True)
    if mode == L2_CHUNK:
        c = 1.0 / torch.sqrt(ss + 1e-6)
        y = x * c
        return c * (dy - y * (y * dy).sum(-1, keepdim=True))
    n = torch.sqrt(ss)
    c = 1.0 / (n + 1e-6)
    y = x * c
    return c * dy - y * (y * dy).sum(-1, keepdim=True) / n


def backward_manual(q, k, v, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None, l2=L2_NONE):
    """Reverse token loop with the gradients written out (delta form: Sd = a S, w = Sd^T k, u = b (v - w),
    S' = Sd + k u^T, o = scale S'^T q). Returns (dq, dk, dv, dg, dbeta, dh0) like ``backward_autograd``."""
    q, k, v, g, beta, do = (_as64(x) for x in (q, k, v, g, beta, do))
    if scale is None:
        scale = k.shape[-1] ** -0.5
    B, T, HV, V = v.shape
    H, K = q.shape[2], q.shape[3]
    rep = HV // H
    qn = l2norm(q, l2).repeat_interleave(rep, dim=2)
    kn = l2norm(k, l2).repeat_interleave(rep, dim=2)
    dqn, dkn = torch.zeros_like(qn), torch.zeros_like(kn)
    dv, dg, db = torch.zeros_like(v), torch.zeros_like(g), torch.zeros_like(beta)
    segs = _segments(B, T, cu_seqlens)
    dh0 = None if initial_state is None else torch.zeros(len(segs), HV, K, V, dtype=torch.float64)
    for n, (b, t0, t1) in enumerate(segs):
        S = torch.zeros(HV, K, V, dtype=torch.float64) if initial_state is None else _as64(initial_state[n])
        decayed = []  # a_t S_{t-1} for every token
        for t in range(t0, t1):
            Sd = S * torch.exp(g[b, t])[:, None, None]
            decayed.append(Sd)
            u = beta[b, t][:, None] * (v[b, t] - torch.einsum("hkv,hk->hv", Sd, kn[b, t]))
            S = Sd + torch.einsum("hk,hv->hkv", kn[b, t], u)
        Hs = torch.zeros(HV, K, V, dtype=torch.float64) if dht is None else _as64(dht[n])
        for t in range(t1 - 1, t0 - 1, -1):
            Sd, kt, qt, bt = decayed[t - t0], kn[b, t], qn[b, t], beta[b, t][:, None]
            G = Hs + scale * torch.einsum("hk,hv->hkv", qt, do[b, t])
            w = torch.einsum("hkv,hk->hv", Sd, kt)
            u = bt * (v[b, t] - w)
            du = torch.einsum("hkv,hk->hv", G, kt)
            dv[b, t] = bt * du
            db[b, t] = (du * (v[b, t] - w)).sum(-1)
            dkn[b, t] = torch.einsum("hkv,hv->hk", G, u) - torch.einsum("hkv,hv->hk", Sd, bt * du)
            dqn[b, t] = scale * (torch.einsum("hkv,hv->hk", Sd, do[b, t]) + kt * (u * do[b, t]).sum(-1, keepdim=True))
            dSd = G - torch.einsum("hk,hv->hkv", kt, bt * du)
            dg[b, t] = (dSd * Sd).sum((-1, -2))
            Hs = dSd * torch.exp(g[b, t])[:, None, None]
        if dh0 is not None:
            dh0[n] = Hs
    fold = lambda x: x.reshape(B, T, H, rep, K).sum(3)  # grouped value heads share their q/k head
    return (_l2norm_backward(q, fold(dqn), l2), _l2norm_backward(k, fold(dkn), l2), dv, dg, db, dh0)
