"""Pins of the gradient oracle (CPU): the two statements against each other, against central finite differences of the
pinned forward oracle, and against the closed form of a single token."""
import pytest
import torch

from oracle import gated_delta as og
from oracle import gated_delta_bwd as ob


def _inputs(B, T, H, HV, K, V, seed, g_scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, K, generator=gen, dtype=torch.float64)
    k = torch.randn(B, T, H, K, generator=gen, dtype=torch.float64)
    k = k / k.norm(dim=-1, keepdim=True)
    v = torch.randn(B, T, HV, V, generator=gen, dtype=torch.float64)
    g = -g_scale * torch.nn.functional.softplus(torch.randn(B, T, HV, generator=gen, dtype=torch.float64))
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen, dtype=torch.float64))
    do = torch.randn(B, T, HV, V, generator=gen, dtype=torch.float64)
    return q, k, v, g, beta, do, gen


@pytest.mark.parametrize("l2", [og.L2_NONE, og.L2_CHUNK, og.L2_RECURRENT])
def test_differentiable_forward_is_the_forward_oracle(l2):
    q, k, v, g, beta, _, gen = _inputs(1, 37, 2, 4, 8, 12, 0)
    h0 = torch.randn(2, 4, 8, 12, generator=gen, dtype=torch.float64)
    cu = torch.tensor([0, 20, 37])
    o, s = ob.forward_differentiable(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu, l2=l2)
    wo, ws = og.recurrent_delta(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu, l2=l2)
    assert torch.allclose(o, wo, rtol=1e-12, atol=1e-12) and torch.allclose(s, ws, rtol=1e-12, atol=1e-12)
    co, cs = og.recurrent_c(q.float(), k.float(), v.float(), g.float(), beta.float(), initial_state=h0.float(),
                            cu_seqlens=cu, l2=l2)
    assert torch.allclose(o, co.double(), atol=2e-5) and torch.allclose(s, cs.double(), atol=2e-5)


@pytest.mark.parametrize("l2", [og.L2_NONE, og.L2_CHUNK, og.L2_RECURRENT])
@pytest.mark.parametrize("varlen", [False, True])
def test_manual_reverse_loop_matches_autograd(l2, varlen):
    B, T = (1, 45) if varlen else (2, 23)
    q, k, v, g, beta, do, gen = _inputs(B, T, 2, 4, 8, 6, 1)
    cu = torch.tensor([0, 0, 17, 45]) if varlen else None
    n = 3 if varlen else B
    h0 = torch.randn(n, 4, 8, 6, generator=gen, dtype=torch.float64)
    dht = torch.randn(n, 4, 8, 6, generator=gen, dtype=torch.float64)
    a = ob.backward_autograd(q, k, v, g, beta, do, dht, 0.3, h0, cu, l2)
    m = ob.backward_manual(q, k, v, g, beta, do, dht, 0.3, h0, cu, l2)
    for name, x, y in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0"), a, m):
        assert torch.allclose(x, y, rtol=1e-9, atol=1e-11), name
    a = ob.backward_autograd(q, k, v, g, beta, do, None, None, None, cu, l2)
    m = ob.backward_manual(q, k, v, g, beta, do, None, None, None, cu, l2)
    assert a[5] is None and m[5] is None
    for name, x, y in zip(("dq", "dk", "dv", "dg", "dbeta"), a, m):
        assert torch.allclose(x, y, rtol=1e-9, atol=1e-11), name


@pytest.mark.parametrize("l2", [og.L2_NONE, og.L2_CHUNK, og.L2_RECURRENT])
def test_gradients_match_central_differences_of_the_forward_oracle(l2):
    """The loss sum(o * do) + sum(final * dht) evaluated with ``oracle.gated_delta.recurrent_delta`` (which shares no
    code with the gradient oracle but the normalisation helper), perturbed entry by entry."""
    q, k, v, g, beta, do, gen = _inputs(1, 6, 1, 2, 4, 3, 2)
    k = k * 1.3  # not unit length: the normalisation's gradient must be non-trivial
    h0 = torch.randn(1, 2, 4, 3, generator=gen, dtype=torch.float64)
    dht = torch.randn(1, 2, 4, 3, generator=gen, dtype=torch.float64)

    def loss(q, k, v, g, beta, h0):
        o, s = og.recurrent_delta(q, k, v, g, beta, scale=0.7, initial_state=h0, l2=l2)
        return float((o * do).sum() + (s * dht).sum())

    args = [q, k, v, g, beta, h0]
    grads = ob.backward_manual(q, k, v, g, beta, do, dht, 0.7, h0, None, l2)
    eps = 1e-6
    for which, (x, gr) in enumerate(zip(args, grads)):
        flat = x.reshape(-1)
        for i in range(flat.numel()):
            keep = float(flat[i])
            flat[i] = keep + eps
            up = loss(*args)
            flat[i] = keep - eps
            down = loss(*args)
            flat[i] = keep
            fd = (up - down) / (2 * eps)
            assert abs(fd - float(gr.reshape(-1)[i])) < 1e-6 * max(1.0, abs(fd)), (which, i, fd, float(gr.reshape(-1)[i]))


def test_single_token_closed_form():
    """One token from a zero state: o = scale b (q . k) v, final = b k v^T, nothing depends on g."""
    q, k, v, g, beta, do, gen = _inputs(1, 1, 1, 1, 5, 4, 3)
    dht = torch.randn(1, 1, 5, 4, generator=gen, dtype=torch.float64)
    scale = 0.4
    for fn in (ob.backward_autograd, ob.backward_manual):
        dq, dk, dv, dg, db, dh0 = fn(q, k, v, g, beta, do, dht, scale)
        qq, kk, vv, dd, b, D = q[0, 0, 0], k[0, 0, 0], v[0, 0, 0], do[0, 0, 0], beta[0, 0, 0], dht[0, 0]
        assert dh0 is None and torch.allclose(dg, torch.zeros_like(dg), atol=1e-14)
        assert torch.allclose(dq[0, 0, 0], scale * b * kk * (vv @ dd))
        assert torch.allclose(dv[0, 0, 0], scale * b * (qq @ kk) * dd + b * (kk @ D))
        assert torch.allclose(db[0, 0, 0], scale * (qq @ kk) * (vv @ dd) + kk @ D @ vv)
        assert torch.allclose(dk[0, 0, 0], scale * b * qq * (vv @ dd) + b * (D @ vv))
