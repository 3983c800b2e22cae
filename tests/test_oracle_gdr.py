"""Pins for the gated-delta oracle: closed forms, invariants and agreement between its four independent
statements (delta form, transition-matrix form, chunk form, C restatement, quadratic form)."""
import torch

from lampa_amd import synth
from oracle import gated_delta as og


def _inputs(B=2, T=37, H=2, K=8, V=6, seed=0, g_scale=1.0, HV=None):
    q, k, v, g, beta = synth.gdr_inputs(B, T, H, K, V, torch.float32, seed, g_scale)
    if HV is not None and HV != H:
        gen = torch.Generator().manual_seed(seed + 100)
        v = torch.randn(B, T, HV, V, generator=gen)
        beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
        g = -torch.nn.functional.softplus(torch.randn(B, T, HV, generator=gen))
    return q, k, v, g, beta


def test_single_token_closed_form():
    # T = 1, S0 = 0: S = beta k v^T, o = scale * beta * (q.k) * v
    q, k, v, g, beta = (x.double() for x in _inputs(T=1))
    o, S = og.recurrent_delta(q, k, v, g, beta, scale=0.37)
    want = 0.37 * beta[..., None] * (q * k).sum(-1, keepdim=True) * v
    assert torch.allclose(o, want, atol=1e-12)
    assert torch.allclose(S, torch.einsum("bh,bhk,bhv->bhkv", beta[:, 0], k[:, 0], v[:, 0]), atol=1e-12)


def test_single_token_with_initial_state():
    # S = e^g (I - beta k k^T) S0 + beta k v^T
    q, k, v, g, beta = _inputs(B=1, T=1, H=1)
    S0 = torch.randn(1, 1, 8, 6, dtype=torch.float64)
    _, S = og.recurrent_delta(q, k, v, g, beta, initial_state=S0)
    kk = k[0, 0, 0].double()
    want = torch.exp(g[0, 0, 0].double()) * (torch.eye(8).double() - beta[0, 0, 0].double() * torch.outer(kk, kk)) @ S0[0, 0]
    want = want + beta[0, 0, 0].double() * torch.outer(kk, v[0, 0, 0].double())
    assert torch.allclose(S[0, 0], want, atol=1e-12)


def test_beta_zero_is_pure_decay():
    q, k, v, g, beta = _inputs(B=1, T=20, H=2)
    S0 = torch.randn(1, 2, 8, 6, dtype=torch.float64)
    o, S = og.recurrent_delta(q, k, v, g, torch.zeros_like(beta), initial_state=S0)
    assert torch.allclose(S, S0 * torch.exp(g.double().sum(1))[:, :, None, None], atol=1e-12)
    # outputs read the decayed state
    t = 7
    St = S0 * torch.exp(g[:, : t + 1].double().sum(1))[:, :, None, None]
    want = (8 ** -0.5) * torch.einsum("bhkv,bhk->bhv", St, q[:, t].double())
    assert torch.allclose(o[:, t], want, atol=1e-12)


def test_orthonormal_keys_recall_and_overwrite():
    # g = 0, beta = 1, orthonormal keys: S k_i = v_i exactly; writing a key twice keeps the last value.
    K, V = 8, 5
    keys = torch.linalg.qr(torch.randn(K, K, dtype=torch.float64))[0]
    vals = torch.randn(K + 1, V, dtype=torch.float64)
    k = torch.cat([keys, keys[:1]], 0)[None, :, None, :]  # key 0 written again at the end
    v = vals[None, :, None, :]
    g = torch.zeros(1, K + 1, 1)
    beta = torch.ones(1, K + 1, 1)
    _, S = og.recurrent_delta(k, k, v, g, beta, scale=1.0)
    recalled = torch.einsum("kv,nk->nv", S[0, 0], keys)
    assert torch.allclose(recalled[1:], vals[1:K], atol=1e-12)
    assert torch.allclose(recalled[0], vals[K], atol=1e-12)


def test_delta_matrix_chunk_quadratic_agree():
    q, k, v, g, beta = _inputs(B=2, T=50, H=2, K=8, V=6, g_scale=0.2)
    o1, s1 = og.recurrent_delta(q, k, v, g, beta)
    o2, s2 = og.recurrent_matrix(q, k, v, g, beta)
    assert torch.allclose(o1, o2, atol=1e-11) and torch.allclose(s1, s2, atol=1e-11)
    for chunk in (16, 32, 64):  # 50 is not a multiple of 16 or 32; 64 > T
        o3, s3 = og.chunk_form(q, k, v, g, beta, chunk=chunk)
        assert torch.allclose(o1, o3, atol=1e-10), chunk
        assert torch.allclose(s1, s3, atol=1e-10), chunk
    o4 = og.quadratic_form(q, k, v, g, beta)
    assert torch.allclose(o1, o4, atol=1e-10)


def test_initial_state_l2norm_varlen_gva():
    q, k, v, g, beta = _inputs(B=1, T=45, H=2, K=8, V=6, HV=4)
    q, k = q * 3.0, k * 0.5  # un-normalised so the l2norm matters
    cu = torch.tensor([0, 13, 13 + 20, 45])
    S0 = torch.randn(3, 4, 8, 6, dtype=torch.float64)
    for l2 in (og.L2_CHUNK, og.L2_RECURRENT):
        o1, s1 = og.recurrent_delta(q, k, v, g, beta, initial_state=S0, cu_seqlens=cu, l2=l2)
        o2, s2 = og.chunk_form(q, k, v, g, beta, initial_state=S0, cu_seqlens=cu, l2=l2, chunk=8)
        o3, s3 = og.recurrent_c(q, k, v, g, beta, initial_state=S0, cu_seqlens=cu, l2=l2)
        assert torch.allclose(o1, o2, atol=1e-10) and torch.allclose(s1, s2, atol=1e-10)
        assert torch.allclose(o1.float(), o3, atol=2e-6) and torch.allclose(s1.float(), s3, atol=2e-6)
    # a varlen run equals independent runs of its pieces
    oa, sa = og.recurrent_delta(q[:, 13:33], k[:, 13:33], v[:, 13:33], g[:, 13:33], beta[:, 13:33],
                                initial_state=S0[1:2], l2=og.L2_CHUNK)
    ob, sb = og.recurrent_delta(q, k, v, g, beta, initial_state=S0, cu_seqlens=cu, l2=og.L2_CHUNK)
    assert torch.allclose(oa[0], ob[0, 13:33], atol=1e-12) and torch.allclose(sa[0], sb[1], atol=1e-12)


def test_l2norm_against_library():
    x = torch.randn(5, 7, dtype=torch.float64)
    want = x * torch.rsqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    assert torch.allclose(og.l2norm(x, og.L2_CHUNK), want, atol=1e-14)
    assert torch.allclose(og.l2norm(x, og.L2_RECURRENT), x / (x.norm(dim=-1, keepdim=True) + 1e-6), atol=1e-14)


def test_stage_one_identities():
    torch.manual_seed(3)
    C, K, V = 24, 8, 6
    k = torch.nn.functional.normalize(torch.randn(C, K), dim=-1)
    v, g, beta = torch.randn(C, V), -torch.rand(C) * 0.3, torch.rand(C)
    gamma, A, Tm, W, U = og.chunk_stage_one(k, v, g, beta)
    eye = torch.eye(C, dtype=torch.float64)
    assert torch.allclose((eye + A) @ Tm, eye, atol=1e-12)
    assert torch.equal(A, torch.tril(A, -1))
    # forward substitution statement of U and W (hssd_minimal.py:236-246 style): u_i = beta_i v_i - sum_{j<i} A_ij u_j
    for i in range(C):
        assert torch.allclose(U[i], beta[i].double() * v[i].double() - A[i, :i] @ U[:i], atol=1e-12)
        assert torch.allclose(W[i], beta[i].double() * torch.exp(gamma[i]) * k[i].double() - A[i, :i] @ W[:i], atol=1e-12)
    # gamma is the per-chunk cumulative sum (cumsum.py:285-286)
    assert torch.allclose(gamma, torch.cumsum(g.double(), 0))


def test_c_oracle_fp32_and_fp64_on_longer_sequence():
    q, k, v, g, beta = _inputs(B=1, T=300, H=2, K=16, V=16, g_scale=0.05)
    o1, s1 = og.recurrent_delta(q, k, v, g, beta)
    o2, s2 = og.recurrent_c(q, k, v, g, beta)
    o3, s3 = og.recurrent_c(q, k, v, g, beta, dtype=torch.float32)
    assert torch.allclose(o1.float(), o2, atol=1e-6) and torch.allclose(s1.float(), s2, atol=1e-6)
    assert torch.allclose(o1.float(), o3, atol=1e-4) and torch.allclose(s1.float(), s3, atol=1e-4)
