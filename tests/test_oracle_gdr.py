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


# ---- the reference's safe_exp masking (positive g) -----------------------------------------------------------------
def test_masked_chunk_form_is_a_noop_for_nonpositive_g():
    q, k, v, g, beta = _inputs(B=1, T=150, H=2, K=8, V=6, g_scale=0.3)
    assert (g <= 0).all()
    o1, s1 = og.chunk_form(q, k, v, g, beta, chunk=64)
    o2, s2 = og.chunk_form(q, k, v, g, beta, chunk=64, masked=True)
    assert torch.equal(o1, o2) and torch.equal(s1, s2)


def test_positive_g_on_a_chunk_start_masks_nothing():
    # gamma_i - gamma_j (j < i in one chunk) and gamma_last - gamma_j are sums of g over tokens AFTER j, so the g of a
    # chunk's first token enters none of the masked ratios: with positive g only there, the masked chunk form must
    # equal the token loop, which applies e^g whatever its sign.
    q, k, v, g, beta = _inputs(B=1, T=200, H=2, K=8, V=6, g_scale=0.3)
    g = g.clone()
    g[:, 64] = 0.7
    g[:, 128] = 0.2
    o1, s1 = og.recurrent_delta(q, k, v, g, beta)
    o2, s2 = og.chunk_form(q, k, v, g, beta, chunk=64, masked=True)
    assert torch.allclose(o1, o2, atol=1e-10) and torch.allclose(s1, s2, atol=1e-10)
    g[:, 70] = 0.7  # ... and inside a chunk it does change the function
    o3, _ = og.chunk_form(q, k, v, g, beta, chunk=64, masked=True)
    o4, _ = og.recurrent_delta(q, k, v, g, beta)
    assert (o3 - o4).abs().max() > 1e-3


def test_large_positive_g_inside_first_chunk_restarts_the_sequence():
    # One g = +40 at token p of the first chunk (zero initial state, every other g <= 0 and small): every ratio that
    # spans p has a positive exponent and is masked, so tokens >= p neither see tokens < p (A and the attention
    # matrix are block diagonal) nor do tokens < p reach the final state (their e^{gamma_last - gamma_j} is masked):
    # outputs from p on and the final state equal those of the sequence that starts at p with its first g set to 0,
    # and outputs before p are untouched.
    T, p = 64, 23
    q, k, v, g, beta = _inputs(B=1, T=T, H=2, K=8, V=6, g_scale=0.05)
    g = g.clone()
    g[:, p] = 40.0
    o, s = og.chunk_form(q, k, v, g, beta, chunk=64, masked=True)
    g_tail = g[:, p:].clone()
    g_tail[:, 0] = 0.0
    # e^{gamma_i} still multiplies (q_i . S_chunk_start) -- S is zero here, so that term vanishes
    o_tail, s_tail = og.recurrent_delta(q[:, p:], k[:, p:], v[:, p:], g_tail, beta[:, p:])
    o_head, _ = og.recurrent_delta(q[:, :p], k[:, :p], v[:, :p], g[:, :p], beta[:, :p])
    assert torch.allclose(o[:, :p], o_head, atol=1e-10)
    assert torch.allclose(o[:, p:], o_tail, atol=1e-10)
    assert torch.allclose(s, s_tail, atol=1e-10)


def test_masked_chunk_form_against_scalar_loops():
    # The masked kernels restated with Python scalars, row by row (forward substitution instead of a matrix inverse):
    #   A_ij = beta_i (k_i.k_j) sexp(gam_i - gam_j), u_i = beta_i v_i - sum_j A_ij u_j, w_i = beta_i e^{gam_i} k_i - sum_j A_ij w_j
    #   vnew_i = u_i - w_i S, o_i = scale (e^{gam_i} q_i S + sum_{j<=i} (q_i.k_j) sexp(gam_i - gam_j) vnew_j)
    #   S' = e^{gam_last} S + sum_j sexp(gam_last - gam_j) k_j vnew_j^T
    import math

    def sexp(x):
        return math.exp(x) if x <= 0 else 0.0

    T, K, V, C = 21, 3, 2, 8
    q, k, v, g, beta = _inputs(B=1, T=T, H=1, K=K, V=V, g_scale=0.5, seed=5)
    g = g.clone()
    g[0, [3, 9, 10, 18], 0] = torch.tensor([0.4, 1.1, 0.3, 0.9])
    qq, kk, vv = q[0, :, 0].double().tolist(), k[0, :, 0].double().tolist(), v[0, :, 0].double().tolist()
    gg, bb = g[0, :, 0].double().tolist(), beta[0, :, 0].double().tolist()
    scale = 0.61
    S = [[0.0] * V for _ in range(K)]
    out = []
    dot = lambda a, b: sum(x * y for x, y in zip(a, b))
    for c0 in range(0, T, C):
        n = min(C, T - c0)
        gam, run = [], 0.0
        for i in range(n):
            run += gg[c0 + i]
            gam.append(run)
        u, w = [], []
        for i in range(n):
            ui = [bb[c0 + i] * x for x in vv[c0 + i]]
            wi = [bb[c0 + i] * math.exp(gam[i]) * x for x in kk[c0 + i]]
            for j in range(i):
                a = bb[c0 + i] * dot(kk[c0 + i], kk[c0 + j]) * sexp(gam[i] - gam[j])
                ui = [x - a * y for x, y in zip(ui, u[j])]
                wi = [x - a * y for x, y in zip(wi, w[j])]
            u.append(ui)
            w.append(wi)
        vnew = [[u[i][c] - sum(w[i][r] * S[r][c] for r in range(K)) for c in range(V)] for i in range(n)]
        for i in range(n):
            row = [math.exp(gam[i]) * sum(qq[c0 + i][r] * S[r][c] for r in range(K)) for c in range(V)]
            for j in range(i + 1):
                p = dot(qq[c0 + i], kk[c0 + j]) * sexp(gam[i] - gam[j])
                row = [x + p * y for x, y in zip(row, vnew[j])]
            out.append([scale * x for x in row])
        dec = math.exp(gam[-1])
        S = [[dec * S[r][c] + sum(sexp(gam[-1] - gam[j]) * kk[c0 + j][r] * vnew[j][c] for j in range(n))
              for c in range(V)] for r in range(K)]
    o, s = og.chunk_form(q, k, v, g, beta, scale=scale, chunk=C, masked=True)
    assert torch.allclose(o[0, :, 0], torch.tensor(out, dtype=torch.float64), atol=1e-10)
    assert torch.allclose(s[0, 0], torch.tensor(S, dtype=torch.float64), atol=1e-10)


def test_headwise_beta_of_the_token_loop():
    """One beta per value column (``gated_delta_rule_ori.py:444-448``). Two pins that do not retype the loop: a
    headwise beta that is constant over the columns is the scalar beta, bit for bit; and since the recurrence acts on
    every value column of the state independently, column j of the headwise result equals column j of a scalar-beta run
    with beta[..., j] -- which a wrong index into beta, v or the state would break."""
    gen = torch.Generator().manual_seed(3)
    B, T, H, HV, K, V = 2, 37, 2, 4, 8, 5
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    v = torch.randn(B, T, HV, V, generator=gen)
    g = -torch.rand(B, T, HV, generator=gen)
    beta = torch.rand(B, T, HV, generator=gen)
    h0 = torch.randn(B, HV, K, V, generator=gen)
    o, s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, l2=og.L2_RECURRENT)
    o2, s2 = og.recurrent_c(q, k, v, g, beta[..., None].expand(B, T, HV, V).contiguous(), initial_state=h0,
                            l2=og.L2_RECURRENT)
    assert torch.equal(o, o2) and torch.equal(s, s2)
    bw = torch.rand(B, T, HV, V, generator=gen)
    ow, sw = og.recurrent_c(q, k, v, g, bw, initial_state=h0, l2=og.L2_RECURRENT)
    assert not torch.equal(ow, o)
    for j in range(V):
        oj, sj = og.recurrent_c(q, k, v, g, bw[..., j].contiguous(), initial_state=h0, l2=og.L2_RECURRENT)
        assert torch.equal(ow[..., j], oj[..., j]) and torch.equal(sw[..., j], sj[..., j])
