"""Pins for the hierarchical gated-delta oracle: the level function against its closed form, the three statements
against each other, reduction to the plain gated delta rule when every level weight is one, and one-hot weights."""
import torch

from lampa_amd import synth
from oracle import gated_delta as og
from oracle import hgdn as oh


def _inputs(B=1, T=45, H=2, K=8, V=6, seed=0, L=None):
    q, k, v, g, beta = synth.gdr_inputs(B, T, H, K, V, torch.float32, seed, 1.0)
    L = L or oh.num_levels(T)
    gen = torch.Generator().manual_seed(seed + 7)
    lam = torch.rand(B, T, H, L, generator=gen) + 0.25
    return q, k, v, g, beta, lam


def test_level_function_is_highest_differing_bit():
    # base.py:41-46 peels the leading power of two off target and source until the source falls below it: that is
    # the position of the highest bit in which they differ, plus one
    for t in range(1, 300):
        for s in range(t):
            assert oh.level_index(t, s) == (t ^ s).bit_length()
    assert oh.num_levels(64) == 7 and oh.num_levels(65) == 8 and oh.num_levels(1) == 1


def test_levels_hold_fenwick_buckets():
    # after t+1 insertions level l > 0 of recurrent.py's cascade holds exactly the sources whose level is l
    L = 8
    for T in (1, 2, 3, 7, 8, 21, 64, 100):
        sets = [set() for _ in range(L)]
        for t in range(T):
            for lvl in range(L):
                if len(sets[lvl]) == 2 ** lvl:
                    sets[lvl + 1] |= sets[lvl]
                    sets[lvl] = set()
                elif len(sets[lvl]) < 2 ** lvl:
                    break
            sets[0] = {t}
            for lvl in range(1, L):
                assert sets[lvl] == {s for s in range(t) if oh.level_index(t, s) == lvl}


def test_three_statements_agree():
    q, k, v, g, beta, lam = _inputs()
    a = oh.recurrent_states(q, k, v, g, beta, lam)
    b = oh.quadratic_form(q, k, v, g, beta, lam)
    c = oh.recurrent_c(q, k, v, g, beta, lam).double()
    assert torch.allclose(a, b, atol=1e-10)
    assert torch.allclose(a, c, atol=2e-6)


def test_grouped_heads_and_batch():
    q, k, v, g, beta, lam = _inputs(B=2, T=33, H=1)
    gen = torch.Generator().manual_seed(5)
    v = torch.randn(2, 33, 2, 6, generator=gen)
    beta = torch.sigmoid(torch.randn(2, 33, 2, generator=gen))
    g = -torch.nn.functional.softplus(torch.randn(2, 33, 2, generator=gen))
    lam = torch.rand(2, 33, 2, oh.num_levels(33), generator=gen)
    a = oh.recurrent_states(q, k, v, g, beta, lam)
    c = oh.recurrent_c(q, k, v, g, beta, lam).double()
    assert torch.allclose(a, c, atol=2e-6)


def test_unit_weights_reduce_to_plain_gated_delta():
    # recurrent.py:96-100: the gate acts on every level alike, so the level states sum to the plain state
    q, k, v, g, beta, lam = _inputs(T=130)
    lam = torch.ones_like(lam)
    want, _ = og.recurrent_c(q, k, v, g, beta, l2=og.L2_CHUNK)
    got = oh.recurrent_c(q, k, v, g, beta, lam)
    assert torch.allclose(got, want, atol=2e-6)


def test_one_hot_weights_select_one_bucket():
    # lambda = e_l: token t sees only the sources of level l; summing over l gives the plain rule back (linearity)
    q, k, v, g, beta, lam = _inputs(T=40, H=1)
    L = lam.shape[-1]
    total = torch.zeros(1, 40, 1, 6)
    for lvl in range(L):
        one = torch.zeros_like(lam)
        one[..., lvl] = 1.0
        part = oh.recurrent_c(q, k, v, g, beta, one)
        if lvl == 0:  # only the token itself: o_t = scale * beta_t (q_t . k_t) v_t
            qn, kn = og.l2norm(q, og.L2_CHUNK), og.l2norm(k, og.L2_CHUNK)
            want = 8 ** -0.5 * beta[..., None] * (qn * kn).sum(-1, keepdim=True) * v
            assert torch.allclose(part, want, atol=2e-6)
        if lvl == L - 1:  # level L-1 = 6 covers sources below 32 for targets 32..39 only
            assert part[:, :32].abs().max() == 0 and part[:, 32:].abs().max() > 0
        total += part
    want, _ = og.recurrent_c(q, k, v, g, beta, l2=og.L2_CHUNK)
    assert torch.allclose(total, want, atol=1e-5)


def test_states_split_the_plain_state_and_continue_exactly():
    q, k, v, g, beta, lam = _inputs(B=2, T=77, H=2, L=9)
    o, S, counts = oh.recurrent_c_state(q, k, v, g, beta, lam)
    # token counts: level 0 holds the last token, level l > 0 is occupied (2^(l-1) tokens) iff bit l-1 of T-1 is set
    want = [1] + [(1 << (l - 1)) if ((76 >> (l - 1)) & 1) else 0 for l in range(1, 9)]
    assert counts.tolist() == want and sum(want) == 77
    assert all(S[..., l].abs().max() == 0 for l in range(9) if want[l] == 0)
    # the level states sum to the plain rule's state (recurrent.py:96-100)
    _, plain = og.recurrent_c(q, k, v, g, beta, l2=og.L2_CHUNK)
    assert torch.allclose(S.sum(-1), plain, atol=1e-5)
    # against the token loop with explicit level states of the first statement
    assert torch.allclose(o.double(), oh.recurrent_states(q, k, v, g, beta, lam), atol=2e-6)
    # stopping after 40 tokens and continuing from the returned state is the same as one run
    cut = lambda x, a, b: x[:, a:b]
    o1, S1, c1 = oh.recurrent_c_state(*(cut(x, 0, 40) for x in (q, k, v, g, beta, lam)))
    o2, S2, c2 = oh.recurrent_c_state(*(cut(x, 40, 77) for x in (q, k, v, g, beta, lam)), states=S1, counts=c1)
    assert torch.allclose(torch.cat([o1, o2], 1), o, atol=1e-5) and torch.allclose(S2, S, atol=1e-5)
    assert c2.tolist() == counts.tolist()
