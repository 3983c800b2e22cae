"""GPU parity of the hierarchical gated-delta forward against the CPU oracle (fp64 token loop with level states).

Tolerances as for the plain chunk forward: bf16 / fp16 inputs with fp32 accumulation -- max-abs 2e-2 and
mean-relative 5e-3 on the outputs.
"""
import pytest
import torch

from lampa_amd import gated_delta as gd
from lampa_amd import hgdn
from lampa_amd import synth
from oracle import hgdn as oh

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 5e-3


def _errors(got, want):
    got, want = got.detach().float().cpu(), want.float()
    diff = (got - want).abs()
    return diff.max().item(), (diff.mean() / want.abs().mean().clamp_min(1e-12)).item()


def _inputs(B, T, H, K, V, dtype, seed, HV=None, g_scale=1.0, L=None):
    q, k, v, g, beta = synth.gdr_inputs(B, T, H, K, V, dtype, seed, g_scale)
    gen = torch.Generator().manual_seed(seed + 11)
    if HV is not None and HV != H:
        v = torch.randn(B, T, HV, V, generator=gen).to(dtype)
        beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
        g = -g_scale * torch.nn.functional.softplus(torch.randn(B, T, HV, generator=gen))
    L = L or hgdn.num_levels(T)
    lam = (torch.rand(B, T, v.shape[2], L, generator=gen) + 0.25).to(dtype)
    return q, k, v, g, beta, lam


def _run(device, q, k, v, g, beta, lam, cps=None):
    old = hgdn.CHUNKS_PER_SEGMENT
    hgdn.CHUNKS_PER_SEGMENT = cps
    try:
        o, state = hgdn.chunk_h_gated_delta_rule(*(x.to(device) for x in (q, k, v, g, lam, beta)),
                                                 use_qk_l2norm_in_kernel=True)
    finally:
        hgdn.CHUNKS_PER_SEGMENT = old
    assert state is None and o.dtype == v.dtype and o.shape == v.shape
    return o


def _want(q, k, v, g, beta, lam):
    # what reaches the kernel of the reference: lambda / scale in lambda's dtype, q * scale
    scale = q.shape[-1] ** -0.5
    return oh.recurrent_c(q, k, v, g, beta, lam / scale, scale=scale)


@pytest.mark.parametrize("T,cps", [(64, None), (256, None), (1024, None), (1024, 4), (4096, 8), (4096, 16), (2560, 8)])
def test_matches_oracle(device, T, cps):
    q, k, v, g, beta, lam = _inputs(1, T, 2, 64, 64, torch.bfloat16, seed=T)
    o = _run(device, q, k, v, g, beta, lam, cps)
    max_abs, mean_rel = _errors(o, _want(q, k, v, g, beta, lam))
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"T={T} cps={cps}: {max_abs:.3e} {mean_rel:.3e}"


def test_batch_grouped_heads_wide_values_fp16(device):
    q, k, v, g, beta, lam = _inputs(2, 1536, 2, 64, 128, torch.float16, seed=5, HV=4, g_scale=0.3, L=14)
    for cps in (None, 8):
        o = _run(device, q, k, v, g, beta, lam, cps)
        max_abs, mean_rel = _errors(o, _want(q, k, v, g, beta, lam))
        assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"cps={cps}: {max_abs:.3e} {mean_rel:.3e}"


def test_unit_weights_equal_plain_chunk_forward(device):
    # every level weighted by `scale` (lambda / scale = 1): the plain gated delta rule, at a size only the GPU walks
    T = 60032
    q, k, v, g, beta, _ = _inputs(1, T, 8, 64, 64, torch.bfloat16, seed=1, g_scale=0.1)
    lam = torch.full((1, T, 8, hgdn.num_levels(T)), 1.0, dtype=torch.bfloat16)
    o = _run(device, q, k, v, g, beta, lam)
    ref, _ = gd.chunk_gated_delta_rule(*(x.to(device) for x in (q, k, v, g, beta)), scale=1.0,
                                       use_qk_l2norm_in_kernel=True)
    max_abs, mean_rel = _errors(o, ref.cpu())
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"{max_abs:.3e} {mean_rel:.3e}"


def test_levels_are_linear_at_full_size(device):
    # o is linear in lambda: two disjoint level masks add up to the run with both
    T = 16384
    q, k, v, g, beta, lam = _inputs(1, T, 4, 64, 64, torch.bfloat16, seed=2, g_scale=0.1)
    lam = lam.float()
    low, high = lam.clone(), lam.clone()
    low[..., 9:] = 0
    high[..., :9] = 0
    o_all = _run(device, q, k, v, g, beta, lam.bfloat16()).float()
    o_sum = _run(device, q, k, v, g, beta, low.bfloat16()).float() + _run(device, q, k, v, g, beta, high.bfloat16()).float()
    max_abs, mean_rel = _errors(o_sum, o_all.cpu())
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"{max_abs:.3e} {mean_rel:.3e}"


def test_argument_checks(device):
    q, k, v, g, beta, lam = (x.to(device) for x in _inputs(1, 128, 2, 64, 64, torch.bfloat16, seed=0))
    with pytest.raises(AssertionError):
        hgdn.chunk_h_gated_delta_rule(q, k, v, g, lam, beta)  # the reference insists on the in-kernel l2norm
    with pytest.raises(AssertionError):
        hgdn.chunk_h_gated_delta_rule(q.float(), k.float(), v.float(), g, lam, beta, use_qk_l2norm_in_kernel=True)
    with pytest.raises(ValueError):
        hgdn.chunk_h_gated_delta_rule(q[:, :100], k[:, :100], v[:, :100], g[:, :100], lam[:, :100], beta[:, :100],
                                      use_qk_l2norm_in_kernel=True)
    with pytest.raises(ValueError):
        hgdn.chunk_h_gated_delta_rule(q, k, v, g, lam[..., :7], beta, use_qk_l2norm_in_kernel=True)
    with pytest.raises(NotImplementedError):  # an initial state without output_final_state (gated_delta_rule_apis.py:73-74)
        hgdn.chunk_h_gated_delta_rule(q, k, v, g, lam, beta, initial_state=object(), use_qk_l2norm_in_kernel=True)


# ------------------------------------------------------------------------------------ level states: prefill and step
def _state_errors(got: "hgdn.HState", want_states, want_counts):
    assert got.counts.tolist() == want_counts.tolist()
    return _errors(got.states, want_states)


@pytest.mark.parametrize("T,cps", [(64, None), (1024, None), (2560, 8), (1000, None), (4096 + 37, 16)])
def test_prefill_returns_the_level_states(device, T, cps):
    q, k, v, g, beta, lam = _inputs(2, T, 2, 64, 64, torch.bfloat16, seed=T + 1, g_scale=0.3, L=hgdn.num_levels(T) + 1)
    old = hgdn.CHUNKS_PER_SEGMENT
    hgdn.CHUNKS_PER_SEGMENT = cps
    try:
        o, st = hgdn.chunk_h_gated_delta_rule(*(x.to(device) for x in (q, k, v, g, lam, beta)), output_final_state=True,
                                              use_qk_l2norm_in_kernel=True)
    finally:
        hgdn.CHUNKS_PER_SEGMENT = old
    want_o, want_s, want_c = oh.recurrent_c_state(q, k, v, g, beta, lam / 0.125, scale=0.125)
    max_abs, mean_rel = _errors(o, want_o)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"o: {max_abs:.3e} {mean_rel:.3e}"
    max_abs, mean_rel = _state_errors(st, want_s, want_c)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"states: {max_abs:.3e} {mean_rel:.3e}"
    assert st.states.shape == (2, 2, 64, 64, lam.shape[-1]) and st.states.dtype == torch.float32


@pytest.mark.parametrize("K,V,T", [(16, 32, 640), (32, 32, 300), (48, 96, 256), (64, 40, 200)])
def test_small_heads_are_padded(device, K, V, T):
    # head sizes below the built ones (the reference layer's d_k = 16, d_v = 32): outputs alone (whole chunks only) and
    # the prefill with ragged T, its level states in the caller's K x V
    q, k, v, g, beta, lam = _inputs(2, T, 2, K, V, torch.bfloat16, seed=K + V, HV=4, g_scale=0.3, L=hgdn.num_levels(T) + 1)
    scale = K ** -0.5
    want_o, want_s, want_c = oh.recurrent_c_state(q, k, v, g, beta, lam / scale, scale=scale)
    d = [x.to(device) for x in (q, k, v, g, lam, beta)]
    o, st = hgdn.chunk_h_gated_delta_rule(*d, output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o.shape == v.shape and st.states.shape == (2, 4, K, V, lam.shape[-1])
    max_abs, mean_rel = _errors(o, want_o)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"o: {max_abs:.3e} {mean_rel:.3e}"
    max_abs, mean_rel = _state_errors(st, want_s, want_c)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"states: {max_abs:.3e} {mean_rel:.3e}"
    if T % 64 == 0:
        o2, none = hgdn.chunk_h_gated_delta_rule(*d, use_qk_l2norm_in_kernel=True)
        assert none is None and torch.equal(o2, o)


def test_steps_continue_a_prefill(device):
    # 256 tokens through the chunk kernels, then 70 single-token calls with the returned state: one run of 326 tokens
    T0, T1 = 256, 70
    q, k, v, g, beta, lam = _inputs(1, T0 + T1, 2, 64, 128, torch.bfloat16, seed=3, HV=4, g_scale=0.3, L=11)
    d = [x.to(device) for x in (q, k, v, g, lam, beta)]
    o0, st = hgdn.chunk_h_gated_delta_rule(*(x[:, :T0] for x in d), output_final_state=True, use_qk_l2norm_in_kernel=True)
    outs = [o0]
    for t in range(T0, T0 + T1):
        o_t, st2 = hgdn.chunk_h_gated_delta_rule(*(x[:, t:t + 1] for x in d), initial_state=st, output_final_state=True,
                                                 use_qk_l2norm_in_kernel=True)
        assert st2 is st and o_t.shape == (1, 1, 4, 128)
        outs.append(o_t)
    want_o, want_s, want_c = oh.recurrent_c_state(q, k, v, g, beta, lam / 0.125, scale=0.125)
    max_abs, mean_rel = _errors(torch.cat(outs, 1), want_o)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"o: {max_abs:.3e} {mean_rel:.3e}"
    max_abs, mean_rel = _state_errors(st, want_s, want_c)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"states: {max_abs:.3e} {mean_rel:.3e}"


def test_steps_from_an_empty_state_any_head_size(device):
    # fewer than 64 tokens: the prefill is the token-serial kernel alone (fp32 arithmetic on bf16 inputs)
    gen = torch.Generator().manual_seed(4)
    T, H, K, V, L = 45, 3, 32, 48, 8
    q, k, v = (torch.randn(2, T, H, d, generator=gen).bfloat16() for d in (K, K, V))
    g = -0.3 * torch.rand(2, T, H, generator=gen)
    beta = torch.rand(2, T, H, generator=gen)
    lam = torch.randn(2, T, H, L, generator=gen).bfloat16()
    o, st = hgdn.chunk_h_gated_delta_rule(*(x.to(device) for x in (q, k, v, g, lam, beta)), scale=0.25,
                                          output_final_state=True, use_qk_l2norm_in_kernel=True)
    want_o, want_s, want_c = oh.recurrent_c_state(q, k, v, g, beta, (lam / 0.25), scale=0.25)
    assert st.counts.tolist() == want_c.tolist()
    assert _errors(o, want_o)[0] <= 2e-2 and _errors(st.states, want_s)[0] <= 1e-4
    with pytest.raises(ValueError):  # one more level than the state has
        for _ in range(100):
            hgdn.chunk_h_gated_delta_rule(*(x[:, :1].to(device) for x in (q, k, v, g, lam, beta)), scale=0.25,
                                          initial_state=st, output_final_state=True, use_qk_l2norm_in_kernel=True)


@pytest.mark.parametrize("B,T,H,HV,K,V,L", [
    (2, 10, 2, 4, 24, 40, 9),    # LDS-staged kernel, pieces of 4 columns; K below the number of row groups
    (2, 10, 2, 4, 24, 30, 9),    # V not a multiple of 4: the register-resident kernel, partial 16-column tile
    (2, 6, 1, 2, 100, 8, 32),    # 32 levels, two row groups
    (130, 3, 2, 4, 64, 64, 12),  # a launch large enough for pieces of 8 columns
])
def test_step_entry_point_fp32_and_odd_sizes(device, B, T, H, HV, K, V, L):
    # the C entry point itself: fp32 tokens, weights taken as given (lam_div = 1), l2norm off; T tokens from an empty state
    import ctypes
    from lampa_amd import _capi
    from lampa_amd._capi import ptr
    gen = torch.Generator().manual_seed(11)
    q, k = (torch.randn(B, T, H, K, generator=gen) for _ in range(2))
    v = torch.randn(B, T, HV, V, generator=gen)
    g = -0.2 * torch.rand(B, T, HV, generator=gen)
    beta = torch.rand(B, T, HV, generator=gen)
    lam = torch.randn(B, T, HV, L, generator=gen)
    want_o, want_s, want_c = oh.recurrent_c_state(q, k, v, g, beta, lam, scale=0.3, l2=0)
    states = torch.zeros(B, HV, K, V, L, device=device)
    st = hgdn.HState(2, hgdn.HType.WEAK, hgdn.HStruct.GDELTA, (B, HV, K, V, L), torch.float32, device)
    outs = []
    lib = _capi.lib()
    for t in range(T):
        z = st.cascade_weak()
        args = [x[:, t].contiguous().to(device) for x in (q, k, v, g, beta, lam)]
        o = torch.empty(B, HV, V, device=device)
        rc = lib.lampa_hgdn_step(ptr(args[0]), ptr(args[1]), ptr(args[2]), ptr(args[3]), ptr(args[4]), ptr(args[5]), 2,
                                 1.0, ptr(states), ptr(o), B, H, HV, K, V, L, z, 2, 0.3, 0,
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0
        st._counts[0] += 1
        outs.append(o.cpu())
    assert st.counts.tolist() == want_c.tolist()
    # fp32 arithmetic against fp64: relative to the size of the values (the keys are not normalised here, so they grow)
    assert (torch.stack(outs, 1) - want_o).abs().max() <= 2e-5 * want_o.abs().max()
    assert (states.cpu() - want_s).abs().max() <= 2e-5 * want_s.abs().max()


@pytest.mark.parametrize("g_scale", [1.0, 0.003])
def test_full_length_prefill_matches_oracle(device, g_scale):
    # the benchmark's sequence length (938 chunks, 17 levels, split into segments by the default rule), two heads:
    # outputs, level states and counts against the fp64 token loop (a few seconds on one core)
    T = 60032
    q, k, v, g, beta, lam = _inputs(1, T, 2, 64, 64, torch.bfloat16, seed=3, g_scale=g_scale)
    o, st = hgdn.chunk_h_gated_delta_rule(*(x.to(device) for x in (q, k, v, g, lam, beta)), output_final_state=True,
                                          use_qk_l2norm_in_kernel=True)
    want_o, want_s, want_c = oh.recurrent_c_state(q, k, v, g, beta, lam / 0.125, scale=0.125)
    max_abs, mean_rel = _errors(o, want_o)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"o: {max_abs:.3e} {mean_rel:.3e}"
    max_abs, mean_rel = _state_errors(st, want_s, want_c)
    assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL, f"states: {max_abs:.3e} {mean_rel:.3e}"


def test_interleaved_calls_on_two_streams(device):
    # The launcher forks part of its work onto a helper stream; every caller stream has its own helper stream and
    # events, so calls issued alternately on two streams with nothing between them must each give what a call on its
    # own gives.
    cases = [_inputs(1, 4096, 2, 64, 64, torch.bfloat16, seed=70 + i) for i in range(2)]
    dev_cases = [tuple(x.to(device) for x in c) for c in cases]
    alone = []
    for q, k, v, g, beta, lam in dev_cases:
        o, _ = hgdn.chunk_h_gated_delta_rule(q, k, v, g, lam, beta, use_qk_l2norm_in_kernel=True)
        alone.append(o.clone())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=device), torch.cuda.Stream(device=device)]
    old = hgdn.CHUNKS_PER_SEGMENT
    hgdn.CHUNKS_PER_SEGMENT = 8  # several segments per sequence: the path that uses the helper stream
    try:
        ref = []
        for q, k, v, g, beta, lam in dev_cases:
            ref.append(hgdn.chunk_h_gated_delta_rule(q, k, v, g, lam, beta, use_qk_l2norm_in_kernel=True)[0].clone())
        torch.cuda.synchronize()
        outs = [[], []]
        for rep in range(4):
            for i in (0, 1):
                with torch.cuda.stream(streams[i]):
                    q, k, v, g, beta, lam = dev_cases[i]
                    outs[i].append(hgdn.chunk_h_gated_delta_rule(q, k, v, g, lam, beta, use_qk_l2norm_in_kernel=True)[0])
        torch.cuda.synchronize()
    finally:
        hgdn.CHUNKS_PER_SEGMENT = old
    for i in (0, 1):
        for o in outs[i]:
            assert torch.equal(o, ref[i])  # same kernels, same data: bit-identical whatever runs beside them
        max_abs, mean_rel = _errors(ref[i], alone[i].cpu())
        assert max_abs <= MAX_ABS and mean_rel <= MEAN_REL
