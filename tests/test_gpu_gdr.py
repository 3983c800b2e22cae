"""GPU parity of the gated-delta operators against the CPU oracle.

Tolerances (from the benchmark contract): bf16 inputs with fp32 accumulation -- max-abs 2e-2 and mean-relative
5e-3 on outputs and final states; fp32 mode -- 1e-4.
"""
import numpy as np
import pytest
import torch

from lampa_amd import gated_delta as gd
from lampa_amd import synth
from oracle import gated_delta as og

pytestmark = pytest.mark.gpu

BF16_MAX_ABS, BF16_MEAN_REL, FP32_TOL = 2e-2, 5e-3, 1e-4


def _errors(got, want):
    got, want = got.detach().float().cpu(), want.float()
    diff = (got - want).abs()
    return diff.max().item(), (diff.mean() / want.abs().mean().clamp_min(1e-12)).item()


def _assert_bf16_close(got, want, what):
    max_abs, mean_rel = _errors(got, want)
    assert max_abs <= BF16_MAX_ABS and mean_rel <= BF16_MEAN_REL, f"{what}: max_abs={max_abs:.3e} mean_rel={mean_rel:.3e}"


def _to(dev, *xs):
    return [None if x is None else x.to(dev) for x in xs]


# ------------------------------------------------------------------------------------------------- token-serial
@pytest.mark.parametrize("K,V,T", [(32, 32, 700), (64, 64, 300), (128, 128, 130), (16, 32, 257), (20, 40, 131),
                                   (30, 70, 90), (8, 8, 65), (100, 24, 64)])
def test_recurrent_fp32_matches_oracle(device, K, V, T):
    # K a multiple of 4: the split-wave kernel (groups of 64 / 32 / 16 tokens: T covers whole groups, a partial one, odd
    # counts); K = 30: the lane-per-column kernel
    q, k, v, g, beta = synth.gdr_inputs(2, T, 3, K, V, torch.float32, seed=K + T, g_scale=0.1)
    h0 = torch.randn(2, 3, K, V, generator=torch.Generator().manual_seed(1))
    for l2, flag in ((og.L2_NONE, False), (og.L2_RECURRENT, True)):
        want_o, want_s = og.recurrent_c(q * 2, k, v, g, beta, initial_state=h0, l2=l2)
        o, s = gd.fused_recurrent_gated_delta_rule(*_to(device, q * 2, k, v, g, beta), initial_state=h0.to(device),
                                                   output_final_state=True, use_qk_l2norm_in_kernel=flag)
        assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL


@pytest.mark.parametrize("dtype,K,V,T", [(torch.float32, 32, 48, 300), (torch.bfloat16, 64, 64, 200),
                                         (torch.float32, 30, 70, 90), (torch.float16, 128, 100, 70)])
def test_recurrent_headwise_beta(device, dtype, K, V, T):
    # one beta per value column, [B, T, HV, V] (gated_delta_rule_ori.py:444-448,515): against the C token loop with the
    # same option; a headwise beta that is constant over the columns must give the bits of the scalar call; varlen with
    # grouped value heads
    gen = torch.Generator().manual_seed(K + V)
    q, k, v, g, beta = synth.gdr_inputs(2, T, 2, K, V, dtype, seed=T, g_scale=0.2)
    v = torch.randn(2, T, 4, V, generator=gen).to(dtype)
    g = -0.2 * torch.rand(2, T, 4, generator=gen)
    bw = torch.rand(2, T, 4, V, generator=gen)
    h0 = torch.randn(2, 4, K, V, generator=gen) * 0.3
    want_o, want_s = og.recurrent_c(q, k, v, g, bw, initial_state=h0, l2=og.L2_RECURRENT)
    o, s = gd.fused_recurrent_gated_delta_rule(*_to(device, q, k, v, g, bw), initial_state=h0.to(device),
                                               output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o.shape == v.shape and o.dtype == dtype
    if dtype == torch.float32:
        assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL
    else:
        _assert_bf16_close(o, want_o, "headwise o")
        assert _errors(s, want_s)[0] <= FP32_TOL * 10
    gd_args = _to(device, q, k, v, g)
    b3 = torch.rand(2, T, 4, generator=gen)
    old = gd.SEGMENT_MIN_TOKENS
    gd.SEGMENT_MIN_TOKENS = None  # the scalar call on the plain token loop as well
    try:
        o3, s3 = gd.fused_recurrent_gated_delta_rule(*gd_args, b3.to(device), output_final_state=True)
    finally:
        gd.SEGMENT_MIN_TOKENS = old
    o4, s4 = gd.fused_recurrent_gated_delta_rule(*gd_args, b3[..., None].expand(2, T, 4, V).contiguous().to(device),
                                                 output_final_state=True)
    if K % 4:  # both calls ran on the lane-per-column kernel: the same bits
        assert torch.equal(o3, o4) and torch.equal(s3, s4)
    else:      # the scalar call ran on the split-wave kernel: fp32 rounding apart
        assert _errors(o4, o3.float().cpu())[0] <= (FP32_TOL if dtype == torch.float32 else BF16_MAX_ABS)
    cu = torch.tensor([0, 17, 17, T + 5, 2 * T])
    flat = [x.reshape(1, 2 * T, *x.shape[2:]) for x in (q, k, v, g, bw)]
    wo, ws = og.recurrent_c(*flat, cu_seqlens=cu)
    o5, s5 = gd.fused_recurrent_gated_delta_rule(*_to(device, *flat), output_final_state=True, cu_seqlens=cu.to(device))
    tol = FP32_TOL if dtype == torch.float32 else BF16_MAX_ABS
    assert _errors(o5, wo)[0] <= tol and _errors(s5, ws)[0] <= tol


def test_config0_fp32_plumbing(device):
    # B=1, H=4, T=8192, d_k=d_v=32, fp32, seed 0, zero initial state
    q, k, v, g, beta = synth.gdr_inputs(1, 8192, 4, 32, 32, torch.float32, seed=0)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta)
    o, s = gd.fused_recurrent_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True)
    assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL
    o2, s2 = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True, allow_fp32=True)
    assert _errors(o2, want_o)[0] <= FP32_TOL and _errors(s2, want_s)[0] <= FP32_TOL
    with pytest.raises(AssertionError):
        gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta))


def test_recurrent_many_short_sequences_both_kernels(device):
    # 700 sequences x 4 value heads of 0 .. 9 tokens: more waves than the split-wave kernel takes (the lane-per-column
    # kernel runs); the first 100 sequences alone go to the split-wave kernel; same oracle
    gen = torch.Generator().manual_seed(8)
    lens = torch.randint(0, 10, (700,), generator=gen)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(lens, 0)])
    T, H, HV, K, V = int(cu[-1]), 2, 4, 32, 32
    q, k = (torch.randn(1, T, H, K, generator=gen) for _ in range(2))
    v = torch.randn(1, T, HV, V, generator=gen)
    g = -torch.rand(1, T, HV, generator=gen) * 0.3
    beta = torch.rand(1, T, HV, generator=gen)
    h0 = torch.randn(700, HV, K, V, generator=gen)
    for n in (700, 100):
        Tn = int(cu[n])
        args = [x[:, :Tn] for x in (q, k, v, g, beta)]
        want_o, want_s = og.recurrent_c(*args, initial_state=h0[:n], cu_seqlens=cu[:n + 1], l2=og.L2_RECURRENT)
        o, s = gd.fused_recurrent_gated_delta_rule(*_to(device, *args), initial_state=h0[:n].to(device),
                                                   output_final_state=True, cu_seqlens=cu[:n + 1].to(device),
                                                   use_qk_l2norm_in_kernel=True)
        assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL, n


@pytest.mark.parametrize("K,V", [(16, 32), (64, 64), (128, 16)])
def test_recurrent_strong_mixed_and_positive_decay(device, K, V):
    """The split kernel keeps the state divided by the decay accumulated inside a group of tokens and falls back to the
    plain form for a group whose decay would leave the fp32 range: runs of g = -9 per token (e^-144 over 16 tokens)
    between runs of weak decay, a stretch of g = -100 (e^g = 0 in fp32: the state is wiped) and a few positive g, with
    and without segments."""
    gen = torch.Generator().manual_seed(K)
    T, H = 1100, 2
    q, k = (torch.randn(1, T, H, K, generator=gen) for _ in range(2))
    v = torch.randn(1, T, H, V, generator=gen)
    g = -0.05 * torch.rand(1, T, H, generator=gen)
    g[:, 100:180] = -9.0
    g[:, 300:303] = -100.0
    g[:, 400:520:7] = 0.3
    g[:, 700:900, 1] = -4.0 * torch.rand(200, generator=gen)
    beta = torch.rand(1, T, H, generator=gen)
    h0 = torch.randn(1, H, K, V, generator=gen)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, l2=og.L2_RECURRENT)
    for seg_min in (512, None):
        old = gd.SEGMENT_MIN_TOKENS
        gd.SEGMENT_MIN_TOKENS = seg_min
        try:
            o, s = gd.fused_recurrent_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                                       output_final_state=True, use_qk_l2norm_in_kernel=True)
        finally:
            gd.SEGMENT_MIN_TOKENS = old
        assert torch.isfinite(o).all() and torch.isfinite(s).all()
        assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL, seg_min


def test_recurrent_segments_scanned_in_groups_unbalanced_sequences(device):
    """Four sequences of very different lengths (one empty, one of two segments) cut into 32-token segments: 129 segments,
    so the scan over them runs as groups' maps -> groups' start states -> segments inside the groups, with groups that
    are full, partial, single and absent."""
    gen = torch.Generator().manual_seed(31)
    lens = [3000, 0, 40, 1000]
    cu_host = [0] + list(np.cumsum(lens))
    T, H, HV, K, V = sum(lens), 1, 2, 32, 48
    q, k = (torch.randn(1, T, H, K, generator=gen) for _ in range(2))
    v = torch.randn(1, T, HV, V, generator=gen)
    g = -torch.rand(1, T, HV, generator=gen) * 0.05
    beta = torch.rand(1, T, HV, generator=gen)
    h0 = torch.randn(4, HV, K, V, generator=gen)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=torch.tensor(cu_host),
                                    l2=og.L2_RECURRENT)
    o, s = gd._recurrent_segmented_launch(*_to(device, q, k, v, g, beta), K ** -0.5, h0.to(device), True,
                                          [int(c) for c in cu_host], 32, gd.L2_RECURRENT)
    assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_recurrent_long_sequences_run_as_segments(device, dtype):
    # a few long sequences (one of them empty, one shorter than a segment) are cut into segments that run in parallel;
    # against the oracle and against the same call with the segments switched off
    gen = torch.Generator().manual_seed(21)
    lens = [1500, 0, 77, 2049]
    cu = torch.tensor([0] + list(np.cumsum(lens)))
    T, H, HV, K, V = sum(lens), 1, 2, 32, 64
    q, k = (torch.randn(1, T, H, K, generator=gen).to(dtype) for _ in range(2))
    v = torch.randn(1, T, HV, V, generator=gen).to(dtype)
    g = -torch.rand(1, T, HV, generator=gen) * 0.1
    beta = torch.rand(1, T, HV, generator=gen)
    h0 = torch.randn(4, HV, K, V, generator=gen)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu, l2=og.L2_RECURRENT)
    run = lambda: gd.fused_recurrent_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                                      output_final_state=True, cu_seqlens=cu.to(device),
                                                      use_qk_l2norm_in_kernel=True)
    o, s = run()
    old = gd.SEGMENT_MIN_TOKENS
    gd.SEGMENT_MIN_TOKENS = None
    try:
        o1, s1 = run()
    finally:
        gd.SEGMENT_MIN_TOKENS = old
    tol = FP32_TOL if dtype == torch.float32 else 2e-2
    assert _errors(o, want_o)[0] <= tol and _errors(s, want_s)[0] <= 10 * FP32_TOL
    assert _errors(o1, want_o)[0] <= tol and _errors(s1, want_s)[0] <= 10 * FP32_TOL
    assert _errors(o, o1.float().cpu())[0] <= tol and _errors(s, s1.cpu())[0] <= 10 * FP32_TOL


def test_recurrent_varlen_gva_bf16(device):
    gen = torch.Generator().manual_seed(3)
    T, H, HV, K, V = 500, 2, 4, 64, 64
    q = torch.randn(1, T, H, K, generator=gen).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(1, T, H, K, generator=gen), dim=-1).bfloat16()
    v = torch.randn(1, T, HV, V, generator=gen).bfloat16()
    g = -torch.rand(1, T, HV, generator=gen) * 0.2
    beta = torch.rand(1, T, HV, generator=gen)
    cu = torch.tensor([0, 100, 101, 333, 500])
    h0 = torch.randn(4, HV, K, V, generator=gen)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu, l2=og.L2_RECURRENT)
    o, s = gd.fused_recurrent_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                               output_final_state=True, cu_seqlens=cu.to(device),
                                               use_qk_l2norm_in_kernel=True)
    _assert_bf16_close(o, want_o, "o")
    assert _errors(s, want_s)[0] <= 1e-3
    # beta=None means all ones
    o1, _ = gd.fused_recurrent_gated_delta_rule(*_to(device, q[:, :, :, :], k, v[:, :, :2], g[:, :, :2]))
    w1, _ = og.recurrent_c(q, k, v[:, :, :2], g[:, :, :2], torch.ones(1, T, 2))
    _assert_bf16_close(o1, w1, "beta none")


# ----------------------------------------------------------------------------------------------------- chunk path
@pytest.mark.parametrize("T", [1, 64, 65, 200, 1000])
@pytest.mark.parametrize("g_scale", [1.0, 0.02])
def test_chunk_bf16_matches_oracle(device, T, g_scale):
    q, k, v, g, beta = synth.gdr_inputs(2, T, 2, 64, 64, torch.bfloat16, seed=T, g_scale=g_scale)
    h0 = 0.5 * torch.randn(2, 2, 64, 64, generator=torch.Generator().manual_seed(2))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                     output_final_state=True)
    assert o.dtype == torch.bfloat16 and s.dtype == torch.float32 and s.shape == (2, 2, 64, 64)
    _assert_bf16_close(o, want_o, f"o T={T}")
    _assert_bf16_close(s, want_s, f"state T={T}")


@pytest.fixture
def output_pass_form():
    """Lets a test force one form of the output pass; the default choice is restored afterwards."""
    yield gd.output_pass_config
    gd.output_pass_config(1)


@pytest.mark.parametrize("narrow", [0, 2])
@pytest.mark.parametrize("K,V,dtype", [(64, 64, torch.bfloat16), (128, 128, torch.bfloat16), (64, 128, torch.float16),
                                       (128, 64, torch.bfloat16)])
def test_both_forms_of_the_output_pass(device, K, V, dtype, narrow, output_pass_form, monkeypatch):
    """The output pass with 32 value columns per recurrence wave and with 16 (narrow waves, 16x16x32 MFMA), each forced
    at every head size it is built for: packed sequences with partial chunks and an empty one, initial states, the norm in
    the kernel, weak decay, one chunk per segment (so that at K = 64 the walk over the group composites runs inside the
    pass) -- against the token loop."""
    output_pass_form(narrow)
    monkeypatch.setattr(gd, "CHUNKS_PER_SEGMENT", 1)
    lens = [64 * 27 - 5, 0, 130, 64]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int64)
    total = int(cu[-1])
    q, k, v, g, beta = synth.gdr_inputs(1, total, 2, K, V, dtype, seed=K + V + narrow, g_scale=0.003)
    h0 = 0.5 * torch.randn(len(lens), 2, K, V, generator=torch.Generator().manual_seed(5))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu, l2=og.L2_CHUNK)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device), output_final_state=True,
                                     cu_seqlens=cu.to(device), use_qk_l2norm_in_kernel=True)
    _assert_bf16_close(o, want_o, f"o narrow={narrow}")
    _assert_bf16_close(s, want_s, f"state narrow={narrow}")


@pytest.mark.parametrize("cps", [1, 3, 16])
def test_chunk_segment_split_is_invisible(device, cps, monkeypatch):
    monkeypatch.setattr(gd, "CHUNKS_PER_SEGMENT", cps)
    q, k, v, g, beta = synth.gdr_inputs(1, 64 * 13 + 7, 2, 64, 64, torch.bfloat16, seed=9, g_scale=0.01)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True)
    _assert_bf16_close(o, want_o, f"o cps={cps}")
    _assert_bf16_close(s, want_s, f"state cps={cps}")


@pytest.mark.parametrize("K,V,n_chunks", [(64, 64, 24), (64, 64, 27), (64, 64, 63), (128, 128, 41), (64, 128, 33)])
def test_two_level_scan_over_many_segments(device, K, V, n_chunks, monkeypatch):
    """One chunk per segment makes 24 or more segments per sequence: the scan then runs as group composites, a scan
    over the groups and a scan inside the groups (groups of 8; 27 / 41 / 33 leave a ragged last group); at K = 64 the
    output pass does the last two itself, at K = 128 a leaf launch does. Weak decay, so
    that the state really travels through all the levels; initial state and final state included."""
    monkeypatch.setattr(gd, "CHUNKS_PER_SEGMENT", 1)
    T = 64 * n_chunks - 5
    q, k, v, g, beta = synth.gdr_inputs(1, T, 2, K, V, torch.bfloat16, seed=n_chunks, g_scale=0.003)
    h0 = 0.5 * torch.randn(1, 2, K, V, generator=torch.Generator().manual_seed(3))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, l2=og.L2_CHUNK)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device), output_final_state=True,
                                     use_qk_l2norm_in_kernel=True)
    _assert_bf16_close(o, want_o, f"o chunks={n_chunks}")
    _assert_bf16_close(s, want_s, f"state chunks={n_chunks}")


def test_two_level_scan_varlen_mixed_lengths(device, monkeypatch):
    """Packed sequences of very different lengths: the long ones take the grouped scan, the short and the empty one
    ride along in the same launches (their groups beyond the first do nothing)."""
    monkeypatch.setattr(gd, "CHUNKS_PER_SEGMENT", 1)
    lens = [64 * 30 + 1, 5, 0, 64 * 9, 64 * 26 - 1]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.long)
    T = int(cu[-1])
    q, k, v, g, beta = synth.gdr_inputs(1, T, 2, 64, 64, torch.bfloat16, seed=11, g_scale=0.003)
    h0 = 0.5 * torch.randn(len(lens), 2, 64, 64, generator=torch.Generator().manual_seed(4))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device), output_final_state=True,
                                     cu_seqlens=cu.to(device))
    _assert_bf16_close(o, want_o, "o varlen")
    _assert_bf16_close(s, want_s, "state varlen")


@pytest.mark.parametrize("K,V", [(128, 128), (64, 128), (128, 64)])
def test_chunk_other_head_sizes_and_l2norm(device, K, V):
    q, k, v, g, beta = synth.gdr_inputs(1, 333, 2, K, V, torch.bfloat16, seed=K + V, g_scale=0.05)
    q, k = (q.float() * 3).bfloat16(), (k.float() * 0.3).bfloat16()
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, l2=og.L2_CHUNK)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True,
                                     use_qk_l2norm_in_kernel=True)
    _assert_bf16_close(o, want_o, "o")
    _assert_bf16_close(s, want_s, "state")


def test_chunk_varlen_equals_separate_runs(device):
    lens = [5, 64, 0, 130, 700, 1]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)))
    T = int(cu[-1])
    q, k, v, g, beta = synth.gdr_inputs(1, T, 2, 64, 64, torch.bfloat16, seed=11, g_scale=0.05)
    h0 = 0.5 * torch.randn(len(lens), 2, 64, 64, generator=torch.Generator().manual_seed(4))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                     output_final_state=True, cu_seqlens=cu.to(device))
    _assert_bf16_close(o, want_o, "o")
    _assert_bf16_close(s, want_s, "state")
    assert torch.equal(s[2].cpu(), h0[2])  # an empty sequence returns its initial state
    # no final state requested -> None; fp16 inputs accepted
    o16, none = gd.chunk_gated_delta_rule(*_to(device, q.half(), k.half(), v.half(), g, beta), cu_seqlens=cu.to(device))
    assert none is None and o16.dtype == torch.float16
    w16, _ = og.recurrent_c(q.half(), k.half(), v.half(), g, beta, cu_seqlens=cu)
    _assert_bf16_close(o16, w16, "fp16 o")


def test_chunk_argument_checks(device):
    q, k, v, g, beta = _to(device, *synth.gdr_inputs(2, 128, 2, 64, 64, torch.bfloat16, seed=0))
    with pytest.raises(ValueError):
        gd.chunk_gated_delta_rule(q, k, v, g, beta, cu_seqlens=torch.tensor([0, 128], device=device))
    with pytest.raises(ValueError):
        gd.chunk_gated_delta_rule(q[:1], k[:1], v[:1], g[:1], beta[:1], cu_seqlens=torch.tensor([0, 100, 128], device=device),
                                  initial_state=torch.zeros(3, 2, 64, 64, device=device))
    with pytest.raises(DeprecationWarning):
        gd.chunk_gated_delta_rule(q, k, v, g, beta, head_first=True)
    with pytest.warns(UserWarning):
        gd.chunk_gated_delta_rule(q[:, :1], k[:, :1], v[:, :1], g[:, :1], beta[:, :1])
    with pytest.raises(Exception):
        gd.chunk_gated_delta_rule(q.cpu(), k.cpu(), v.cpu(), g.cpu(), beta.cpu())  # no CPU fallback


def test_chunk_positive_g_follows_the_reference_masking(device):
    # g > 0 is outside the operator's intended domain, but the reference's kernels define what happens: every decay
    # RATIO inside a chunk goes through safe_exp (fla_op.py:27-29). The oracle's chunk form applies the same masking;
    # positive entries sit on chunk starts (where nothing is masked) and inside chunks (where tokens are cut off).
    T = 300
    q, k, v, g, beta = synth.gdr_inputs(1, T, 2, 64, 64, torch.bfloat16, seed=21, g_scale=0.1)
    g = g.clone()
    g[0, [64, 128], 0] = 0.5
    g[0, [5, 70, 71, 190, 299], :] = torch.tensor([0.3, 1.0, 0.2, 0.6, 0.4])[:, None]
    h0 = 0.1 * torch.randn(1, 2, 64, 64, generator=torch.Generator().manual_seed(2))
    want_o, want_s = og.chunk_form(q, k, v, g, beta, initial_state=h0, chunk=64, masked=True)
    plain_o, _ = og.recurrent_delta(q, k, v, g, beta, initial_state=h0)
    assert (want_o - plain_o).abs().max() > 0.05  # the masking matters on this input
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device), output_final_state=True)
    _assert_bf16_close(o, want_o, "o")
    _assert_bf16_close(s, want_s, "state")
    # the in-kernel l2norm path goes through the same masked ratios
    want_o, want_s = og.chunk_form(q * 3, k * 2, v, g, beta, chunk=64, masked=True, l2=og.L2_CHUNK)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q * 3, k * 2, v, g, beta), output_final_state=True,
                                     use_qk_l2norm_in_kernel=True)
    _assert_bf16_close(o, want_o, "o l2")
    _assert_bf16_close(s, want_s, "state l2")


@pytest.mark.parametrize("D", [64, 128])
def test_chunk_fp16_weak_decay_long_sequence(device, D):
    # fp16 is the type the reference's layer feeds (modeling_gated_deltaproduct.py:583-587). With next to no decay the
    # state keeps everything it was ever given, the regime in which rounding errors of the operands accumulate the most;
    # fp16 operands stay fp16 on the MFMA (11-bit mantissa), so the result sits far inside the bf16 contract.
    T, H = 20000, 2
    q, k, v, g, beta = synth.gdr_inputs(1, T, H, D, D, torch.float16, seed=D, g_scale=0.003)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True)
    assert o.dtype == torch.float16
    _assert_bf16_close(o, want_o, "fp16 o")
    _assert_bf16_close(s, want_s, "fp16 state")
    max_abs, mean_rel = _errors(o, want_o)
    assert mean_rel <= 1.5e-3, f"fp16 operands should beat the bf16 error level by far: {mean_rel:.3e}"
    # the same inputs rounded to bf16 go through the bf16 MFMA and stay inside the same contract
    ob, sb = gd.chunk_gated_delta_rule(*_to(device, q.bfloat16(), k.bfloat16(), v.bfloat16(), g, beta), output_final_state=True)
    wb_o, wb_s = og.recurrent_c(q.bfloat16(), k.bfloat16(), v.bfloat16(), g, beta)
    _assert_bf16_close(ob, wb_o, "bf16 o")
    _assert_bf16_close(sb, wb_s, "bf16 state")


@pytest.mark.parametrize("K,V", [(16, 32), (32, 32), (96, 40)])
def test_chunk_small_heads_long_sequence_fp16(device, K, V):
    # the head sizes of the reference's own layer (d_k = 16, d_v = 32, fp16: modeling_gated_deltaproduct.py:583-587)
    # go through the chunk kernels as a zero-padded 64- or 128-wide head, not through the token loop
    T, H = 30000, 6
    q, k, v, g, beta = synth.gdr_inputs(1, T, H, K, V, torch.float16, seed=K + V, g_scale=0.05)
    h0 = torch.randn(1, H, K, V, generator=torch.Generator().manual_seed(1)) * 0.1
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0)
    dq, dk, dv, dg, db = _to(device, q, k, v, g, beta)
    o, s = gd.chunk_gated_delta_rule(dq, dk, dv, dg, db, initial_state=h0.to(device), output_final_state=True)
    assert o.shape == (1, T, H, V) and s.shape == (1, H, K, V) and o.dtype == torch.float16 and o.is_contiguous()
    _assert_bf16_close(o, want_o, "small-head o")
    _assert_bf16_close(s, want_s, "small-head state")
    if (K, V) == (16, 32):  # the token-serial operator on a prefix of the same inputs (its timing is a bench.py leg)
        o2, s2 = gd.fused_recurrent_gated_delta_rule(dq[:, :4096], dk[:, :4096], dv[:, :4096], dg[:, :4096],
                                                     db[:, :4096], initial_state=h0.to(device), output_final_state=True)
        _assert_bf16_close(o[:, :4096], o2.float().cpu(), "chunk vs token loop")


def test_chunk_bf16_weak_decay_at_the_headline_length(device):
    # The regime in which the bf16 error is largest: next to no decay (g scaled by 3e-3), so the state keeps everything
    # it was ever given and the rounding of the MFMA operands accumulates over all 60 000 tokens. The contract
    # (max-abs 2e-2, mean-rel 5e-3) is asserted and the measured margin printed.
    T, H, D = 60000, 2, 64
    q, k, v, g, beta = synth.gdr_inputs(1, T, H, D, D, torch.bfloat16, seed=11, g_scale=0.003)
    want_o, want_s = og.recurrent_c(q, k, v, g, beta)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True)
    for got, want, what in ((o, want_o, "o"), (s, want_s, "state")):
        max_abs, mean_rel = _errors(got, want)
        print(f"bf16 weak decay T={T} H={H} K=V={D} g x 0.003: {what} max-abs {max_abs:.3e} (bound 2e-2), "
              f"mean-rel {mean_rel:.3e} (bound 5e-3)")
        _assert_bf16_close(got, want, f"weak-decay bf16 {what}")


@pytest.mark.parametrize("T", [1, 64, 65, 200, 1000])
def test_chunk_32_wide_heads_short_sequences(device, T):
    # the 32 x 32 build of the chunk kernels: batch 2, grouped value heads, initial state, both l2norm settings
    gen = torch.Generator().manual_seed(T)
    B, H, HV = 2, 2, 4
    q = torch.randn(B, T, H, 32, generator=gen).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, T, H, 32, generator=gen), dim=-1).bfloat16()
    v = torch.randn(B, T, HV, 32, generator=gen).bfloat16()
    g = -torch.rand(B, T, HV, generator=gen) * 0.3
    beta = torch.rand(B, T, HV, generator=gen)
    h0 = 0.5 * torch.randn(B, HV, 32, 32, generator=gen)
    for l2, flag in ((og.L2_NONE, False), (og.L2_CHUNK, True)):
        want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, l2=l2)
        o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                         output_final_state=True, use_qk_l2norm_in_kernel=flag)
        _assert_bf16_close(o, want_o, f"o T={T} l2={flag}")
        _assert_bf16_close(s, want_s, f"state T={T} l2={flag}")


def test_chunk_32_wide_heads_varlen_and_many_segments(device, monkeypatch):
    # packed sequences incl. an empty one; one chunk per segment, so that long sequences take the two-level scan
    monkeypatch.setattr(gd, "CHUNKS_PER_SEGMENT", 1)
    lens = [64 * 30 + 1, 5, 0, 64 * 9, 64 * 26 - 1]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.long)
    T = int(cu[-1])
    q, k, v, g, beta = synth.gdr_inputs(1, T, 3, 32, 32, torch.float16, seed=12, g_scale=0.003)
    h0 = 0.5 * torch.randn(len(lens), 3, 32, 32, generator=torch.Generator().manual_seed(4))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, cu_seqlens=cu)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device), output_final_state=True,
                                     cu_seqlens=cu.to(device))
    _assert_bf16_close(o, want_o, "o varlen 32")
    _assert_bf16_close(s, want_s, "state varlen 32")


def test_chunk_matches_token_serial_kernel_on_gpu(device):
    q, k, v, g, beta = _to(device, *synth.gdr_inputs(1, 5000, 4, 64, 64, torch.bfloat16, seed=21, g_scale=0.1))
    o1, s1 = gd.chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    o2, s2 = gd.fused_recurrent_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    _assert_bf16_close(o1, o2.float().cpu(), "o")
    _assert_bf16_close(s1, s2.cpu(), "state")


@pytest.mark.parametrize("g_scale", [1.0, 0.003])
def test_fp32_mode_at_the_config2_shape(device, g_scale):
    # the fp32 mode of the chunk operator (allow_fp32) at the headline shape, T = 60000, d = 64 (four heads): fp32 inputs
    # through the token-serial kernels as parallel segments, 1e-4 against the fp64 token loop, with strong and weak decay
    q, k, v, g, beta = synth.gdr_inputs(1, 60000, 4, 64, 64, torch.float32, seed=5, g_scale=g_scale)
    h0 = 0.5 * torch.randn(1, 4, 64, 64, generator=torch.Generator().manual_seed(6))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta, initial_state=h0, l2=og.L2_CHUNK)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), initial_state=h0.to(device),
                                     output_final_state=True, allow_fp32=True, use_qk_l2norm_in_kernel=True)
    assert o.dtype == torch.float32
    assert _errors(o, want_o)[0] <= FP32_TOL and _errors(s, want_s)[0] <= FP32_TOL


def test_config2_full_size(device):
    # B=1, H=8, T=60000, d=64, bf16 q/k/v, fp32 g/beta, tokens in the LSH-sorted order of a config-1 event
    from lampa_amd import lsh

    q, k, v, g, beta = synth.gdr_inputs(1, 60000, 8, 64, 64, torch.bfloat16, seed=0)
    coords, _, _ = synth.collider_event(60000, seed=0)
    alpha, b = synth.lsh_params(4, 3, 4, 0.5, 1)
    perm = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), b.to(device), 0.5, 3, 4)["perm"][0].long().cpu()
    q, k, v, g, beta = (x[:, perm].contiguous() for x in (q, k, v, g, beta))
    want_o, want_s = og.recurrent_c(q, k, v, g, beta)
    o, s = gd.chunk_gated_delta_rule(*_to(device, q, k, v, g, beta), output_final_state=True)
    _assert_bf16_close(o, want_o, "o")
    _assert_bf16_close(s, want_s, "state")
    # size-independent property: splitting the sequence and carrying the state reproduces the one-shot run
    cut = 64 * 400 + 17
    oa, sa = gd.chunk_gated_delta_rule(*_to(device, q[:, :cut], k[:, :cut], v[:, :cut], g[:, :cut], beta[:, :cut]),
                                       output_final_state=True)
    ob, sb = gd.chunk_gated_delta_rule(*_to(device, q[:, cut:], k[:, cut:], v[:, cut:], g[:, cut:], beta[:, cut:]),
                                       initial_state=sa, output_final_state=True)
    _assert_bf16_close(torch.cat([oa, ob], 1), o.float().cpu(), "split o")
    _assert_bf16_close(sb, s.cpu(), "split state")


def test_config4_varlen_batch_d128(device):
    # 16 events of U[6000, 60000] hits packed with cu_seqlens, H=8, d_k=d_v=128, bf16 (about 528k tokens)
    lens, cu = synth.varlen_lengths(16, 6000, 60000, seed=0)
    T = int(cu[-1])
    q, k, v, g, beta = synth.gdr_inputs(1, T, 8, 128, 128, torch.bfloat16, seed=4)
    dq, dk, dv, dg, db = _to(device, q, k, v, g, beta)
    cud = cu.to(device)
    o, s = gd.chunk_gated_delta_rule(dq, dk, dv, dg, db, output_final_state=True, cu_seqlens=cud)
    assert o.shape == (1, T, 8, 128) and s.shape == (16, 8, 128, 128)
    # the whole batch against the token-serial kernel (fp32 state, itself checked against the oracle above)
    o2, s2 = gd.fused_recurrent_gated_delta_rule(dq, dk, dv, dg, db, output_final_state=True, cu_seqlens=cud)
    _assert_bf16_close(o, o2.float().cpu(), "o vs token-serial")
    _assert_bf16_close(s, s2.cpu(), "state vs token-serial")
    # the shortest event against the CPU oracle
    i = int(torch.argmin(lens))
    a, b = int(cu[i]), int(cu[i + 1])
    want_o, want_s = og.recurrent_c(q[:, a:b], k[:, a:b], v[:, a:b], g[:, a:b], beta[:, a:b])
    _assert_bf16_close(o[:, a:b], want_o, "o vs oracle")
    _assert_bf16_close(s[i:i + 1], want_s, "state vs oracle")
    # packing is invisible: the same event run alone gives the same result
    o1, s1 = gd.chunk_gated_delta_rule(dq[:, a:b], dk[:, a:b], dv[:, a:b], dg[:, a:b], db[:, a:b], output_final_state=True)
    _assert_bf16_close(o[:, a:b], o1.float().cpu(), "o alone")
    _assert_bf16_close(s[i:i + 1], s1.cpu(), "state alone")


def test_traffic_probe_writes_every_output_row(device):
    """The memory-only twin of the output pass (a measurement aid): it must touch exactly the rows the real kernel
    writes. Its stores carry (chunk, row, 16-byte piece) so that coverage can be checked; ragged last segment."""
    from lampa_amd import _capi
    n_chunks, H, cps = 11, 3, 4
    T = 64 * n_chunks
    q, k, v = (torch.zeros(T, H, 64, dtype=torch.bfloat16, device=device) for _ in range(3))
    rec = torch.zeros(n_chunks * H * 6656, dtype=torch.uint8, device=device)
    o = torch.full((T, H, 64), -1.0, dtype=torch.bfloat16, device=device)
    _capi.check(_capi.lib().lampa_gdr_traffic_probe(q.data_ptr(), k.data_ptr(), v.data_ptr(), rec.data_ptr(), o.data_ptr(),
                                                    n_chunks, H, cps, torch.cuda.current_stream().cuda_stream), "probe")
    torch.cuda.synchronize()
    words = o.view(torch.int32).reshape(n_chunks, 64, H, 8, 4).cpu()  # [chunk, row, head, piece, word]
    want = torch.zeros_like(words)
    want[..., 0] = torch.arange(n_chunks).view(-1, 1, 1, 1)
    want[..., 1] = torch.arange(64).view(1, -1, 1, 1)
    want[..., 2] = torch.arange(8).view(1, 1, 1, -1)
    assert torch.equal(words, want)
    assert _capi.lib().lampa_gdr_traffic_probe(None, k.data_ptr(), v.data_ptr(), rec.data_ptr(), o.data_ptr(), n_chunks, H,
                                               cps, None) == -1
    # the form that also reads the composites of the walk (27 one-chunk segments: four groups, walks of up to 3 + 7 steps)
    n2 = 27
    q2, k2, v2 = (torch.zeros(64 * n2, H, 64, dtype=torch.bfloat16, device=device) for _ in range(3))
    rec2 = torch.zeros(n2 * H * 6656, dtype=torch.uint8, device=device)
    comp = torch.zeros((n2 + 4) * H * 24576, dtype=torch.uint8, device=device)
    o2 = torch.full((64 * n2, H, 64), -1.0, dtype=torch.bfloat16, device=device)
    _capi.check(_capi.lib().lampa_gdr_traffic_probe_walk(q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), rec2.data_ptr(),
                                                         comp.data_ptr(), o2.data_ptr(), n2, H, 1,
                                                         torch.cuda.current_stream().cuda_stream), "probe walk")
    torch.cuda.synchronize()
    words2 = o2.view(torch.int32).reshape(n2, 64, H, 8, 4).cpu()
    assert torch.equal(words2[..., 0], torch.arange(n2).view(-1, 1, 1, 1).expand(n2, 64, H, 8).int())
    assert _capi.lib().lampa_gdr_traffic_probe_walk(q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), rec2.data_ptr(), None,
                                                    o2.data_ptr(), n2, H, 1, None) == -1
