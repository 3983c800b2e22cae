"""GPU parity of the gated-delta backward pass (``lampa_gdr_bwd`` behind ``chunk_gated_delta_rule``'s autograd) against
the gradient oracle (``oracle.gated_delta_bwd.backward_manual``, float64 on the same, already rounded, inputs).

Tolerances: the token-serial kernels (``lampa_gdr_bwd``) compute in fp32 from the inputs as given, so fp32 inputs must
agree to 1e-4 (max-abs relative to the largest entry of the gradient; 1e-5 mean-relative); with bf16 / fp16 inputs dq,
dk and dv are rounded to that type on output (mean-relative 5e-3, the forward's bound), dg, dbeta and d(initial state)
stay fp32 (1e-4). The chunked form (``lampa_gdr_bwd_chunk``: 16-bit inputs, K = V = 64, one value head per q/k head)
rounds every MFMA operand to the input type, as the reference's backward kernels do: all six gradients then carry that
type's rounding through a chain of five to six rounded intermediates (max-abs 2e-2 of the largest entry; mean-relative
8e-3; measured 3e-3 to 5.2e-3 for bf16, 5e-4 for fp16).
"""
import pytest
import torch

from lampa_amd import gated_delta as gd
from oracle import gated_delta as og
from oracle import gated_delta_bwd as ob

pytestmark = pytest.mark.gpu

NAMES = ("dq", "dk", "dv", "dg", "dbeta", "dh0")


def _inputs(B, T, H, HV, K, V, dtype, seed, unit, g_scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    if unit:
        q, k = q / q.norm(dim=-1, keepdim=True), k / k.norm(dim=-1, keepdim=True)
    v = torch.randn(B, T, HV, V, generator=gen)
    g = -g_scale * torch.nn.functional.softplus(torch.randn(B, T, HV, generator=gen))
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
    do = torch.randn(B, T, HV, V, generator=gen)
    return [x.to(dtype) for x in (q, k, v)] + [g, beta, do.to(dtype)], gen


def _gpu_grads(device, q, k, v, g, beta, do, h0, dht, cu, l2, scale=None):
    args = [x.to(device).requires_grad_(True) for x in (q, k, v, g, beta)]
    h0d = None if h0 is None else h0.to(device).requires_grad_(True)
    o, ht = gd.chunk_gated_delta_rule(*args, scale=scale, initial_state=h0d, output_final_state=dht is not None,
                                      cu_seqlens=None if cu is None else cu.to(device), use_qk_l2norm_in_kernel=l2,
                                      allow_fp32=True)
    loss = (o.float() * do.to(device).float()).sum()
    if dht is not None:
        loss = loss + (ht * dht.to(device)).sum()
    loss.backward()
    return [a.grad for a in args] + [None if h0d is None else h0d.grad]


def _check(got, want, dtype, chunked=None):
    """chunked: the gradients came from the chunked form (default: every 16-bit case while ``gd.CHUNKED_BACKWARD``)."""
    if chunked is None:
        chunked = dtype != torch.float32 and gd.CHUNKED_BACKWARD
    for name, a, b in zip(NAMES, got, want):
        if b is None:
            assert a is None, name
            continue
        a = a.double().cpu()
        assert a.shape == b.shape, name
        diff = (a - b).abs()
        rel_max = diff.max().item() / b.abs().max().clamp_min(1e-30).item()
        rel_mean = (diff.mean() / b.abs().mean().clamp_min(1e-30)).item()
        rounded = dtype != torch.float32 and (chunked or name in ("dq", "dk", "dv"))
        mean_bound = (8e-3 if chunked else 5e-3) if rounded else 1e-5
        assert rel_max <= (2e-2 if rounded else 1e-4) and rel_mean <= mean_bound, \
            f"{name}: max {rel_max:.3e} mean {rel_mean:.3e}"


@pytest.mark.parametrize("K,V,H,HV", [(16, 32, 2, 4), (64, 64, 2, 2), (128, 128, 1, 2), (32, 48, 1, 1), (24, 40, 2, 2),
                                      (10, 6, 1, 3), (128, 20, 1, 1)])
@pytest.mark.parametrize("l2", [False, True])
def test_gradients_fp32_match_oracle(device, K, V, H, HV, l2):
    """Equal-length batches with an initial state and a gradient into the final state; T = 75 leaves a partial block of
    8 tokens and a partial segment; head sizes on and off the kernels' shapes (10 x 6 is zero-padded to 12 x 8)."""
    (q, k, v, g, beta, do), gen = _inputs(2, 75, H, HV, K, V, torch.float32, K + V, unit=not l2)
    h0 = 0.5 * torch.randn(2, HV, K, V, generator=gen)
    dht = torch.randn(2, HV, K, V, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, 0.37, h0, None, og.L2_CHUNK if l2 else og.L2_NONE)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, None, l2, scale=0.37), want, torch.float32)


@pytest.mark.parametrize("dtype,chunked", [(torch.float32, False), (torch.bfloat16, False), (torch.float16, False),
                                           (torch.bfloat16, True), (torch.float16, True)])
def test_gradients_varlen_segments(device, dtype, chunked, monkeypatch):
    """Packed sequences (an empty one, one shorter than a block, lengths off the block and segment sizes), cut into
    segments of 64 tokens so that the reverse maps and the reverse scan carry the state gradient over many segments.
    16-bit inputs through both forms: token-serial, and chunked with the 32 x 32 heads zero-padded to 64 x 64 and the
    two value heads of a group sharing their q / k head."""
    monkeypatch.setattr(gd, "BACKWARD_UNITS", 1 << 20)
    monkeypatch.setattr(gd, "CHUNKED_BACKWARD", chunked)
    lens = [0, 5, 333, 64, 1, 500, 97]
    T = sum(lens)
    (q, k, v, g, beta, do), gen = _inputs(1, T, 2, 4, 32, 32, dtype, 7, unit=False)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.long)
    h0 = 0.5 * torch.randn(len(lens), 4, 32, 32, generator=gen)
    dht = torch.randn(len(lens), 4, 32, 32, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, None, h0, cu, og.L2_CHUNK)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, cu, True), want, dtype)


def test_gradients_many_short_sequences_more_units_than_workgroups(device):
    """700 packed sequences of 1 .. 20 tokens: 700 segments x 4 heads x 2 slabs = 5 600 units for the segment kernel's
    4 096 workgroups, so some workgroups take a second unit (and reuse their spill area and LDS for it)."""
    gen = torch.Generator().manual_seed(13)
    lens = torch.randint(1, 21, (700,), generator=gen).tolist()
    T = sum(lens)
    (q, k, v, g, beta, do), gen = _inputs(1, T, 2, 4, 16, 32, torch.float32, 17, unit=False)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.long)
    h0 = 0.5 * torch.randn(700, 4, 16, 32, generator=gen)
    dht = torch.randn(700, 4, 16, 32, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, None, h0, cu, og.L2_CHUNK)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, cu, True), want, torch.float32)


def test_gradients_scans_in_groups_unbalanced_sequences(device, monkeypatch):
    """Three sequences (one empty, one of a single short segment) cut into 64-token segments, 75 of them: both scans of
    the backward pass (forward, and reversed with one extra row per sequence) run in their three-launch form over groups
    of segments."""
    monkeypatch.setattr(gd, "BACKWARD_UNITS", 1 << 20)
    lens = [0, 4700, 30]
    T = sum(lens)
    (q, k, v, g, beta, do), gen = _inputs(1, T, 1, 2, 16, 16, torch.float32, 23, unit=False, g_scale=0.05)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.long)
    h0 = 0.5 * torch.randn(3, 2, 16, 16, generator=gen)
    dht = torch.randn(3, 2, 16, 16, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, None, h0, cu, og.L2_CHUNK)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, cu, True), want, torch.float32)


def test_gradients_without_states_and_with_unused_output(device):
    """No initial state (no d h0), no final state; and a loss that uses the final state only (d o is zero)."""
    (q, k, v, g, beta, do), gen = _inputs(1, 200, 1, 2, 64, 64, torch.float32, 3, unit=True)
    want = ob.backward_manual(q, k, v, g, beta, do, None, None, None, None, og.L2_NONE)
    _check(_gpu_grads(device, q, k, v, g, beta, do, None, None, None, False), want, torch.float32)
    dht = torch.randn(1, 2, 64, 64, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, torch.zeros_like(do), dht, None, None, None, og.L2_NONE)
    args = [x.to(device).requires_grad_(True) for x in (q, k, v, g, beta)]
    _, ht = gd.chunk_gated_delta_rule(*args, output_final_state=True, allow_fp32=True)
    (ht * dht.to(device)).sum().backward()
    _check([a.grad for a in args] + [None], want, torch.float32)


def test_gradients_long_sequence_weak_decay(device):
    """4 096 tokens with g of the order of -0.003 per token: the state and its gradient carry over hundreds of tokens
    and through every segment (token-serial form; the chunked form has its own case below)."""
    gd_chunked = gd.CHUNKED_BACKWARD
    gd.CHUNKED_BACKWARD = False
    try:
        _weak_decay_case(device)
    finally:
        gd.CHUNKED_BACKWARD = gd_chunked


def _weak_decay_case(device):
    (q, k, v, g, beta, do), gen = _inputs(1, 4096, 1, 2, 64, 64, torch.bfloat16, 11, unit=False, g_scale=0.003)
    h0 = 0.5 * torch.randn(1, 2, 64, 64, generator=gen)
    dht = torch.randn(1, 2, 64, 64, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, None, h0, None, og.L2_CHUNK)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, None, True), want, torch.bfloat16)


def test_gradients_do_not_depend_on_the_segmentation_at_full_size(device, monkeypatch):
    """Config-2 shape (60 032 tokens, 8 heads, K = V = 64, bf16), too long for the float64 loop, on the token-serial
    form: the same gradients from 63 segments per head and from 8 (fp32 rounding apart), and linear in (d o, d final
    state)."""
    monkeypatch.setattr(gd, "CHUNKED_BACKWARD", False)
    (q, k, v, g, beta, do), gen = _inputs(1, 60032, 8, 8, 64, 64, torch.bfloat16, 5, unit=False)
    dht = torch.randn(1, 8, 64, 64, generator=gen)
    a = _gpu_grads(device, q, k, v, g, beta, do, None, dht, None, True)
    monkeypatch.setattr(gd, "BACKWARD_UNITS", 256)
    b = _gpu_grads(device, q, k, v, g, beta, do, None, dht, None, True)
    for name, x, y in zip(NAMES[:5], a, b):
        x, y = x.float(), y.float()
        assert torch.isfinite(x).all(), name
        rounded = name in ("dq", "dk", "dv")  # bf16 outputs: one rounding step apart at most
        assert (x - y).abs().max().item() <= (1e-2 if rounded else 2e-4) * y.abs().max().item(), name
    c = _gpu_grads(device, q, k, v, g, beta, (2 * do.float()).to(do.dtype), None, 2 * dht, None, True)
    for name, x, y in zip(NAMES[3:5], b[3:5], c[3:5]):  # the fp32 outputs: exactly twice (a power of two)
        assert torch.equal(2 * x, y), name


def test_fused_recurrent_backward_raises_like_the_reference(device):
    (q, k, v, g, beta, do), _ = _inputs(1, 16, 1, 1, 16, 16, torch.float32, 0, unit=True)
    args = [x.to(device).requires_grad_(True) for x in (q, k, v, g, beta)]
    o, _ = gd.fused_recurrent_gated_delta_rule(*args)
    with pytest.raises(NotImplementedError):
        o.sum().backward()


def test_backward_refuses_positive_log_decay(device):
    # for g > 0 the chunk forward masks decay ratios with positive exponents (safe_exp) while the backward pass
    # differentiates the unmasked recurrence: the two would belong to different functions, so backward raises
    (q, k, v, g, beta, do), _ = _inputs(1, 130, 2, 2, 64, 64, torch.bfloat16, 0, True)
    g = g.clone()
    g[0, 70, 1] = 0.25
    args = [x.to(device).requires_grad_(True) for x in (q, k, v, g, beta)]
    o, _ = gd.chunk_gated_delta_rule(*args)          # the forward itself accepts it, as the reference's does
    with pytest.raises(ValueError, match="g <= 0"):
        o.float().sum().backward()


# ------------------------------------------------------------------------------------- chunked form on the MFMA
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("l2", [False, True])
@pytest.mark.parametrize("T", [1, 64, 75, 1000])
def test_chunked_gradients_match_oracle(device, dtype, l2, T):
    """K = V = 64, H = HV, 16-bit inputs take ``lampa_gdr_bwd_chunk``: batches with an initial state and a gradient into
    the final state; one token, one chunk, a partial second chunk, 16 chunks (two levels of the scan)."""
    assert gd._backward_chunk_supported(torch.empty(1, 1, 2, 64, dtype=dtype), torch.empty(1, 1, 2, 64, dtype=dtype))
    (q, k, v, g, beta, do), gen = _inputs(2, T, 2, 2, 64, 64, dtype, T, unit=not l2)
    h0 = 0.5 * torch.randn(2, 2, 64, 64, generator=gen)
    dht = torch.randn(2, 2, 64, 64, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, 0.2, h0, None, og.L2_CHUNK if l2 else og.L2_NONE)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, None, l2, scale=0.2), want, dtype, chunked=True)


def test_chunked_gradients_varlen_and_without_states(device):
    """Packed sequences (an empty one, one token, lengths off the chunk size, one of 80 chunks: three levels of the
    scan) with states; then no initial state and no gradient into the final state; then a loss on the final state only."""
    lens = [0, 5, 333, 64, 1, 5100, 97]
    T = sum(lens)
    (q, k, v, g, beta, do), gen = _inputs(1, T, 3, 3, 64, 64, torch.bfloat16, 7, unit=False, g_scale=0.3)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.long)
    h0 = 0.5 * torch.randn(len(lens), 3, 64, 64, generator=gen)
    dht = torch.randn(len(lens), 3, 64, 64, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, None, h0, cu, og.L2_CHUNK)
    _check(_gpu_grads(device, q, k, v, g, beta, do, h0, dht, cu, True), want, torch.bfloat16, chunked=True)
    want = ob.backward_manual(q, k, v, g, beta, do, None, None, None, cu, og.L2_CHUNK)
    _check(_gpu_grads(device, q, k, v, g, beta, do, None, None, cu, True), want, torch.bfloat16, chunked=True)
    want = ob.backward_manual(q, k, v, g, beta, torch.zeros_like(do), dht, None, None, cu, og.L2_CHUNK)
    args = [x.to(device).requires_grad_(True) for x in (q, k, v, g, beta)]
    _, ht = gd.chunk_gated_delta_rule(*args, output_final_state=True, cu_seqlens=cu.to(device),
                                      use_qk_l2norm_in_kernel=True)
    (ht * dht.to(device)).sum().backward()
    _check([a.grad for a in args] + [None], want, torch.bfloat16, chunked=True)


def test_chunked_gradients_long_sequence_weak_decay_against_oracle(device):
    """16 448 tokens (257 chunks + the extra item: three levels of the scan, a ragged last group) with g of the order of
    -0.003 per token, so that states and their gradients carry over thousands of tokens, against the float64 loop."""
    (q, k, v, g, beta, do), gen = _inputs(1, 16448, 2, 2, 64, 64, torch.bfloat16, 11, unit=True, g_scale=0.003)
    h0 = 0.5 * torch.randn(1, 2, 64, 64, generator=gen)
    dht = torch.randn(1, 2, 64, 64, generator=gen)
    want = ob.backward_manual(q, k, v, g, beta, do, dht, None, h0, None, og.L2_NONE)
    got = _gpu_grads(device, q, k, v, g, beta, do, h0, dht, None, False)
    for name, a, b in zip(NAMES, got, want):
        d = (a.double().cpu() - b).abs()
        print(f"chunked backward T=16448 weak decay {name}: max-rel {d.max().item() / b.abs().max().item():.2e} "
              f"mean-rel {(d.mean() / b.abs().mean()).item():.2e}")
    _check(got, want, torch.bfloat16, chunked=True)


def test_chunked_gradients_at_full_size_against_the_token_serial_form(device, monkeypatch):
    """Config-2 shape (60 000 tokens, 8 heads, K = V = 64, bf16), too long for the float64 loop: the chunked form on the
    MFMA against the fp32 token-serial form, two implementations that share no kernel of the backward pass."""
    (q, k, v, g, beta, do), gen = _inputs(1, 60000, 8, 8, 64, 64, torch.bfloat16, 5, unit=False)
    dht = torch.randn(1, 8, 64, 64, generator=gen)
    h0 = 0.5 * torch.randn(1, 8, 64, 64, generator=gen)
    a = _gpu_grads(device, q, k, v, g, beta, do, h0, dht, None, True)
    monkeypatch.setattr(gd, "CHUNKED_BACKWARD", False)
    b = _gpu_grads(device, q, k, v, g, beta, do, h0, dht, None, True)
    _check(a, [x.double().cpu() for x in b], torch.bfloat16, chunked=True)
