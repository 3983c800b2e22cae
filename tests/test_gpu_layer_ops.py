"""GPU parity of the short convolution and the (gated) RMS norm against the float64 CPU oracle.

Tolerances: the kernels compute in fp32 and round once to the output type, so the bound is one rounding of the output
(2^-8 relative for bf16, 2^-11 for fp16) plus fp32 noise; fp32 outputs must agree to 2e-6 relative + 2e-6 absolute."""
import numpy as np
import pytest
import torch

from lampa_amd import layer_ops as lo
from oracle import layer_ops as ol

pytestmark = pytest.mark.gpu

TOL = {torch.float32: (2e-6, 2e-6), torch.bfloat16: (2 ** -8, 1e-5), torch.float16: (2 ** -11, 1e-6)}


def _close(got: torch.Tensor, want: np.ndarray, dtype):
    rtol, atol = TOL[dtype]
    got = got.detach().double().cpu().numpy()
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + atol
    assert np.all(err <= bound), (float(err.max()), float((err - bound).max()))


def _f64(t):
    return t.detach().double().cpu().numpy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,T,D,W", [(1, 1, 8, 4), (2, 37, 64, 4), (1, 1000, 512, 4), (3, 65, 24, 2), (1, 50, 16, 1)])
def test_causal_conv1d_dense(device, dtype, B, T, D, W):
    gen = torch.Generator().manual_seed(B * 1000 + T)
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    w = (torch.randn(D, W, generator=gen) * 0.5).to(dtype)
    b = torch.randn(D, generator=gen).to(dtype)
    res = torch.randn(B, T, D, generator=gen).to(dtype)
    for bias, residual, act in ((None, None, None), (b, None, "silu"), (b, res, "swish")):
        got = lo.causal_conv1d(x.to(device), w.to(device), None if bias is None else bias.to(device),
                               None if residual is None else residual.to(device), act)
        want = ol.causal_conv1d(_f64(x), _f64(w), None if bias is None else _f64(bias),
                                None if residual is None else _f64(residual), act)
        assert got.shape == (B, T, D) and got.dtype == dtype
        _close(got, want, dtype)


def test_causal_conv1d_varlen_strided_and_config_shape(device):
    gen = torch.Generator().manual_seed(3)
    T, D, W = 60000, 512, 4
    proj = torch.randn(1, T, 3 * D, generator=gen).to(torch.bfloat16).to(device)     # fused q|k|v projection output
    w = (torch.randn(D, W, generator=gen) * 0.5).to(torch.bfloat16)
    cu = torch.tensor([0, 17, 17, 4099, 4100, 33333, 60000])
    for part in range(3):
        x = proj[..., part * D:(part + 1) * D]                                       # a strided slice, not copied
        got = lo.causal_conv1d(x, w.to(device), activation="silu", cu_seqlens=cu.to(device))
        want = ol.causal_conv1d(_f64(x), _f64(w), activation="silu", cu_seqlens=cu.numpy())
        _close(got, want, torch.bfloat16)
    dense = lo.causal_conv1d(proj[..., :D], w.to(device), activation="silu")
    _close(dense, ol.causal_conv1d(_f64(proj[..., :D]), _f64(w), activation="silu"), torch.bfloat16)
    with pytest.raises(ValueError):
        lo.causal_conv1d(proj[..., :D], w.to(device), activation="gelu")


def test_causal_conv1d_split_equals_separate_calls(device):
    gen = torch.Generator().manual_seed(6)
    T, D = 3001, 128
    proj = torch.randn(1, T, 3 * D + 16, generator=gen).to(torch.bfloat16).to(device)
    ws = [(torch.randn(D, 1, 4, generator=gen) * 0.5).to(torch.bfloat16).to(device) for _ in range(3)]
    bs = [torch.randn(D, generator=gen).to(torch.bfloat16).to(device) for _ in range(3)]
    cu = torch.tensor([0, 5, 1000, 3001], device=device)
    for biases, cu_t in ((None, None), (bs, cu)):
        outs = lo.causal_conv1d_split(proj[..., :3 * D], ws, biases, "silu", cu_t)
        for i, y in enumerate(outs):
            one = lo.causal_conv1d(proj[..., i * D:(i + 1) * D], ws[i].reshape(D, 4), None if biases is None else bs[i],
                                   None, "silu", cu_t)
            assert y.is_contiguous() and torch.equal(y, one)
    with torch.no_grad():                                   # remembered fp32 copies follow in-place weight updates
        ws[0].mul_(2.0)
    again = lo.causal_conv1d_split(proj[..., :3 * D], ws, None, "silu")[0]
    assert torch.equal(again, lo.causal_conv1d(proj[..., :D].contiguous(), ws[0].reshape(D, 4).clone(), None, None, "silu"))


@pytest.mark.parametrize("B,T,tokens_per_wg", [(1, 1, 0), (1, 31, 0), (2, 700, 64), (1, 5000, 512), (3, 333, 96)])
def test_fused_projection_convolution(device, B, T, tokens_per_wg):
    """One kernel for projections + convolution + SiLU against the float64 oracle (tolerance: the projection output is
    rounded to bf16 before the convolution, as a bf16 linear layer's is, then one more rounding of the result) and
    against the two-step route on the GPU (same roundings, different summation order inside the GEMM)."""
    gen = torch.Generator().manual_seed(B * 100 + T)
    x = torch.randn(B, T, 128, generator=gen).to(torch.bfloat16)
    W = (torch.randn(3 * 512 + 512 + 16, 128, generator=gen) * 0.1).to(torch.bfloat16)
    cws = [(torch.randn(512, 1, 4, generator=gen) * 0.5).to(torch.bfloat16) for _ in range(3)]
    cbs = [torch.randn(512, generator=gen).to(torch.bfloat16) for _ in range(3)]
    for biases in (None, cbs):
        (q, k, v), g, ab = lo.proj_conv(x.to(device), W.to(device), [w.to(device) for w in cws],
                                        None if biases is None else [b.to(device) for b in biases], 512, 512, tokens_per_wg)
        assert q.shape == (B, T, 512) and g.shape == (B, T, 512) and ab.shape == (B, T, 16) and q.is_contiguous()
        pre = _f64(x) @ _f64(W).T                                             # [B, T, 2064]
        pre_b = torch.from_numpy(pre).to(torch.bfloat16)                        # the rounding the kernel applies
        for i, got in enumerate((q, k, v)):
            want = ol.causal_conv1d(_f64(pre_b[..., 512 * i:512 * (i + 1)]), _f64(cws[i]).reshape(512, 4),
                                    None if biases is None else _f64(biases[i]), None, "silu")
            err = np.abs(_f64(got) - want)
            # one bf16 rounding of the result plus the effect of last-bit differences of the rounded projections
            assert np.all(err <= 2 ** -7 * np.abs(want) + 2e-2), float(err.max())
            assert err.mean() < 2e-3
        assert np.all(np.abs(_f64(g) - pre[..., 1536:2048]) <= 2 ** -8 * np.abs(pre[..., 1536:2048]) + 1e-6)
        assert np.all(np.abs(_f64(ab) - pre[..., 2048:]) <= 2 ** -8 * np.abs(pre[..., 2048:]) + 1e-6)
    # two-step route on the GPU
    proj = torch.nn.functional.linear(x.to(device), W.to(device))
    q2, k2, v2 = lo.causal_conv1d_split(proj[..., :1536], [w.to(device) for w in cws], [b.to(device) for b in cbs], "silu")
    for a, b2 in ((q, q2), (k, k2), (v, v2)):
        assert (a.float() - b2.float()).abs().max() < 0.1 and (a.float() - b2.float()).abs().mean() < 2e-3
    assert (g.float() - proj[..., 1536:2048].float()).abs().max() < 0.05


@pytest.mark.parametrize("B,T,tokens_per_wg", [(1, 1, 0), (2, 333, 64), (1, 6000, 0), (1, 100, 32)])
def test_fused_gated_norm_output_projection(device, B, T, tokens_per_wg):
    gen = torch.Generator().manual_seed(T)
    o = torch.randn(B, T, 8, 64, generator=gen).to(torch.bfloat16)
    wide = torch.randn(B, T, 1024, generator=gen).to(torch.bfloat16).to(device)
    g = wide[..., 256:768].unflatten(-1, (8, 64))                               # a strided view, read in place
    nw = (torch.rand(64, generator=gen) + 0.5).to(torch.bfloat16)
    W = (torch.randn(128, 512, generator=gen) * 0.05).to(torch.bfloat16)
    y = lo.norm_proj(o.to(device), g, nw.to(device), W.to(device), 1e-6, tokens_per_wg)
    assert y.shape == (B, T, 128) and y.dtype == torch.bfloat16
    normed, _ = ol.rms_norm(_f64(o), _f64(g), _f64(nw), eps=1e-6, activation="swish")
    normed_b = torch.from_numpy(normed).to(torch.bfloat16)                     # the rounding the kernel applies
    want = _f64(normed_b).reshape(B, T, 512) @ _f64(W).T
    err = np.abs(_f64(y) - want)
    # one bf16 rounding of the result plus last-bit differences of the rounded normalised tensor (512 terms)
    assert np.all(err <= 2 ** -7 * np.abs(want) + 2e-2), float(err.max())
    assert err.mean() < 3e-3
    two_step = torch.nn.functional.linear(lo.rms_norm_gated(o.to(device), g, nw.to(device), None, "swish", eps=1e-6)
                                          .reshape(B, T, 512), W.to(device))
    assert (y.float() - two_step.float()).abs().max() < 0.06 and (y.float() - two_step.float()).abs().mean() < 3e-3
    # with the residual add and the next pre-norm applied in the same kernel
    res = torch.randn(B, T, 128, generator=gen).to(torch.bfloat16)
    nxt = (torch.rand(128, generator=gen) + 0.5).to(torch.bfloat16)
    h, r = lo.norm_proj(o.to(device), g, nw.to(device), W.to(device), 1e-6, tokens_per_wg, residual=res.to(device),
                        next_norm_weight=nxt.to(device), next_eps=1e-6)
    y_b = _f64(torch.from_numpy(want).to(torch.bfloat16))                        # the projection as the kernel rounds it
    want_h, want_r = ol.rms_norm(y_b, None, _f64(nxt), residual=_f64(res), eps=1e-6)
    assert h.shape == (B, T, 128) and r.dtype == torch.bfloat16
    err_r, err_h = np.abs(_f64(r) - want_r), np.abs(_f64(h) - want_h)
    assert np.all(err_r <= 2 ** -7 * np.abs(want_r) + 3e-2) and err_r.mean() < 4e-3
    assert np.all(err_h <= 2 ** -6 * np.abs(want_h) + 3e-2) and err_h.mean() < 4e-3
    h2, r2 = lo.rms_norm(y, nxt.to(device), None, residual=res.to(device), eps=1e-6, prenorm=True)   # two-step route
    assert (r.float() - r2.float()).abs().max() < 0.04 and (h.float() - h2.float()).abs().max() < 0.06


def test_short_convolution_module_cache_and_step(device):
    torch.manual_seed(4)
    D, W, T = 64, 4, 19
    conv = lo.ShortConvolution(D, W, bias=True, activation="silu").to(device)
    x = torch.randn(2, T, D, device=device)
    y, cache = conv(x, output_final_state=True)
    w, b = _f64(conv.weight).reshape(D, W), _f64(conv.bias)
    _close(y, ol.causal_conv1d(_f64(x), w, b, activation="silu"), torch.float32)
    assert cache.shape == (2, D, W) and np.array_equal(_f64(cache), ol.conv_final_state(_f64(x), W))
    # decoding one token at a time from an empty cache reproduces the full forward
    state = torch.zeros(2, D, W, device=device)
    steps = [conv(x[:, t:t + 1], cache=state)[0] for t in range(T)]
    _close(torch.cat(steps, 1), ol.causal_conv1d(_f64(x), w, b, activation="silu"), torch.float32)
    assert torch.equal(state, cache)
    # packed sequences: final state per sequence
    cu = torch.tensor([0, 2, 2, 19], device=device)
    yv, cv = conv(x[:1], output_final_state=True, cu_seqlens=cu)
    _close(yv, ol.causal_conv1d(_f64(x[:1]), w, b, activation="silu", cu_seqlens=cu.cpu().numpy()), torch.float32)
    assert np.array_equal(_f64(cv), ol.conv_final_state(_f64(x[:1]), W, cu.cpu().numpy()))
    with pytest.raises(ValueError):
        conv(x[:1], mask=torch.ones(1, T, device=device), cu_seqlens=cu)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 5, 8, 64), (2, 100, 4, 128), (3, 7, 1, 8), (1, 9, 2, 1000), (1, 3, 1, 2048)])
def test_rms_norm_gated_and_plain(device, dtype, shape):
    gen = torch.Generator().manual_seed(sum(shape))
    D = shape[-1]
    x, g = torch.randn(shape, generator=gen).to(dtype), torch.randn(shape, generator=gen).to(dtype)
    w, b = (torch.rand(D, generator=gen) + 0.5).to(dtype), torch.randn(D, generator=gen).to(dtype)
    res = torch.randn(shape, generator=gen).to(dtype)
    for act in ("swish", "sigmoid"):
        got = lo.rms_norm_gated(x.to(device), g.to(device), w.to(device), None, act, eps=1e-6)
        _close(got, ol.rms_norm(_f64(x), _f64(g), _f64(w), eps=1e-6, activation=act)[0], dtype)
    got, res_out = lo.rms_norm(x.to(device), w.to(device), b.to(device), residual=res.to(device), eps=1e-5, prenorm=True)
    want, s = ol.rms_norm(_f64(x), None, _f64(w), _f64(b), residual=_f64(res), eps=1e-5)
    _close(got, want, dtype)
    _close(res_out, s, dtype)
    assert res_out.dtype == dtype
    # fp32 residual stream next to low-precision activations
    got, res_out = lo.rms_norm(x.to(device), w.to(device), None, residual=res.float().to(device), prenorm=True)
    want, s = ol.rms_norm(_f64(x), None, _f64(w), residual=_f64(res), eps=1e-5)
    _close(got, want, dtype)
    _close(res_out, s, torch.float32)
    assert res_out.dtype == torch.float32
    y, r32 = lo.rms_norm(x.to(device), None, None, prenorm=True, residual_in_fp32=True)
    assert r32.dtype == torch.float32 and torch.equal(r32, x.float().to(device))
    _close(y, ol.rms_norm(_f64(x), eps=1e-5)[0], dtype)


def test_norm_modules_and_errors(device):
    torch.manual_seed(5)
    o, g = torch.randn(1, 60000, 8, 64, device=device).bfloat16(), torch.randn(1, 60000, 8, 64, device=device).bfloat16()
    norm = lo.FusedRMSNormSwishGate(64, eps=1e-6).to(device)
    with torch.no_grad():
        norm.weight.copy_(torch.rand(64) + 0.5)
    y = norm(o, g)
    assert y.shape == o.shape and y.dtype == torch.bfloat16
    _close(y, ol.rms_norm(_f64(o), _f64(g), _f64(norm.weight), eps=1e-6)[0], torch.bfloat16)
    plain = lo.RMSNorm(64, eps=1e-6).to(device)
    h, r = plain(o, o, True)
    want, s = ol.rms_norm(_f64(o), residual=_f64(o), weight=_f64(plain.weight), eps=1e-6)
    _close(h, want, torch.bfloat16)
    _close(r, s, torch.bfloat16)
    with pytest.raises(ValueError):
        lo.FusedRMSNormGated(64, activation="relu")
    with pytest.raises(_capi_error()):
        lo.rms_norm(torch.randn(4, 12, device=device), None, None)          # 12 channels: not a multiple of 8
    with pytest.raises(_capi_error()):
        lo.rms_norm(torch.randn(4, 64), None, None)                         # CPU tensor: no fallback


def _capi_error():
    from lampa_amd._capi import LampaError
    return LampaError
