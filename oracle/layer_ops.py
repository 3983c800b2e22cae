"""CPU oracle for the operators around the gated-delta forward (TEST INFRASTRUCTURE ONLY): the depthwise causal short
convolution and the (gated) RMS norm, in float64 numpy.

Reference lines restated: ``models/hattention/short_convolution.py:39-99`` (taps, bias, SiLU, residual, sequence
starts) and ``:478-498`` (final state of packed sequences); ``models/hattention/fused_norm.py:40-111`` (residual add,
rstd, weight, bias, swish / sigmoid gate). Pinned in ``tests/test_oracle_layer_ops.py`` against ``F.conv1d``,
``F.rms_norm``, ``F.silu``, impulse responses and scale invariance.
"""
import numpy as np


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def causal_conv1d(x, weight, bias=None, residual=None, activation=None, cu_seqlens=None):
    """x [B, T, D], weight [D, W]: y[t] = act(bias + sum_j weight[:, j] * x[t - (W-1) + j]) + residual, taps before the
    start of the token's sequence are zero. ``cu_seqlens`` (B == 1) packs several sequences along T."""
    x = np.asarray(x, np.float64)
    weight = np.asarray(weight, np.float64)
    B, T, D = x.shape
    W = weight.shape[1]
    if cu_seqlens is None:
        start = np.zeros((B, T), np.int64)
    else:
        cu = np.asarray(cu_seqlens, np.int64)
        start = np.zeros((1, T), np.int64)
        for s in range(len(cu) - 1):
            start[0, cu[s]:cu[s + 1]] = cu[s]
    t_idx = np.arange(T)[None, :]
    y = np.zeros_like(x)
    for j in range(W):
        src = t_idx - (W - 1) + j                                   # [1, T]
        ok = src >= start                                           # [B, T]
        gathered = np.take_along_axis(x, np.broadcast_to(np.clip(src, 0, None), (B, T))[..., None], axis=1)
        y += np.where(ok[..., None], gathered, 0.0) * weight[None, None, :, j]
    if bias is not None:
        y += np.asarray(bias, np.float64)
    if activation in ("silu", "swish"):
        y = y * _sigmoid(y)
    elif activation is not None:
        raise ValueError(activation)
    if residual is not None:
        y += np.asarray(residual, np.float64)
    return y


def conv_final_state(x, W, cu_seqlens=None):
    """Cache of the last W inputs per sequence, [N, D, W], zero where the sequence is shorter than W."""
    x = np.asarray(x, np.float64)
    B, T, D = x.shape
    bounds = [(b * T, (b + 1) * T) for b in range(B)] if cu_seqlens is None else \
        [(int(cu_seqlens[s]), int(cu_seqlens[s + 1])) for s in range(len(cu_seqlens) - 1)]
    flat = x.reshape(B * T, D)
    out = np.zeros((len(bounds), D, W))
    for n, (bos, eos) in enumerate(bounds):
        for w in range(W):
            t = eos - W + w
            if t >= bos:
                out[n, :, w] = flat[t]
    return out


def rms_norm(x, g=None, weight=None, bias=None, residual=None, eps=1e-5, activation="swish"):
    """Returns (y, x + residual). The norm runs over the last dimension."""
    s = np.asarray(x, np.float64)
    if residual is not None:
        s = s + np.asarray(residual, np.float64)
    rstd = 1.0 / np.sqrt((s * s).mean(-1, keepdims=True) + eps)
    y = s * rstd
    if weight is not None:
        y = y * np.asarray(weight, np.float64)
    if bias is not None:
        y = y + np.asarray(bias, np.float64)
    if g is not None:
        g = np.asarray(g, np.float64)
        if activation in ("swish", "silu"):
            y = y * g * _sigmoid(g)
        elif activation == "sigmoid":
            y = y * _sigmoid(g)
        else:
            raise ValueError(activation)
    return y, s
