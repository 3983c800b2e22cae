"""CPU oracle of a gated-delta layer and of the `lshgd`-style block (TEST INFRASTRUCTURE ONLY), float64 between the
operators, built from the other oracle modules: LSH bucket sort (``oracle.lsh``), short convolution and RMS norm
(``oracle.layer_ops``), token-serial gated delta (``oracle.gated_delta.recurrent_c``, float64 state).

Reference lines restated: ``models/hattention/modeling_gated_deltaproduct.py:505-625`` (one householder step:
projections, convolutions with SiLU, beta = sigmoid, g = -exp(A_log) softplus(a + dt_bias), l2-normalised gated delta,
swish-gated RMS norm, output projection) and ``:1029-1056`` (pre-norm residual wiring). Every piece is pinned in its own
module's tests; this file only composes them, so its own checks are about the wiring (``tests/test_oracle_block.py``).
"""
import numpy as np
import torch

from . import gated_delta as og
from . import layer_ops as ol
from . import lsh as olsh


def _softplus(x):
    return np.where(x > 20.0, x, np.log1p(np.exp(np.minimum(x, 20.0))))


def gates(a, b, A_log, dt_bias, beta_scale=1.0):
    g = -np.exp(np.asarray(A_log, np.float64)) * _softplus(np.asarray(a, np.float64) + np.asarray(dt_bias, np.float64))
    beta = beta_scale / (1.0 + np.exp(-np.asarray(b, np.float64)))
    return g, beta


def gated_delta_layer(p, prefix, x, num_heads, head_dim, eps=1e-6, cu_seqlens=None):
    """x [1, T, hidden] float64; p maps parameter names to float64 arrays. Returns [1, T, hidden]."""
    w = lambda name: p[prefix + name]
    T = x.shape[1]
    H, dk = num_heads, head_dim
    proj = lambda name: x @ w(name + ".weight").T
    conv = lambda name, t: ol.causal_conv1d(t, w(name + ".weight").reshape(t.shape[-1], -1), None, None, "silu", cu_seqlens)
    q, k, v = conv("q_conv1d", proj("q_proj")), conv("k_conv1d", proj("k_proj")), conv("v_conv1d", proj("v_proj"))
    dv = v.shape[-1] // H
    g, beta = gates(proj("a_proj"), proj("b_proj"), w("A_log"), w("dt_bias"))
    t = lambda a, d: torch.from_numpy(np.ascontiguousarray(a.reshape(1, T, H, d)))
    o, _ = og.recurrent_c(t(q, dk), t(k, dk), t(v, dv), torch.from_numpy(g), torch.from_numpy(beta),
                          cu_seqlens=cu_seqlens, l2=og.L2_CHUNK, dtype=torch.float64)
    gate = proj("g_proj").reshape(1, T, H, dv)
    o, _ = ol.rms_norm(o.double().numpy(), gate, w("o_norm.weight"), eps=eps, activation="swish")
    return o.reshape(1, T, H * dv) @ w("o_proj.weight").T


def lshgd_block(p, feats, coords, n_layers, num_heads, head_dim, n_tables, n_proj, bucket_width):
    """feats [N, in], coords [N, c] -> [N, out] float64, in the input hit order."""
    perm = olsh.bucket_sort(np.asarray(coords, np.float32), p["lsh_alpha"].astype(np.float32),
                            p["lsh_beta"].astype(np.float32), bucket_width, n_tables, n_proj)["perm"][0]
    x = np.asarray(feats, np.float64) @ p["input.weight"].T + p["input.bias"]
    x = x[perm][None]
    residual = None
    for i in range(n_layers):
        h, residual = ol.rms_norm(x, weight=p[f"norms.{i}.weight"], residual=residual, eps=1e-6)
        x = gated_delta_layer(p, f"layers.{i}.", h, num_heads, head_dim)
    h, _ = ol.rms_norm(x, weight=p["norm_f.weight"], residual=residual, eps=1e-6)
    out = np.empty_like(h[0])
    out[perm] = h[0]
    return out @ p["head.weight"].T + p["head.bias"]
