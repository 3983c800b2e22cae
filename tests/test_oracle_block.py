"""Wiring checks of the block oracle (its operators are pinned in their own test modules)."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import block as ob


def test_gates_match_library_softplus_and_sigmoid():
    rng = np.random.default_rng(0)
    a, b = rng.normal(size=(50, 8)) * 10, rng.normal(size=(50, 8)) * 3
    A_log, dt = rng.normal(size=8), rng.normal(size=8)
    g, beta = ob.gates(a, b, A_log, dt, 2.0)
    want_g = -torch.from_numpy(A_log).exp() * F.softplus(torch.from_numpy(a) + torch.from_numpy(dt))
    assert np.abs(g - want_g.numpy()).max() < 1e-12 and np.all(g <= 0)
    assert np.abs(beta - 2 * torch.sigmoid(torch.from_numpy(b)).numpy()).max() < 1e-12


def _params(rng, hidden, H, d, n_layers, in_dim, out_dim, coord_dim, n_cols):
    p = {"input.weight": rng.normal(size=(hidden, in_dim)) * 0.3, "input.bias": rng.normal(size=hidden) * 0.1,
         "head.weight": rng.normal(size=(out_dim, hidden)) * 0.3, "head.bias": rng.normal(size=out_dim) * 0.1,
         "norm_f.weight": np.ones(hidden), "lsh_alpha": rng.normal(size=(coord_dim, n_cols)),
         "lsh_beta": rng.uniform(0, 0.5, n_cols)}
    for i in range(n_layers):
        p[f"norms.{i}.weight"] = np.ones(hidden)
        pre = f"layers.{i}."
        for name, rows in (("q_proj", H * d), ("k_proj", H * d), ("v_proj", H * d), ("g_proj", H * d), ("b_proj", H),
                           ("a_proj", H)):
            p[pre + name + ".weight"] = rng.normal(size=(rows, hidden)) * 0.3
        for name in ("q_conv1d", "k_conv1d", "v_conv1d"):
            p[pre + name + ".weight"] = rng.normal(size=(H * d, 1, 4)) * 0.5
        p[pre + "A_log"], p[pre + "dt_bias"] = np.log(rng.uniform(0.5, 8, H)), rng.normal(size=H)
        p[pre + "o_norm.weight"] = np.ones(d)
        p[pre + "o_proj.weight"] = rng.normal(size=(hidden, H * d)) * 0.2
    return p


def test_block_wiring_order_equivariance_and_causality():
    rng = np.random.default_rng(1)
    hidden, H, d, L, N = 16, 2, 8, 2, 150
    p = _params(rng, hidden, H, d, L, 6, 5, 4, 12)
    feats, coords = rng.normal(size=(N, 6)), rng.normal(size=(N, 4)).astype(np.float32)
    out = ob.lshgd_block(p, feats, coords, L, H, d, 3, 4, 0.5)
    assert out.shape == (N, 5) and np.all(np.isfinite(out))
    # the block sorts the hits itself, so shuffling the input hits shuffles the output rows the same way -- except
    # that hits with equal bucket keys keep their input order; distinct keys here make the order unique
    from oracle import lsh as olsh
    keys = olsh.bucket_sort(coords, p["lsh_alpha"].astype(np.float32), p["lsh_beta"].astype(np.float32), 0.5, 3, 4)["keys"][0]
    if len(np.unique(keys)) == N:
        sh = rng.permutation(N)
        out_sh = ob.lshgd_block(p, feats[sh], coords[sh], L, H, d, 3, 4, 0.5)
        assert np.abs(out_sh - out[sh]).max() < 1e-9
    # causality in the LSH order: changing the features of the last hit of the order changes no other row
    perm = olsh.bucket_sort(coords, p["lsh_alpha"].astype(np.float32), p["lsh_beta"].astype(np.float32), 0.5, 3, 4)["perm"][0]
    f2 = feats.copy()
    f2[perm[-1]] += 1.0
    out2 = ob.lshgd_block(p, f2, coords, L, H, d, 3, 4, 0.5)
    others = np.ones(N, bool)
    others[perm[-1]] = False
    assert np.abs(out2[others] - out[others]).max() < 1e-12 and np.abs(out2[perm[-1]] - out[perm[-1]]).max() > 1e-6
    # and changing the first hit of the order changes the hits after it: the convolution reaches 3 tokens, the state
    # carries it further (with these strong decays it fades within tens of tokens)
    f3 = feats.copy()
    f3[perm[0]] += 1.0
    out3 = ob.lshgd_block(p, f3, coords, L, H, d, 3, 4, 0.5)
    assert np.abs(out3[perm[2]] - out[perm[2]]).max() > 1e-3 and np.abs(out3[perm[8]] - out[perm[8]]).max() > 1e-9


def test_layer_is_a_residual_free_map_with_zero_output_projection():
    rng = np.random.default_rng(2)
    hidden, H, d = 16, 2, 8
    p = _params(rng, hidden, H, d, 1, 6, 5, 4, 12)
    x = rng.normal(size=(1, 40, hidden))
    y = ob.gated_delta_layer(p, "layers.0.", x, H, d)
    assert y.shape == x.shape
    p["layers.0.o_proj.weight"][:] = 0
    assert np.all(ob.gated_delta_layer(p, "layers.0.", x, H, d) == 0)
