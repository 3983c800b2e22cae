"""Pins for the LSH oracle: library routines (torch.bmm, torch.sort(stable=True), torch.gather), float64
evaluation away from bucket edges, Python-integer packing and brute-force sorting."""
import numpy as np
import torch

from lampa_amd import synth
from oracle import lsh as ol


def _event(n=5000, seed=0):
    coords, feats, _ = synth.collider_event(n, seed)
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    return coords.numpy(), feats.numpy(), alpha.numpy(), beta.numpy()


def test_projection_matches_bmm_and_float64():
    coords, _, alpha, _ = _event()
    proj = ol.project(coords, alpha)
    bmm = torch.bmm(torch.from_numpy(coords)[None], torch.from_numpy(alpha)[None])[0].T.numpy()
    exact = (coords.astype(np.float64) @ alpha.astype(np.float64)).T
    assert np.abs(proj - exact).max() < 2e-6
    assert np.abs(proj - bmm).max() < 2e-6
    # a single-term projection is the plain product
    one = ol.project(coords[:, :1].copy(), alpha[:1].copy())
    assert np.array_equal(one, (coords[:, :1] * alpha[:1]).T)


def test_bucket_ids_match_float64_floor_away_from_edges():
    coords, _, alpha, beta = _event()
    w = 0.5
    ids = ol.bucket_ids(coords, alpha, beta, w)
    t = (coords.astype(np.float64) @ alpha.astype(np.float64) + beta.astype(np.float64)).T / w
    safe = np.abs(t - np.round(t)) > 1e-4  # not within rounding distance of a bucket edge
    assert safe.mean() > 0.999
    assert np.array_equal(ids[safe], np.floor(t[safe]).astype(np.int32))
    # and how many ids differ from a plain torch evaluation of the same formula (expected: a handful)
    tb = torch.floor((torch.from_numpy(coords) @ torch.from_numpy(alpha) + torch.from_numpy(beta)) / w).T.int().numpy()
    assert (ids != tb).mean() < 1e-3


def test_bucket_ids_saturate_and_nan():
    coords = np.array([[1e30, 0, 0, 0], [-1e30, 0, 0, 0], [np.nan, 0, 0, 0], [0.26, 0, 0, 0]], np.float32)
    alpha = np.zeros((4, 1), np.float32)
    alpha[0, 0] = 1.0
    ids = ol.bucket_ids(coords, alpha, np.zeros(1, np.float32), 0.5)
    assert ids.tolist() == [[2**31 - 1, -(2**31), 2**31 - 1, 0]]


def test_pack_keys_against_python_integers():
    rng = np.random.default_rng(0)
    T, J, N = 3, 4, 1000
    ids = rng.integers(-20, 25, size=(T * J, N)).astype(np.int32)
    keys, meta = ol.pack_keys(ids, T, J)
    for t in range(T):
        lo = [int(ids[t * J + j].min()) for j in range(J)]
        rg = [int(ids[t * J + j].max()) - lo[j] + 1 for j in range(J)]
        stride, total = [], 1
        for j in range(J):
            stride.append(total)
            total *= rg[j]
        want = [sum((int(ids[t * J + j, n]) - lo[j]) * stride[j] for j in range(J)) for n in range(N)]
        assert keys[t].tolist() == want
        assert meta[t].tolist() == lo + rg + [total, max(1, (total - 1).bit_length()), 0]
    # keys order lexicographically with the LAST projection most significant
    order = np.lexsort([ids[j] for j in range(J)])  # lexsort: last key is primary
    assert np.array_equal(ol.stable_argsort(keys[:1], ol.KEY_I32)[0], order.astype(np.int32))


def test_pack_keys_padding_and_overflow():
    ids = np.array([[0, 3, 1, 99], [5, 5, 6, 99]], np.int32)  # T=1, J=2, N=4, last hit is padding
    keys, meta = ol.pack_keys(ids, 1, 2, n_valid=3)
    assert meta[0].tolist() == [0, 5, 4, 2, 8, 4, 0]  # total 8 is also the padding key -> 4 bits
    assert keys[0].tolist() == [0, 3, 1 + 4, 8]
    big = np.array([[0, 70000], [0, 70000]], np.int32)
    _, meta = ol.pack_keys(big, 1, 2)
    assert meta[0, -1] == 1 and meta[0, -2] == 32 and meta[0, -3] == 2**31 - 1


def test_stable_argsort_against_torch_and_sorted():
    rng = np.random.default_rng(1)
    keys = rng.integers(-50, 50, size=(3, 4096)).astype(np.int32)  # many ties
    perm, kout = ol.stable_argsort(keys, ol.KEY_I32, return_keys=True)
    want = torch.sort(torch.from_numpy(keys), dim=-1, stable=True)
    assert np.array_equal(perm, want.indices.numpy().astype(np.int32))
    assert np.array_equal(kout, want.values.numpy())
    for s in range(3):
        assert perm[s].tolist() == sorted(range(4096), key=lambda i: keys[s, i])
    # float keys incl. -0.0/+0.0 ties, infinities and NaN (NaN last, as torch.sort)
    f = rng.standard_normal((2, 3000)).astype(np.float32)
    f[0, :40] = 0.0
    f[0, 40:80] = -0.0
    f[1, 5], f[1, 17], f[1, 900], f[1, 901] = np.inf, -np.inf, np.nan, np.nan
    perm = ol.stable_argsort(f, ol.KEY_F32)
    want = torch.sort(torch.from_numpy(f), dim=-1, stable=True).indices.numpy()
    assert np.array_equal(perm, want.astype(np.int32))
    u = rng.integers(0, 2**32, size=(1, 2000), dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(ol.stable_argsort(u, ol.KEY_U32)[0], np.argsort(u[0], kind="stable").astype(np.int32))
    # payload values ride along
    vals = rng.permutation(2000).astype(np.int32)[None]
    assert np.array_equal(ol.stable_argsort(u, ol.KEY_U32, vals=vals)[0], vals[0][np.argsort(u[0], kind="stable")])


def test_gather_scatter_invert():
    rng = np.random.default_rng(2)
    feats = rng.standard_normal((500, 24)).astype(np.float32)
    perm = np.stack([rng.permutation(500) for _ in range(3)]).astype(np.int32)
    g = ol.gather_rows(feats, perm)
    tg = torch.from_numpy(feats)[None].expand(3, -1, -1).gather(1, torch.from_numpy(perm).long()[..., None].expand(-1, -1, 24))
    assert np.array_equal(g, tg.numpy())
    inv = ol.invert_perm(perm)
    assert np.array_equal(inv, np.argsort(perm, axis=-1).astype(np.int32))
    assert np.array_equal(ol.scatter_rows(g, perm), np.broadcast_to(feats, (3, 500, 24)))
    assert np.array_equal(ol.gather_rows(g, inv), np.broadcast_to(feats, (3, 500, 24)))


def test_lsh_ordering_against_torch_restating_reference_lines():
    # full_mamba2.py:181-208 evaluated with torch on the CPU: key = sum_h proj_h 2^h, argsort(norm), stable sort.
    coords, _, _, _ = _event(3000)
    gen = torch.Generator().manual_seed(5)
    alpha = torch.normal(0.0, 1.0, (1, 4, 3), generator=gen)
    c = torch.from_numpy(coords)
    proj = torch.bmm(c[None], alpha).permute(2, 1, 0)           # (H, N, 1)
    scores = proj.sum(-1)                                        # shift == 0 for a single head
    bucket_matrix = scores.view(3, 1, -1).permute(1, 2, 0)
    keys = (bucket_matrix * torch.tensor([1, 2, 4])).sum(-1)[0]
    norm_idx = c.norm(dim=1).argsort(stable=True)
    _, bk = keys[norm_idx].sort(stable=True)
    want = norm_idx[bk].numpy()
    got = ol.lsh_ordering(coords, alpha[0].numpy())
    # fp32 summation order inside torch may differ in the last bit; orders agree except at near-ties
    assert (got != want).mean() < 2e-3
    key, norm = ol.lsh_ordering_keys(coords, alpha[0].numpy())
    assert np.abs(key - keys.numpy()).max() < 1e-5 and np.abs(norm - c.norm(dim=1).numpy()).max() < 1e-6
    assert np.all(np.diff(key[got]) >= 0)


def test_config1_pipeline_properties():
    coords, feats, alpha, beta = _event(60000)
    out = ol.bucket_sort(coords, alpha, beta, 0.5, 3, 4, feats)
    assert out["meta"][:, -1].max() == 0 and out["meta"][:, -2].max() <= 31
    for t in range(3):
        k = out["keys"][t][out["perm"][t]]
        assert np.all(np.diff(k) >= 0)
        ties = np.diff(k) == 0
        assert np.all(np.diff(out["perm"][t])[ties] > 0)  # stability: equal keys keep input order
        assert np.array_equal(np.sort(out["perm"][t]), np.arange(60000))
        assert np.array_equal(out["feats"][t], feats[out["perm"][t]])


# ------------------------------------------------------------------------------- HEPT region (AND-hash) front end
def test_quantile_regions_against_python_integers_and_invariants():
    rng = np.random.default_rng(3)
    n = 1003
    coord = rng.permutation(n).astype(np.float64)            # distinct values: the rank is a plain count
    order = np.argsort(coord, kind="stable")
    regions = np.array([1.0, 2.0, 7.0, 10.0, 3 + 1 / 3, 6 + 2 / 3, 1003.0, 5000.0], np.float32)
    got = ol.quantile_regions(order, regions)
    assert got.shape == (len(regions), n) and got.dtype == np.float32
    for r, reg in enumerate(regions):
        # exact integer restatement: hits with a smaller coordinate // ceil(N / regions) + 1; the rational N / regions
        # is taken on the float32 value actually stored (thirds are not exact) and is far from an integer here
        from fractions import Fraction
        size = -((-Fraction(n)) // Fraction(float(reg)))      # ceil
        want = [int(sum(coord < c)) // int(size) + 1 for c in coord]
        assert got[r].tolist() == [float(w) for w in want], reg
        # invariants: 1-based, monotone along the coordinate, every region but the last holds exactly `size` hits
        along = got[r][order]
        assert along[0] == 1 and np.all(np.diff(along) >= 0) and np.all(np.diff(along) <= 1)
        counts = np.bincount(got[r].astype(np.int64))[1:]
        assert np.all(counts[:-1] == int(size)) and 0 < counts[-1] <= int(size)
    # a rank array that is not the identity: the region follows the hit, not the position
    assert not np.array_equal(got[2], got[2][order])


def test_geo_shift_orders_lexicographically_by_phi_region_eta_region_hash():
    # With integer-valued inputs every float32 operation is exact, so the key must equal the Python-integer
    # mixed-radix value, and sorting by it must equal a lexicographic sort on (phi region, eta region, hash).
    rng = np.random.default_rng(4)
    rows, n = 3, 500
    regions_eta = np.array([2.0, 3 + 1 / 3, 5.0], np.float32)     # ceil -> 2, 4, 5 eta regions at most
    reg_eta = np.stack([rng.integers(1, int(np.ceil(r)) + 1, n) for r in regions_eta]).astype(np.float32)
    reg_phi = rng.integers(1, 5, (rows, n)).astype(np.float32)
    hashed = rng.integers(-40, 41, (rows, n)).astype(np.float32)
    shift = np.array([81.0, 90.0, 200.0], np.float32)             # strictly above the hash range: no boundary ties
    got = ol.geo_shift(regions_eta, shift, reg_eta, reg_phi)
    for r in range(rows):
        mult = int(np.ceil(regions_eta[r])) + 1
        want = [int(p) * int(shift[r]) * mult + int(e) * int(shift[r]) for e, p in zip(reg_eta[r], reg_phi[r])]
        assert got[r].tolist() == [float(w) for w in want]
        key = hashed[r] + got[r]
        order = np.argsort(key, kind="stable")
        lex = np.lexsort((np.arange(n), hashed[r], reg_eta[r], reg_phi[r]))
        assert np.array_equal(order, lex)
    # asymmetry pins the operand roles: swapping eta and phi regions changes the result
    assert not np.array_equal(got, ol.geo_shift(regions_eta, shift, reg_phi, reg_eta))


def test_hept_sort_keys_padding_and_composition():
    rng = np.random.default_rng(5)
    rows, n, n_raw = 4, 300, 257
    eta, phi = rng.normal(size=n), rng.uniform(-3, 3, n)
    eta[n_raw:], phi[n_raw:] = np.inf, np.inf
    s_eta, s_phi = np.argsort(eta, kind="stable"), np.argsort(phi, kind="stable")
    regions = np.array([[2.0, 3.0, 4 + 1 / 3, 6.0], [5.0, 3 + 2 / 3, 3.0, 2.0]], np.float32)
    hashed = rng.normal(size=(rows, n)).astype(np.float32)
    shift = (hashed.max(1) - hashed.min(1)).astype(np.float32)
    keys = ol.hept_sort_keys(hashed, s_eta, s_phi, regions, shift, n_raw)
    assert np.all(np.isinf(keys[:, n_raw:])) and np.all(np.isfinite(keys[:, :n_raw]))
    # padded hits sort last and keep their order; real hits of a lower (phi, eta) region pair never follow a higher one
    reg_eta, reg_phi = ol.quantile_regions(s_eta, regions[0]), ol.quantile_regions(s_phi, regions[1])
    for r in range(rows):
        order = np.argsort(keys[r], kind="stable")
        assert np.array_equal(order[n_raw:], np.arange(n_raw, n))
        pair = reg_phi[r][order[:n_raw]] * 100 + reg_eta[r][order[:n_raw]]
        # float rounding can only swap neighbours at a region boundary whose hashes sit at opposite ends of the range
        assert np.mean(np.diff(pair) < 0) < 0.02
    # the input hashes are not modified
    assert np.all(np.isfinite(hashed))


def test_prep_qk_distance_identity_and_column_roles():
    # The appended columns turn a weighted coordinate distance into part of the Euclidean one:
    # |q_hat_i - k_hat_j|^2 = |q_i - k_j|^2 + sum_c 2 qw'[h, c] (coords_i,c - coords_j,c)^2, qw' = [qw_0, qw_0, qw_1, ...].
    rng = np.random.default_rng(6)
    n, H, d, R, K = 9, 3, 5, 2, 4
    q, k = rng.normal(size=(n, H, d)), rng.normal(size=(n, H, d))
    w, coords = rng.normal(size=(H, d, R, K)) * 0.3, rng.normal(size=(n, R + 1))
    q_hat, k_hat = ol.prep_qk(q, k, w, coords)
    assert q_hat.shape == (n, H, d + R + 1) and np.array_equal(q_hat[..., :d], q) and np.array_equal(k_hat[..., :d], k)
    wt = torch.from_numpy(w)
    qw = wt.sum(dim=1).clamp(max=50).exp().sum(dim=-1).numpy()                   # library evaluation, [H, R]
    qwx = np.concatenate([qw[:, :1], qw], axis=1)
    for h in range(H):
        lhs = ((q_hat[:, None, h] - k_hat[None, :, h]) ** 2).sum(-1)
        rhs = ((q[:, None, h] - k[None, :, h]) ** 2).sum(-1) + \
            (2 * qwx[h] * (coords[:, None] - coords[None]) ** 2).sum(-1)
        assert np.abs(lhs - rhs).max() < 1e-10
    # the clamp: a huge weight sum saturates at exp(50) instead of overflowing
    w_big = w.copy()
    w_big[0, :, 1, 2] = 100.0
    big, _ = ol.prep_qk(q, k, w_big, coords)
    assert np.all(np.isfinite(big)) and big[0, 0, d + 2] != q_hat[0, 0, d + 2]
    assert np.array_equal(big[:, 1:], q_hat[:, 1:])                              # other heads untouched
