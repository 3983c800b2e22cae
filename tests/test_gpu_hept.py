"""GPU parity of the HEPT region (AND-hash) front end against the CPU oracle: bit-exact regions, shifts, keys and
bucket positions."""
import numpy as np
import pytest
import torch

from lampa_amd import hept, lsh, synth
from oracle import lsh as ol

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _regions(n_hashes=3, n_heads=8, num_regions=140, seed=6):
    torch.manual_seed(seed)
    regions = hept.get_regions(num_regions, n_hashes, n_heads)          # [c, a, h]
    c, a, h = regions.shape
    return regions, regions.permute(1, 0, 2).reshape(a, c * h).contiguous()


def test_get_regions_shape_and_product():
    regions, regions_h = _regions()
    assert regions.shape == (3, 2, 8) and regions_h.shape == (2, 24)
    assert torch.allclose(regions * 3, torch.round(regions * 3))        # multiples of one third
    prod = regions_h[0] * regions_h[1]
    assert (prod > 0.6 * 140).all() and (prod < 1.6 * 140).all()        # the factors multiply to about num_regions


@pytest.mark.parametrize("n", [1, 5, 1023, 60000])
def test_quantile_partition_and_geo_shift_bit_exact(device, n):
    _, regions_h = _regions()
    coords = synth.collider_event(n, seed=1)[0]
    s_eta = torch.sort(coords[:, 0], stable=True).indices
    s_phi = torch.sort(coords[:, 1], stable=True).indices
    got_eta = hept.quantile_partition(s_eta.to(device), regions_h[0][:, None].to(device))
    got_phi = hept.quantile_partition(s_phi.to(device).int(), regions_h[1])          # int32 ranks, CPU regions
    want_eta = ol.quantile_regions(s_eta.numpy(), regions_h[0].numpy())
    want_phi = ol.quantile_regions(s_phi.numpy(), regions_h[1].numpy())
    assert got_eta.shape == (24, n) and got_eta.dtype == torch.float32
    assert np.array_equal(_np(got_eta), want_eta) and np.array_equal(_np(got_phi), want_phi)
    gen = torch.Generator().manual_seed(2)
    shift = torch.rand(24, 1, generator=gen) * 7 + 0.1
    got = hept.get_geo_shift(regions_h.to(device), shift.to(device), (got_eta, got_phi), 3)
    want = ol.geo_shift(regions_h[0].numpy(), shift.numpy(), want_eta, want_phi)
    assert got.shape == (2, 3, 8, n)
    assert np.array_equal(_np(got[0]).reshape(24, n), want) and torch.equal(got[0], got[1])


@pytest.mark.parametrize("n,n_raw", [(7, 7), (4100, 4001), (60100, 60000)])
def test_hept_sort_keys_and_positions_bit_exact(device, n, n_raw):
    _, regions_h = _regions()
    torch.manual_seed(8)
    e = lsh.E2LSH(n_hashes=3, n_heads=8, dim=6).to(device)
    coords = torch.full((n, 2), float("inf"))
    coords[:n_raw] = synth.collider_event(n_raw, seed=2)[0][:, :2]
    s_eta = torch.sort(coords[:, 0], stable=True).indices
    s_phi = torch.sort(coords[:, 1], stable=True).indices
    rank_eta = lsh.invert_permutation(s_eta.to(device)).int()
    rank_phi = lsh.invert_permutation(s_phi.to(device)).int()
    q_hat, k_hat = torch.randn(8, n, 6), torch.randn(8, n, 6)
    q_hat[:, n_raw:], k_hat[:, n_raw:] = 0.0, 0.0                       # hept.py:126-128
    qh, kh, shift = lsh.lsh_mapping(e, q_hat.to(device), k_hat.to(device))
    keys = hept.hept_sort_keys(qh, rank_eta, rank_phi, regions_h.to(device), shift, n_raw)
    want = ol.hept_sort_keys(_np(qh).reshape(24, n), s_eta.numpy(), s_phi.numpy(), regions_h.numpy(),
                             _np(shift).reshape(-1), n_raw)
    assert keys.shape == (3, 8, n) and np.array_equal(_np(keys).reshape(24, n), want)
    # the unfused route through the reference-named functions gives the same bits
    reg = (hept.quantile_partition(s_eta.to(device), regions_h[0]), hept.quantile_partition(s_phi.to(device), regions_h[1]))
    qs, _ = hept.get_geo_shift(regions_h, shift.reshape(24, 1), reg, 3)
    hashed = qh.clone()
    hashed[..., n_raw:] = float("inf")
    assert torch.equal(hashed + qs, keys)
    q_pos, k_pos = hept.hept_positions(e, q_hat.to(device), k_hat.to(device), regions_h, rank_eta, rank_phi, n_raw)
    want_pos = ol.stable_argsort(want, ol.KEY_F32)
    assert q_pos.shape == (3, 8, n) and np.array_equal(_np(q_pos).reshape(24, n), want_pos)
    want_k = ol.hept_sort_keys(_np(kh).reshape(24, n), s_eta.numpy(), s_phi.numpy(), regions_h.numpy(),
                               _np(shift).reshape(-1), n_raw)
    assert np.array_equal(_np(k_pos).reshape(24, n), ol.stable_argsort(want_k, ol.KEY_F32))
    assert np.array_equal(_np(q_pos)[..., n_raw:].reshape(24, -1), np.broadcast_to(np.arange(n_raw, n), (24, n - n_raw)))


def test_prepare_input_matches_oracle(device):
    regions, regions_h = _regions(num_regions=60)
    n_raw, block = 4001, 100
    coords, feats, _ = synth.collider_event(n_raw, seed=3)
    x, mask, kw = hept.prepare_input(feats.to(device), None, coords.to(device), torch.zeros(n_raw, dtype=torch.long),
                                     {"block_size": block, "regions": regions})
    n = 4100
    assert mask is None and kw["raw_size"] == n_raw and x.shape == (n, 24) and kw["coords"].shape == (n, 4)
    assert torch.equal(x[:n_raw].cpu(), feats) and (x[n_raw:] == 0).all() and (kw["coords"][n_raw:] == 0).all()
    assert torch.equal(kw["coords"][:n_raw].cpu(), coords) and torch.equal(kw["regions_h"].cpu(), regions_h)
    padded = torch.full((n, 4), float("inf"))
    padded[:n_raw] = coords
    for a in range(2):
        order = torch.sort(padded[:, a], stable=True).indices.numpy()
        assert np.array_equal(_np(kw["region_indices"][a]), ol.quantile_regions(order, regions_h[a].numpy()))


@pytest.mark.parametrize("n,n_raw", [(1, 1), (1000, 1000), (4100, 4001)])
def test_prep_qk_against_oracle(device, n, n_raw):
    gen = torch.Generator().manual_seed(n)
    H, d, R, K = 8, 24, 2, 3
    q, k = torch.randn(n, H, d, generator=gen), torch.randn(n, H, d, generator=gen)
    w, coords = torch.randn(H, d, R, K, generator=gen) * 0.2, torch.randn(n, R + 1, generator=gen)
    w[1, :, 0, 0] = 40.0                                     # one weight sum beyond the clamp at 50
    want_q, want_k = ol.prep_qk(q.numpy(), k.numpy(), w.numpy(), coords.numpy())
    q_hat, k_hat = hept.prep_qk(q.to(device), k.to(device), w.to(device), coords.to(device))
    assert q_hat.shape == (n, H, d + R + 1) and q_hat.dtype == torch.float32
    for got, want in ((q_hat, want_q), (k_hat, want_k)):
        assert np.allclose(_np(got), want, rtol=3e-6, atol=1e-6)
        assert np.array_equal(_np(got)[..., :d], want[..., :d].astype(np.float32))      # the copied part is exact
    qh, kh = hept.prep_qk_heads(q.to(device), k.to(device), w.to(device), coords.to(device), n_raw)
    assert qh.shape == (H, n, d + R + 1)
    assert torch.equal(qh[:, :n_raw], q_hat.permute(1, 0, 2)[:, :n_raw]) and (qh[:, n_raw:] == 0).all()
    assert torch.equal(kh[:, :n_raw], k_hat.permute(1, 0, 2)[:, :n_raw]) and (kh[:, n_raw:] == 0).all()
