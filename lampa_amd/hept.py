"""Region (AND-hash) front end of the HEPT bucketing: quantile regions of the eta / phi order, the per-(hash, head)
region shift, and the sort that turns hashes plus shifts into bucket positions.

Mirrors the reference's names and argument orders: ``quantile_partition`` / ``get_regions``
(``models/model_utils/hash_utils.py:14-43``), ``get_geo_shift`` (``models/attention/hept.py:78-88``),
``prepare_input`` (``models/hattention/modeling_gated_deltaproduct.py:1201-1223``), ``prep_qk`` (``hept.py:54-62``).
``hept_positions`` is the fused form of ``hept.py:127-139``, ``prep_qk_heads`` of ``hept.py:118-128``. GPU tensors only; there is no CPU fallback.
"""
from typing import Optional

import torch

from . import _capi
from ._capi import check, ptr, require_cuda, stream_of
from .lsh import (_idx_bytes, invert_permutation, lsh_mapping, pad_to_multiple, sort_to_buckets,  # noqa: F401
                  stable_argsort, unsort_from_buckets)


def get_regions(num_regions, num_or_hashes, num_heads, num_and_hashes=2):
    """``hash_utils.py:29-43``: random split of ``num_regions`` into ``num_and_hashes`` factors for every
    (hash, head), rounded to thirds; returns a CPU float32 tensor [num_or_hashes, num_and_hashes, num_heads].
    One ``torch.rand(1)`` per factor, so a seed gives the reference's values."""
    lb = 2
    ub = 2 * num_regions ** (1 / num_and_hashes) - lb
    rows = [[torch.rand(1).item() * (ub - lb) + lb for _ in range(num_and_hashes)]
            for _ in range(num_or_hashes * num_heads)]
    regions = torch.tensor(rows)
    regions = (num_regions / regions.prod(dim=1, keepdim=True)) ** (1 / num_and_hashes) * regions
    regions = torch.round(regions * 3) / 3
    return regions.reshape(num_heads, num_or_hashes, num_and_hashes).permute(1, 2, 0)  # "(h c) a -> c a h"


def _regions_on(regions: torch.Tensor, device) -> torch.Tensor:
    return regions.detach().to(device=device, dtype=torch.float32).contiguous()


@torch.no_grad()
def quantile_partition(sorted_indices: torch.Tensor, num_regions: torch.Tensor) -> torch.Tensor:
    """``hash_utils.py:14-26``: sorted_indices [N] (the argsort of a coordinate), num_regions [R, 1] or [R] ->
    float32 [R, N] with the 1-based quantile region of every hit: floor(rank / ceil(N / num_regions)) + 1."""
    require_cuda(sorted_indices)
    if sorted_indices.dim() != 1:
        raise ValueError("quantile_partition: sorted_indices must be 1-d (one event)")
    n = sorted_indices.shape[0]
    regions = _regions_on(num_regions, sorted_indices.device).reshape(-1)
    rank = invert_permutation(sorted_indices)
    out = torch.empty((regions.numel(), n), dtype=torch.float32, device=sorted_indices.device)
    if out.numel():
        check(_capi.lib().lampa_quantile_regions(ptr(rank), _idx_bytes(rank), n, ptr(regions), regions.numel(), ptr(out),
                                                 stream_of(rank)), "lampa_quantile_regions")
    return out


@torch.no_grad()
def get_geo_shift(regions_h, hash_shift: torch.Tensor, region_indices, num_or_hashes: int) -> torch.Tensor:
    """``hept.py:78-88``: regions_h [2, R] (or a list of two [R] rows), hash_shift [R, 1], region_indices =
    (eta [R, N], phi [R, N]) -> [2, num_or_hashes, R / num_or_hashes, N]; the query and key halves are the same
    values (as in the reference) and share memory."""
    region_eta, region_phi = region_indices
    require_cuda(region_eta, region_phi, hash_shift)
    region_eta = region_eta.contiguous().float()
    region_phi = region_phi.contiguous().float()
    rows, n = region_eta.shape
    shift = hash_shift.detach().reshape(-1).contiguous().float()
    regions_eta = _regions_on(regions_h[0], region_eta.device).reshape(-1)
    if shift.numel() != rows or regions_eta.numel() != rows or region_phi.shape != region_eta.shape:
        raise ValueError("get_geo_shift: regions_h, hash_shift and region_indices disagree on the number of rows")
    out = torch.empty((rows, n), dtype=torch.float32, device=region_eta.device)
    if out.numel():
        check(_capi.lib().lampa_geo_shift(ptr(region_eta), ptr(region_phi), ptr(shift), ptr(regions_eta), rows, n,
                                          ptr(out), stream_of(out)), "lampa_geo_shift")
    return out.reshape(1, num_or_hashes, rows // num_or_hashes, n).expand(2, -1, -1, -1)


@torch.no_grad()
def hept_sort_keys(hashed: torch.Tensor, rank_eta: torch.Tensor, rank_phi: torch.Tensor, regions_h: torch.Tensor,
                   hash_shift: torch.Tensor, raw_size: Optional[int] = None) -> torch.Tensor:
    """Sort keys of ``hept.py:130-136`` in one pass: hashed [c, h, N] (+inf from raw_size on) plus the region shift
    of its (hash, head) row. rank_eta / rank_phi [N] int32 = inverse of the eta / phi argsort; regions_h [2, c*h];
    hash_shift [c*h, 1] or [c, h, 1]."""
    require_cuda(hashed, rank_eta, rank_phi, hash_shift)
    hashed = hashed.contiguous().float()
    n = hashed.shape[-1]
    rows = hashed.numel() // max(n, 1)
    regions = _regions_on(regions_h, hashed.device).reshape(2, -1)
    shift = hash_shift.detach().reshape(-1).contiguous().float()
    if regions.shape[1] != rows or shift.numel() != rows or rank_eta.numel() != n or rank_phi.numel() != n:
        raise ValueError("hept_sort_keys: hashed, regions_h, hash_shift and the ranks disagree on shapes")
    rank_eta = rank_eta.to(torch.int32).contiguous()
    rank_phi = rank_phi.to(torch.int32).contiguous()
    keys = torch.empty_like(hashed)
    if keys.numel():
        check(_capi.lib().lampa_hept_sort_keys(ptr(hashed), ptr(rank_eta), ptr(rank_phi), ptr(regions), ptr(shift), rows, n,
                                               n if raw_size is None else int(raw_size), ptr(keys), stream_of(keys)),
              "lampa_hept_sort_keys")
    return keys


@torch.no_grad()
def _prep(query, key, w, coords, raw_size, heads_first):
    require_cuda(query, key, w, coords)
    n, H, d = query.shape
    R, Kw = w.shape[2], w.shape[3]
    if key.shape != query.shape or w.shape[:2] != (H, d) or coords.shape != (n, R + 1):
        raise ValueError("prep_qk: query/key [n, H, d], w [H, d, R, K] and coords [n, R + 1] disagree on shapes")
    query, key, w, coords = (t.detach().float().contiguous() for t in (query, key, w, coords))
    D = d + R + 1
    shape = (H, n, D) if heads_first else (n, H, D)
    q_hat = torch.empty(shape, dtype=torch.float32, device=query.device)
    k_hat = torch.empty_like(q_hat)
    scale = torch.empty(H * (R + 1), dtype=torch.float32, device=query.device)
    check(_capi.lib().lampa_hept_prep_qk(ptr(query), ptr(key), ptr(w), ptr(coords), n, n if raw_size is None else int(raw_size),
                                         H, d, R, Kw, int(heads_first), ptr(scale), ptr(q_hat), ptr(k_hat), stream_of(query)),
          "lampa_hept_prep_qk")
    return q_hat, k_hat


def prep_qk(query: torch.Tensor, key: torch.Tensor, w: torch.Tensor, coords: torch.Tensor):
    """``hept.py:54-62``: query, key [n, H, d], w [H, d, R, K], coords [n, R + 1] -> (q_hat, k_hat) [n, H, d + R + 1]:
    the inputs with ``sqrt(2 qw) * coords`` appended, qw[h, r] = sum_k exp(min(sum_d w[h, d, r, k], 50)) and the first
    appended column reusing qw[h, 0]."""
    return _prep(query, key, w, coords, None, False)


def prep_qk_heads(query, key, w, coords, raw_size: Optional[int] = None):
    """``prep_qk`` followed by the rearrange to [H, n, D] and the zeroing of the rows from ``raw_size`` on
    (``hept.py:118-128``) in one pass: the form ``hept_positions`` and ``E2LSH`` take."""
    return _prep(query, key, w, coords, raw_size, True)


@torch.no_grad()
def hept_positions(e2lsh, q_hat: torch.Tensor, k_hat: torch.Tensor, regions_h: torch.Tensor, rank_eta: torch.Tensor,
                   rank_phi: torch.Tensor, raw_size: Optional[int] = None):
    """``hept.py:127-139`` from ``lsh_mapping`` to the two argsorts: hashes of q_hat and k_hat [h, N, dim], their joint
    range, region shifts, then one stable segmented sort per side. Returns (q_positions, k_positions), int32
    [n_hashes, h, N]; ties keep the input order (the reference's argsort leaves them unspecified)."""
    qh, kh, shift = lsh_mapping(e2lsh, q_hat, k_hat)
    q_keys = hept_sort_keys(qh, rank_eta, rank_phi, regions_h, shift, raw_size)
    k_keys = hept_sort_keys(kh, rank_eta, rank_phi, regions_h, shift, raw_size)
    return stable_argsort(q_keys), stable_argsort(k_keys)


def prepare_input(x, edge_index, coords, batch, helper_funcs):
    """``modeling_gated_deltaproduct.py:1201-1223``: pad hits and coordinates to a multiple of the block size
    (padded coordinates +inf so they sort last), eta / phi orders, quantile regions per (hash, head) row; the
    padded coordinates are zeroed afterwards. Returns (x, mask, kwargs) with the reference's keys."""
    kwargs = {}
    assert batch.max() == 0
    kwargs["key_padding_mask"] = None
    kwargs["edge_index"] = edge_index
    with torch.no_grad():
        block_size = helper_funcs["block_size"]
        kwargs["raw_size"] = x.shape[0]
        x = pad_to_multiple(x, block_size, dims=0)
        coords = pad_to_multiple(coords, block_size, dims=0, value=float("inf"))
        sorted_eta_idx = stable_argsort(coords[..., 0].contiguous()).long()
        sorted_phi_idx = stable_argsort(coords[..., 1].contiguous()).long()
        regions = helper_funcs["regions"]
        c, a, h = regions.shape
        regions_h = _regions_on(regions, coords.device).permute(1, 0, 2).reshape(a, c * h)  # "c a h -> a (c h)"
        kwargs["region_indices"] = [quantile_partition(sorted_eta_idx, regions_h[0][:, None]),
                                    quantile_partition(sorted_phi_idx, regions_h[1][:, None])]
        kwargs["regions_h"] = regions_h
        coords[kwargs["raw_size"]:] = 0.0  # only rows added by the padding (an empty slice when nothing was added)
        kwargs["coords"] = coords
    return x, None, kwargs
