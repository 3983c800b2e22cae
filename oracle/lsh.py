"""CPU oracle for the LSH stage (TEST INFRASTRUCTURE ONLY).

Thin numpy front-ends to ``lsh_oracle.c`` plus independent brute-force restatements used to pin it.
Reference lines restated: ``models/model_utils/hash_utils.py:14-26,46-57,83-93,333-371``,
``models/attention/hept.py:9-19,78-88,130-136``, ``models/baselines/full_mamba2.py:155-218,678-682``.
"""
import ctypes

import numpy as np

from ._lib import lib, ptr

KEY_U32, KEY_I32, KEY_F32 = 0, 1, 2
_c = ctypes


def project(coords: np.ndarray, alpha: np.ndarray) -> np.ndarray:
    """proj[c, n] = <coords[n], alpha[:, c]> with the left-to-right fmaf chain. coords [N,D], alpha [D,C]."""
    coords = np.ascontiguousarray(coords, np.float32)
    alpha = np.ascontiguousarray(alpha, np.float32)
    n, d = coords.shape
    c = alpha.shape[1]
    out = np.empty((c, n), np.float32)
    lib().oracle_lsh_project(ptr(coords), _c.c_int64(n), d, ptr(alpha), c, ptr(out))
    return out


def bucket_ids(coords, alpha, beta, w: float) -> np.ndarray:
    """ids[c, n] = floor((proj + beta[c]) * (1/w)) as int32 (saturating)."""
    coords = np.ascontiguousarray(coords, np.float32)
    alpha = np.ascontiguousarray(alpha, np.float32)
    beta = np.ascontiguousarray(beta, np.float32).reshape(-1)
    n, d = coords.shape
    c = alpha.shape[1]
    inv_w = np.float32(1.0) / np.float32(w)
    out = np.empty((c, n), np.int32)
    lib().oracle_lsh_bucket_ids(ptr(coords), _c.c_int64(n), d, ptr(alpha), ptr(beta), c, _c.c_float(inv_w),
                                ptr(out))
    return out


def pack_keys(ids: np.ndarray, n_tables: int, n_proj: int, n_valid=None):
    """ids [T*J, N] -> (keys [T,N] int32, meta [T, 2J+3] int32 = lo[J], range[J], total, key_bits, overflow)."""
    ids = np.ascontiguousarray(ids, np.int32)
    n = ids.shape[-1]
    n_valid = n if n_valid is None else n_valid
    keys = np.empty((n_tables, n), np.int32)
    meta = np.empty((n_tables, 2 * n_proj + 3), np.int32)
    lib().oracle_lsh_pack_keys(ptr(ids), n_tables, n_proj, _c.c_int64(n), _c.c_int64(n_valid), ptr(keys),
                               ptr(meta))
    return keys, meta


def stable_argsort(keys: np.ndarray, kind: int = KEY_I32, vals=None, return_keys: bool = False):
    """Stable ascending argsort of each row of keys [S,N] (u32 / i32 / f32 by ``kind``)."""
    keys = np.ascontiguousarray(keys)
    assert keys.dtype.itemsize == 4
    s, n = keys.shape
    perm = np.empty((s, n), np.int32)
    kout = np.empty((s, n), keys.dtype) if return_keys else None
    if vals is not None:
        vals = np.ascontiguousarray(vals, np.int32)
    lib().oracle_stable_argsort(ptr(keys), s, _c.c_int64(n), kind, ptr(vals), ptr(perm), ptr(kout))
    return (perm, kout) if return_keys else perm


def gather_rows(src: np.ndarray, idx: np.ndarray) -> np.ndarray:
    """dst[s, n] = src[(s or 0), idx[s, n]]; src [N,D] or [S,N,D], idx [S,N] int32."""
    src = np.ascontiguousarray(src)
    idx = np.ascontiguousarray(idx, np.int32)
    s, n = idx.shape
    segs = 1 if src.ndim == 2 else src.shape[0]
    row_bytes = src.shape[-1] * src.dtype.itemsize
    dst = np.empty((s, n, src.shape[-1]), src.dtype)
    lib().oracle_gather_rows(ptr(src), segs, ptr(idx), s, _c.c_int64(n), _c.c_int64(row_bytes), ptr(dst))
    return dst


def scatter_rows(src: np.ndarray, idx: np.ndarray) -> np.ndarray:
    """dst[s, idx[s, n]] = src[s, n]; src [S,N,D], idx [S,N] a permutation per row."""
    src = np.ascontiguousarray(src)
    idx = np.ascontiguousarray(idx, np.int32)
    s, n = idx.shape
    row_bytes = src.shape[-1] * src.dtype.itemsize
    dst = np.empty_like(src)
    lib().oracle_scatter_rows(ptr(src), ptr(idx), s, _c.c_int64(n), _c.c_int64(row_bytes), ptr(dst))
    return dst


def invert_perm(perm: np.ndarray) -> np.ndarray:
    perm = np.ascontiguousarray(perm, np.int32)
    s, n = perm.shape
    inv = np.empty_like(perm)
    lib().oracle_invert_perm(ptr(perm), s, _c.c_int64(n), ptr(inv))
    return inv


def lsh_ordering_keys(coords: np.ndarray, alpha: np.ndarray):
    """(key [N] = sum_h 2^h proj_h, norm [N] = |coords|) by the fp32 chains of the C oracle."""
    coords = np.ascontiguousarray(coords, np.float32)
    alpha = np.ascontiguousarray(alpha, np.float32)
    n, d = coords.shape
    h = alpha.shape[1]
    key = np.empty(n, np.float32)
    norm = np.empty(n, np.float32)
    lib().oracle_lsh_ordering_keys(ptr(coords), _c.c_int64(n), d, ptr(alpha), h, ptr(key), ptr(norm))
    return key, norm


def lsh_ordering(coords: np.ndarray, alpha: np.ndarray) -> np.ndarray:
    """LSHOrdering permutation (full_mamba2.py:199-208): stable sort by norm, then stable sort by key."""
    key, norm = lsh_ordering_keys(coords, alpha)
    norm_idx = stable_argsort(norm[None], KEY_F32)[0]
    return stable_argsort(key[norm_idx][None], KEY_F32, vals=norm_idx[None])[0]


def bucket_sort(coords, alpha, beta, w, n_tables, n_proj, feats=None, n_valid=None):
    """Whole config-1 pipeline: ids -> packed keys -> stable perm -> (optional) permuted features."""
    ids = bucket_ids(coords, alpha, beta, w)
    if n_valid is not None:
        ids[:, n_valid:] = 0
    keys, meta = pack_keys(ids, n_tables, n_proj, n_valid)
    perm = stable_argsort(keys, KEY_I32)
    out = {"ids": ids, "keys": keys, "meta": meta, "perm": perm}
    if feats is not None:
        out["feats"] = gather_rows(feats, perm)
    return out


# ------------------------------------------------------------------------------- HEPT region (AND-hash) front end
def quantile_regions(sorted_indices: np.ndarray, regions: np.ndarray) -> np.ndarray:
    """``hash_utils.py:14-26``: out[r, n] = floor(rank[n] / ceil(N / regions[r])) + 1 in float32, where rank is the
    inverse of ``sorted_indices`` (the position of hit n in the coordinate order)."""
    sorted_indices = np.asarray(sorted_indices, np.int64)
    n = sorted_indices.shape[-1]
    rank = np.empty(n, np.int64)
    rank[sorted_indices] = np.arange(n)
    size = np.ceil(np.float32(n) / np.asarray(regions, np.float32).reshape(-1, 1))
    return (np.floor(rank.astype(np.float32)[None] / size) + np.float32(1)).astype(np.float32)


def geo_shift(regions_eta: np.ndarray, hash_shift: np.ndarray, region_eta: np.ndarray, region_phi: np.ndarray):
    """``hept.py:78-88``: (region_phi * shift) * (ceil(regions_eta) + 1) + region_eta * shift, each product and the
    sum rounded once to float32. regions_eta, hash_shift [R]; region_* [R, N]."""
    shift = np.asarray(hash_shift, np.float32).reshape(-1, 1)
    mult = np.ceil(np.asarray(regions_eta, np.float32).reshape(-1, 1)) + np.float32(1)
    a = (np.asarray(region_phi, np.float32) * shift) * mult
    b = np.asarray(region_eta, np.float32) * shift
    return (a + b).astype(np.float32)


def hept_sort_keys(hashed: np.ndarray, sorted_eta, sorted_phi, regions: np.ndarray, hash_shift, n_raw: int):
    """``hept.py:130-136``: hashed [R, N] with +inf at and beyond n_raw, plus the region shift. regions [2, R]."""
    h = np.array(hashed, np.float32, copy=True)
    h[:, n_raw:] = np.inf
    reg_eta = quantile_regions(sorted_eta, regions[0])
    reg_phi = quantile_regions(sorted_phi, regions[1])
    return (h + geo_shift(regions[0], hash_shift, reg_eta, reg_phi)).astype(np.float32)


def prep_qk(query, key, w, coords):
    """``hept.py:54-62`` in float64: query, key [n, H, d], w [H, d, R, K], coords [n, R + 1] -> q_hat, k_hat
    [n, H, d + R + 1]."""
    query, key, w, coords = (np.asarray(t, np.float64) for t in (query, key, w, coords))
    qw = np.exp(np.minimum(w.sum(axis=1), 50.0)).sum(axis=-1)               # [H, R]
    expand = np.concatenate([qw[:, :1], qw], axis=-1)                       # [H, R + 1]
    extra = np.sqrt(2.0 * expand)[None] * coords[:, None]                   # [n, H, R + 1]
    return np.concatenate([query, extra], axis=-1), np.concatenate([key, extra], axis=-1)
