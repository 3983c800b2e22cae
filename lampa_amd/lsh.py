"""LSH stage on the GPU: E2LSH hashing, bucket-key packing, stable radix sort, gather / unsort.

Drop-in operator names and signatures of the reference (chengjiang123/Lampa):
``E2LSH``, ``lsh_mapping``, ``lsh_mapping1``, ``invert_permutation``, ``batched_index_select``,
``pad_to_multiple`` (``models/model_utils/hash_utils.py:46-93,333-371``), ``sort_to_buckets``,
``unsort_from_buckets`` (``models/attention/hept.py:9-19``) and ``LSHOrdering``
(``models/baselines/full_mamba2.py:144-218``), plus the quantised E2LSH bucket sort
(``lsh_bucket_sort``) and the primitives they are built from (``stable_argsort``, ``gather_rows``,
``scatter_rows``).  Everything runs in hand-written HIP kernels behind the C ABI of ``liblampa_amd.so``;
torch only owns the memory and the stream.
"""
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _capi
from ._capi import LampaError, check, ptr, require_cuda, stream_of

KEY_U32, KEY_I32, KEY_F32 = 0, 1, 2


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------------------------------------ primitives
def stable_argsort(keys: torch.Tensor, values: Optional[torch.Tensor] = None, key_bits: int = 32,
                   key_bits_dev: Optional[torch.Tensor] = None, key_bits_stride: int = 1, n_passes: int = 0,
                   unsigned: bool = False) -> torch.Tensor:
    """Stable ascending argsort along the last dimension of ``keys`` (int32 / float32, any leading shape).

    Returns int32 positions (or ``values`` permuted the same way when given). ``unsigned=True`` treats int32
    keys as uint32, which lets ``key_bits`` / ``key_bits_dev`` restrict the sort to the low bits.
    """
    require_cuda(keys, values, key_bits_dev)
    if keys.dtype == torch.float32:
        kind = KEY_F32
    elif keys.dtype == torch.int32:
        kind = KEY_U32 if unsigned else KEY_I32
    else:
        raise TypeError(f"stable_argsort: keys must be int32 or float32, got {keys.dtype}")
    keys = keys.contiguous()
    n = keys.shape[-1]
    segs = max(1, keys.numel() // max(n, 1))
    out = torch.empty(keys.shape, dtype=torch.int32, device=keys.device)
    if keys.numel() == 0:
        return out
    if values is not None:
        values = values.to(torch.int32).contiguous()
        assert values.shape == keys.shape
    lib = _capi.lib()
    ws = _workspace(check(lib.lampa_sort_workspace_bytes(segs, n), "lampa_sort_workspace_bytes"), keys.device)
    check(lib.lampa_sort_pairs(ptr(keys), kind, ptr(values), segs, n, key_bits, ptr(key_bits_dev), key_bits_stride,
                               n_passes, ptr(out), ptr(ws), ws.numel(), stream_of(keys)), "lampa_sort_pairs")
    return out


def _idx_bytes(idx: torch.Tensor) -> int:
    if idx.dtype == torch.int32:
        return 4
    if idx.dtype == torch.int64:
        return 8
    raise TypeError(f"index tensors must be int32 or int64, got {idx.dtype}")


def gather_rows(src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """``dst[s, n, :] = src[s % S_src, idx[s, n], :]``; src [S_src, N_src, D] (or [N_src, D]), idx [S, N]."""
    require_cuda(src, idx)
    if src.dim() == 2:
        src = src.unsqueeze(0)
    src, idx = src.contiguous(), idx.contiguous()
    s, n = idx.shape
    dst = torch.empty((s, n, src.shape[-1]), dtype=src.dtype, device=src.device)
    row_bytes = src.shape[-1] * src.element_size()
    if dst.numel():
        check(_capi.lib().lampa_gather_rows(ptr(src), src.shape[0], src.shape[1], ptr(idx), _idx_bytes(idx), s, n,
                                            row_bytes, ptr(dst), stream_of(src)), "lampa_gather_rows")
    return dst


def scatter_rows(src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """``dst[s, idx[s, n], :] = src[s, n, :]`` for a permutation ``idx`` [S, N] (the unsort by scatter)."""
    require_cuda(src, idx)
    src, idx = src.contiguous(), idx.contiguous()
    s, n = idx.shape
    dst = torch.empty_like(src)
    row_bytes = src.shape[-1] * src.element_size()
    if dst.numel():
        check(_capi.lib().lampa_scatter_rows(ptr(src), ptr(idx), _idx_bytes(idx), s, n, row_bytes, ptr(dst),
                                             stream_of(src)), "lampa_scatter_rows")
    return dst


def invert_permutation(perm: torch.Tensor) -> torch.Tensor:
    """``hash_utils.py:46-57``: inverse of a permutation along the last dimension, O(n) scatter of arange."""
    require_cuda(perm)
    perm = perm.contiguous()
    n = perm.shape[-1]
    inv = torch.empty_like(perm)
    if perm.numel():
        check(_capi.lib().lampa_invert_perm(ptr(perm), _idx_bytes(perm), perm.numel() // n, n, ptr(inv),
                                            stream_of(perm)), "lampa_invert_perm")
    return inv


def row_minmax(x: torch.Tensor):
    """(min, max) over the last dimension of a float32 tensor, keepdim."""
    require_cuda(x)
    x = x.contiguous().float()
    rows = x.numel() // x.shape[-1]
    out = torch.empty((rows, 2), dtype=torch.float32, device=x.device)
    check(_capi.lib().lampa_row_minmax_f32(ptr(x), rows, x.shape[-1], ptr(out), stream_of(x)), "lampa_row_minmax_f32")
    shape = x.shape[:-1] + (1,)
    return out[:, 0].reshape(shape), out[:, 1].reshape(shape)


# ------------------------------------------------------------------------------------ reference-named helpers
def batched_index_select(values: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """``hash_utils.py:83-93``: values (1 or n_hashes, batch, seqlen, dim), indices (n_hashes, batch, seqlen)
    -> (n_hashes, batch, seqlen, dim)."""
    lead = indices.shape[:-1]
    src = values.reshape(-1, values.shape[-2], values.shape[-1])
    idx = indices.reshape(-1, indices.shape[-1])
    return gather_rows(src, idx).reshape(*lead, indices.shape[-1], values.shape[-1])


def pad_to_multiple(tensor: torch.Tensor, multiple: int, dims=-1, value=0):
    """``hash_utils.py:61-80``: pad the given dims up to a multiple (padding on the high side)."""
    try:
        dims = list(dims)
    except TypeError:
        dims = [dims]
    dims = [d if d >= 0 else tensor.ndim + d for d in dims]
    padding = [0] * (2 * tensor.ndim)
    for d in dims:
        remainder = tensor.size(d) % multiple
        if remainder != 0:
            padding[2 * (tensor.ndim - d - 1) + 1] = multiple - remainder
    if all(p == 0 for p in padding):
        return tensor
    return F.pad(tensor, tuple(padding), value=value)


def sort_to_buckets(x: torch.Tensor, perm: torch.Tensor, bucketsz: int) -> torch.Tensor:
    """``hept.py:9-14``: x (b, s, d), perm (h, b, s) -> (h, b, s / bucketsz, bucketsz, d)."""
    g = batched_index_select(x.unsqueeze(0), perm)
    h, b, s, d = g.shape
    return g.reshape(h, b, s // bucketsz, bucketsz, d)


def unsort_from_buckets(s_x: torch.Tensor, perm_inverse: torch.Tensor) -> torch.Tensor:
    """``hept.py:17-19``: s_x (h, b, nbuckets, bucketsz, d), perm_inverse (h, b, s) -> (h, b, s, d)."""
    h, b, nb, bs, d = s_x.shape
    return batched_index_select(s_x.reshape(h, b, nb * bs, d), perm_inverse)


class E2LSH(nn.Module):
    """``hash_utils.py:359-371``: alpha ~ N(0,1) [n_heads, dim, n_hashes], beta ~ U(0,r) [1, n_hashes] (kept,
    unused by forward as in the reference); forward(vecs [n_heads, N, dim]) -> [n_hashes, n_heads, N].
    ``layout="hnN"`` is the ``hash_utils`` layout; ``layout="hNn"`` gives [n_hashes, N, n_heads]
    (``full_mamba2.py:128-141``)."""

    def __init__(self, n_hashes, n_heads, dim, r=1, layout="hnN"):
        super().__init__()
        self.alpha = nn.Parameter(torch.normal(0, 1, (n_heads, dim, n_hashes)), requires_grad=False)
        self.beta = nn.Parameter(torch.rand(1, n_hashes) * r, requires_grad=False)
        self.layout = layout

    @torch.no_grad()
    def forward(self, vecs: torch.Tensor) -> torch.Tensor:
        require_cuda(vecs, self.alpha)
        n_heads, n, dim = vecs.shape
        n_hashes = self.alpha.shape[-1]
        vecs = vecs.contiguous().float()
        alpha = self.alpha.detach().contiguous().float()
        if self.layout == "hnN":
            out = torch.empty((n_hashes, n_heads, n), dtype=torch.float32, device=vecs.device)
            strides = (n_heads * n, n, 1)
        else:
            out = torch.empty((n_hashes, n, n_heads), dtype=torch.float32, device=vecs.device)
            strides = (n * n_heads, 1, n_heads)
        if out.numel():
            check(_capi.lib().lampa_lsh_project_f32(ptr(vecs), n_heads, n, dim, ptr(alpha), n_hashes, ptr(out),
                                                    strides[0], strides[1], strides[2], stream_of(vecs)),
                  "lampa_lsh_project_f32")
        return out


@torch.no_grad()
def lsh_mapping(e2lsh, queries, keys):
    """``hash_utils.py:333-340``: hashes of queries and keys plus their joint range over the hits."""
    qh, kh = e2lsh(queries), e2lsh(keys)
    qlo, qhi = row_minmax(qh)
    klo, khi = row_minmax(kh)
    return qh, kh, torch.maximum(qhi, khi) - torch.minimum(qlo, klo)


@torch.no_grad()
def lsh_mapping1(e2lsh, hidden_states):
    """``hash_utils.py:343-356``."""
    hh = e2lsh(hidden_states)
    lo, hi = row_minmax(hh)
    return hh, hi - lo


class LSHOrdering(nn.Module):
    """``full_mamba2.py:144-218``: order the points of each batch element by a scalar LSH key
    (sum_h 2^h <coords, alpha_h>), ties broken by the norm of the coordinates, then by input order.
    Returns (ordered_points [B, L, D], indices [B, L] int64)."""

    def __init__(self, input_dim: int, num_hashes: int = 3):
        super().__init__()
        self.num_hashes = num_hashes
        self.e2lsh = E2LSH(self.num_hashes, n_heads=1, dim=input_dim, layout="hNn")

    @torch.no_grad()
    def forward(self, points: torch.Tensor, coords: Optional[torch.Tensor] = None):
        require_cuda(points, coords)
        B, L, D = points.shape
        src = points if coords is None else coords
        C = src.shape[-1]
        flat = src.reshape(B * L, C).contiguous().float()
        alpha = self.e2lsh.alpha.detach()[0].contiguous().float()  # [C, H]
        key = torch.empty(B * L, dtype=torch.float32, device=points.device)
        norm = torch.empty_like(key)
        lib = _capi.lib()
        if B * L:
            check(lib.lampa_lsh_ordering_keys(ptr(flat), B * L, C, ptr(alpha), self.num_hashes, ptr(key), ptr(norm),
                                              stream_of(flat)), "lampa_lsh_ordering_keys")
        norm_idx = stable_argsort(norm.view(B, L))
        key_sorted_by_norm = gather_rows(key.view(B, L, 1), norm_idx).view(B, L)
        indices = stable_argsort(key_sorted_by_norm, values=norm_idx)
        ordered = gather_rows(points.contiguous(), indices)
        return ordered, indices.long()


# -------------------------------------------------------------------------------- quantised E2LSH bucket sort
def lsh_bucket_keys(coords: torch.Tensor, alpha: torch.Tensor, beta: torch.Tensor, w: float, n_tables: int,
                    n_proj: int, n_valid: Optional[int] = None, return_ids: bool = True):
    """ids[c, n] = floor((<coords[n], alpha[:, c]> + beta[c]) / w) (int32, c = table * n_proj + projection) and the
    mixed-radix bucket key of every table. Returns (ids [T*J, N] or None, keys [T, N] int32,
    meta [T, 2J+3] int32 = lo[J], range[J], total, key_bits, overflow). Hits at n >= n_valid are padding: their
    ids are 0 and their key is ``total`` so that they sort last."""
    require_cuda(coords, alpha, beta)
    coords = coords.contiguous().float()
    alpha = alpha.contiguous().float()
    beta = beta.contiguous().float().reshape(-1)
    n, dim = coords.shape
    assert alpha.shape == (dim, n_tables * n_proj) and beta.numel() == n_tables * n_proj
    n_valid = n if n_valid is None else int(n_valid)
    dev = coords.device
    ids = torch.empty((n_tables * n_proj, n), dtype=torch.int32, device=dev) if return_ids else None
    keys = torch.empty((n_tables, n), dtype=torch.int32, device=dev)
    meta = torch.empty((n_tables, 2 * n_proj + 3), dtype=torch.int32, device=dev)
    lib = _capi.lib()
    ws = _workspace(check(lib.lampa_lsh_bucket_workspace_bytes(n, n_tables, n_proj), "workspace"), dev)
    check(lib.lampa_lsh_bucket_keys(ptr(coords), n, n_valid, dim, ptr(alpha), ptr(beta), n_tables, n_proj, float(w),
                                    ptr(ids), ptr(keys), ptr(meta), ptr(ws), ws.numel(), stream_of(coords)),
          "lampa_lsh_bucket_keys")
    return ids, keys, meta


META_KEY_OVERFLOW, META_GAVE_UP = 1, 2  # bits of meta[..., -1]


def decode_meta_flags(meta) -> dict:
    """The flag field ``meta[..., -1]`` of every table as booleans: ``key_overflow`` (bit 0: the id ranges of the table
    multiply to more than 2^31 - 1 buckets, its order is meaningless) and ``gave_up`` (bit 1: a workgroup of the
    one-launch kernel gave up waiting for the others of its table; the table's perm is then all -1 and its sorted
    features all zero). Takes the device tensor (one host synchronisation) or anything ``torch.as_tensor`` accepts."""
    flags = torch.as_tensor(meta)[..., -1].cpu()
    return {"key_overflow": (flags & META_KEY_OVERFLOW) != 0, "gave_up": (flags & META_GAVE_UP) != 0}


def one_launch_config(enabled: bool = True, wait_limit: int = -1, tile: int = 0) -> None:
    """Process-wide switches of the one-launch form of the stage (``lampa_lsh_one_launch_config``): ``enabled=False``
    sends every call to the separate kernels; ``wait_limit`` is the number of polls a workgroup spends in one wait
    before it gives up (< 0: the built-in bound; 0: give up at once, for tests of the give-up path); ``tile`` = 1024
    or 768 forces that form of the kernel (512 threads x 2 hits, 768 threads x 1 hit) for every call whose workgroups fit
    the GPU at once (0: the library chooses between them and the separate kernels)."""
    code = {0: 1, 1024: 100, 768: 101}[tile]
    check(_capi.lib().lampa_lsh_one_launch_config(code if enabled else 0, int(wait_limit)), "lampa_lsh_one_launch_config")


def _raise_on_overflow(meta: torch.Tensor, strict: bool):
    if not strict:
        return
    flags = decode_meta_flags(meta)
    if bool(flags["gave_up"].any()):
        raise LampaError("lsh_bucket_sort: a workgroup of the one-launch kernel gave up waiting for the other "
                         "workgroups of its table (the GPU was shared with another kernel that waits in the same way); "
                         "the outputs of this call are not to be used")
    if bool(flags["key_overflow"].any()):
        raise LampaError("lsh_bucket_sort: the id ranges of a table multiply to more than 2^31 - 1 buckets, so its "
                         "32-bit bucket key overflowed and the order is meaningless (use a larger w or fewer "
                         "projections per table)")


def lsh_bucket_sort(coords, alpha, beta, w, n_tables, n_proj, feats: Optional[torch.Tensor] = None,
                    n_valid=None, return_ids: bool = True, n_passes: int = 0, strict: bool = False):
    """E2LSH bucketing in one library call: bucket ids -> packed keys -> stable sort permutation per table ->
    (optionally) the hit features in sorted order. No host synchronisation: the sort reads the number of key bits
    from ``meta`` on the device.

    One event: coords [N, dim], feats [N, D], n_valid an int -> dict with ids [T*J, N], keys / perm [T, N] int32,
    meta [T, 2J+3], feats [T, N, D].
    A batch of events of N hits each (pad shorter ones): coords [E, N, dim], feats [E, N, D], n_valid an int32
    tensor [E] on the device (or None) -> the same entries with a leading event dimension; one set of launches for
    the whole batch.

    A table whose id ranges multiply to more than 2^31 - 1 buckets cannot be packed into one 32-bit key: the kernel
    then sets ``meta[..., -1]`` (overflow) and the order of that table is meaningless. ``strict=True`` reads the flag
    (one host synchronisation) and raises ``LampaError``; otherwise the caller has to look at the flag.

    A call of at most 64 tables in total whose tiles of 1 024 hits come to at most two workgroups per CU (one or two
    events of 60 000 hits do, four of 30 000) runs as ONE kernel whose workgroups wait for each other; larger calls run as separate kernels. The waits of the
    one-launch kernel are bounded: should one run out (two such kernels sharing a GPU can starve each other) bit 1 of
    ``meta[..., -1]`` is set, the table's ``perm`` is all -1 and its ``feats`` all zero; ``strict=True`` raises for it as
    well (``decode_meta_flags`` reads the field). Calls that may run at the same time on one GPU (different streams,
    processes) should be serialised by the caller."""
    require_cuda(coords, alpha, beta, feats)
    coords = coords.contiguous().float()
    alpha = alpha.contiguous().float()
    beta = beta.contiguous().float().reshape(-1)
    batched = coords.dim() == 3
    n, dim = coords.shape[-2:]
    n_events = coords.shape[0] if batched else 1
    lead = (n_events,) if batched else ()
    assert alpha.shape == (dim, n_tables * n_proj) and beta.numel() == n_tables * n_proj
    dev = coords.device
    ids = torch.empty(lead + (n_tables * n_proj, n), dtype=torch.int32, device=dev) if return_ids else None
    keys = torch.empty(lead + (n_tables, n), dtype=torch.int32, device=dev)
    meta = torch.empty(lead + (n_tables, 2 * n_proj + 3), dtype=torch.int32, device=dev)
    perm = torch.empty(lead + (n_tables, n), dtype=torch.int32, device=dev)
    out = {"ids": ids, "keys": keys, "meta": meta, "perm": perm}
    fo, row_bytes = None, 0
    if feats is not None:
        feats = feats.contiguous()
        assert feats.shape[:-1] == coords.shape[:-1]
        fo = torch.empty(lead + (n_tables, n, feats.shape[-1]), dtype=feats.dtype, device=dev)
        row_bytes = feats.shape[-1] * feats.element_size()
        out["feats"] = fo
    if n == 0 or n_events == 0:
        return out
    lib = _capi.lib()
    if batched:
        nv = None
        if n_valid is not None:
            nv = torch.as_tensor(n_valid, dtype=torch.int32, device=dev).contiguous()
            assert nv.shape == (n_events,)
        ws = _workspace(check(lib.lampa_lsh_bucket_sort_batch_workspace_bytes(n_events, n, n_tables, n_proj),
                              "workspace"), dev)
        check(lib.lampa_lsh_bucket_sort_batch(ptr(coords), n_events, n, ptr(nv), dim, ptr(alpha), ptr(beta), n_tables,
                                              n_proj, float(w), ptr(ids), ptr(keys), ptr(meta), ptr(perm), ptr(feats),
                                              row_bytes, ptr(fo), n_passes, ptr(ws), ws.numel(), stream_of(coords)),
              "lampa_lsh_bucket_sort_batch")
        _raise_on_overflow(meta, strict)
        return out
    n_valid = n if n_valid is None else int(n_valid)
    ws = _workspace(check(lib.lampa_lsh_bucket_sort_workspace_bytes(n, n_tables, n_proj), "workspace"), dev)
    check(lib.lampa_lsh_bucket_sort(ptr(coords), n, n_valid, dim, ptr(alpha), ptr(beta), n_tables, n_proj, float(w),
                                    ptr(ids), ptr(keys), ptr(meta), ptr(perm), ptr(feats), row_bytes, ptr(fo), n_passes,
                                    ptr(ws), ws.numel(), stream_of(coords)), "lampa_lsh_bucket_sort")
    _raise_on_overflow(meta, strict)
    return out
