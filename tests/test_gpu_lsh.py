"""GPU parity of the LSH stage against the CPU oracle: bit-exact ids, keys, permutations and features."""
import numpy as np
import pytest
import torch

from lampa_amd import lsh, synth
from oracle import lsh as ol

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("n", [1, 63, 2048, 2049, 60000])
def test_config1_bucket_sort_bit_exact(device, n):
    coords, feats, _ = synth.collider_event(n, seed=0)
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    want = ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats.numpy())
    got = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.5, 3, 4, feats.to(device))
    assert np.array_equal(_np(got["ids"]), want["ids"])
    assert np.array_equal(_np(got["meta"]), want["meta"])
    assert np.array_equal(_np(got["keys"]), want["keys"])
    assert np.array_equal(_np(got["perm"]), want["perm"])
    assert np.array_equal(_np(got["feats"]), want["feats"])


def test_bucket_sort_padding_and_dim3(device):
    coords, feats, _ = synth.collider_event(5000, seed=3)
    coords = coords[:, :3].contiguous()
    alpha, beta = synth.lsh_params(3, 2, 3, 0.25, 7)
    want = ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.25, 2, 3, feats.numpy(), n_valid=4321)
    got = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.25, 2, 3, feats.to(device),
                              n_valid=4321)
    for name in ("ids", "meta", "keys", "perm", "feats"):
        assert np.array_equal(_np(got[name]), want[name]), name
    assert (_np(got["perm"])[:, 4321:] >= 4321).all()  # padding sorts last, in input order


def test_bucket_overflow_flag(device):
    coords = torch.tensor([[0.0, 0, 0, 0], [1e6, 1e6, 0, 0]])
    alpha = torch.eye(4)[:, :2].contiguous()
    beta = torch.zeros(2)
    _, _, meta = lsh.lsh_bucket_keys(coords.to(device), alpha.to(device), beta.to(device), 1.0, 1, 2)
    ids = ol.bucket_ids(coords.numpy(), alpha.numpy(), beta.numpy(), 1.0)
    _, want = ol.pack_keys(ids, 1, 2)
    assert np.array_equal(_np(meta), want) and want[0, -1] == 1
    # the one-call stage reports it on request instead of returning a meaningless order silently
    from lampa_amd._capi import LampaError
    with pytest.raises(LampaError, match="overflow"):
        lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 1.0, 1, 2, strict=True)
    lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 1.0, 1, 2)  # default: flag only


def test_gather_out_of_range_index_reads_zeros(device):
    src = torch.arange(1, 13, dtype=torch.float32, device=device).reshape(1, 3, 4)
    idx = torch.tensor([[2, 5, 0, -1]], dtype=torch.int32, device=device)
    got = lsh.gather_rows(src, idx)
    want = torch.stack([src[0, 2], torch.zeros(4, device=device), src[0, 0], torch.zeros(4, device=device)])[None]
    assert torch.equal(got, want)


@pytest.mark.parametrize("kind", ["i32", "f32", "u32bits"])
@pytest.mark.parametrize("shape", [(1, 1), (3, 777), (2, 20000), (5, 4096)])
def test_stable_argsort_matches_torch(device, kind, shape):
    gen = torch.Generator().manual_seed(hash((kind, shape)) % 1000)
    if kind == "i32":
        keys = torch.randint(-300, 300, shape, generator=gen, dtype=torch.int32)  # many ties
        got = lsh.stable_argsort(keys.to(device))
    elif kind == "f32":
        keys = torch.randn(shape, generator=gen)
        keys[..., ::7] = 0.0
        keys[..., 3::11] = -0.0
        if shape[1] > 100:
            keys[0, 5], keys[0, 17], keys[0, 50], keys[0, 51] = float("inf"), float("-inf"), float("nan"), float("nan")
        got = lsh.stable_argsort(keys.to(device))
    else:
        keys = torch.randint(0, 1 << 13, shape, generator=gen, dtype=torch.int32)
        got = lsh.stable_argsort(keys.to(device), key_bits=13, unsigned=True)
    want = torch.sort(keys, dim=-1, stable=True).indices
    assert torch.equal(got.cpu().long(), want)


def test_stable_argsort_full_range_and_values(device):
    gen = torch.Generator().manual_seed(0)
    keys = torch.randint(-2**31, 2**31 - 1, (2, 50000), generator=gen, dtype=torch.int64).to(torch.int32)
    vals = torch.stack([torch.randperm(50000, generator=gen) for _ in range(2)]).to(torch.int32)
    for passes in (0, 3, 4):
        got = lsh.stable_argsort(keys.to(device), values=vals.to(device), n_passes=passes)
        want = torch.gather(vals, 1, torch.sort(keys, dim=-1, stable=True).indices)
        assert torch.equal(got.cpu(), want)
    want = ol.stable_argsort(keys.numpy(), ol.KEY_I32)
    assert np.array_equal(_np(lsh.stable_argsort(keys.to(device))), want)


def test_stable_argsort_per_segment_device_bits(device):
    """Segments whose significant key bits differ (read from device memory) take different numbers of radix passes in
    the same launch: 1-bit, one-digit, just over one digit, two digits and just over, three digits and 32-bit keys."""
    gen = torch.Generator().manual_seed(7)
    bits = [1, 5, 11, 12, 22, 23, 32]
    n = 9000
    rows = []
    for b in bits:
        r = torch.randint(0, 1 << min(b, 31), (n,), generator=gen, dtype=torch.int64)
        if b == 32:
            r = r * 2 + torch.randint(0, 2, (n,), generator=gen, dtype=torch.int64)
        rows.append(r)
    keys64 = torch.stack(rows)
    keys = keys64.to(torch.int32) if max(bits) < 32 else (keys64 - ((keys64 >> 31) << 32)).to(torch.int32)
    want = torch.sort(keys64, dim=-1, stable=True).indices
    # stride 2: the bit counts sit in every other element, as in the per-table meta rows of the bucket keys
    bits_dev = torch.zeros(len(bits) * 2, dtype=torch.int32)
    bits_dev[::2] = torch.tensor(bits, dtype=torch.int32)
    for passes in (0, 3, 4):
        got = lsh.stable_argsort(keys.to(device), key_bits_dev=bits_dev.to(device), key_bits_stride=2,
                                 n_passes=passes, unsigned=True)
        assert torch.equal(got.cpu().long(), want), passes


def test_stable_argsort_device_bits_many_segments(device):
    """Many segments (40 x 15 tiles, spread over the XCDs by segment) with ties: segments that skip the launches only
    wide keys need and segments that need them (23 .. 32 bits) in one call, three and four launches."""
    gen = torch.Generator().manual_seed(11)
    n, bits = 30000, [9, 19, 22, 23, 27, 30, 31, 32] * 5
    rows = []
    for b in bits:
        r = torch.randint(0, 1 << min(b, 31), (n,), generator=gen, dtype=torch.int64)
        if b == 32:
            r = r * 2 + torch.randint(0, 2, (n,), generator=gen, dtype=torch.int64)
        r[::7] = r[0]  # ties, so that stability is tested
        rows.append(r)
    keys64 = torch.stack(rows)
    keys = (keys64 - ((keys64 >> 31) << 32)).to(torch.int32)
    want = torch.sort(keys64, dim=-1, stable=True).indices
    bits_dev = torch.tensor(bits, dtype=torch.int32, device=device)
    for passes in (0, 4):
        got = lsh.stable_argsort(keys.to(device), key_bits_dev=bits_dev, n_passes=passes, unsigned=True)
        assert torch.equal(got.cpu().long(), want), passes


def test_gather_scatter_invert_roundtrip(device):
    gen = torch.Generator().manual_seed(1)
    for d, dtype in ((24, torch.float32), (5, torch.float32), (3, torch.int16), (64, torch.bfloat16)):
        x = torch.randn(4, 3000, d, generator=gen).to(dtype)
        perm = torch.stack([torch.randperm(3000, generator=gen) for _ in range(4)])
        for idx in (perm, perm.int()):
            g = lsh.gather_rows(x.to(device), idx.to(device))
            assert torch.equal(g.cpu(), torch.gather(x, 1, perm[..., None].expand(-1, -1, d)))
            inv = lsh.invert_permutation(idx.to(device))
            assert torch.equal(inv.cpu().long(), torch.argsort(perm, dim=-1))
            assert torch.equal(lsh.gather_rows(g, inv).cpu(), x)
            assert torch.equal(lsh.scatter_rows(g, idx.to(device)).cpu(), x)
    x = torch.randn(3000, 24, generator=gen)
    assert np.array_equal(_np(lsh.gather_rows(x.to(device), perm.int().to(device))),
                          ol.gather_rows(x.numpy(), perm.int().numpy()))


def test_reference_named_helpers(device):
    gen = torch.Generator().manual_seed(2)
    h, b, s, d, bucket = 3, 2, 600, 16, 100
    x = torch.randn(b, s, d, generator=gen)
    keys = torch.randn(h, b, s, generator=gen)
    perm = lsh.stable_argsort(keys.to(device)).long()
    assert torch.equal(perm.cpu(), keys.argsort(dim=-1, stable=True))
    sx = lsh.sort_to_buckets(x.to(device), perm, bucket)
    want = x[None].expand(h, -1, -1, -1).gather(-2, perm.cpu()[..., None].expand(-1, -1, -1, d))
    assert sx.shape == (h, b, s // bucket, bucket, d) and torch.equal(sx.cpu().reshape(h, b, s, d), want)
    back = lsh.unsort_from_buckets(sx, lsh.invert_permutation(perm))
    assert torch.equal(back.cpu(), x[None].expand(h, -1, -1, -1))
    p = lsh.pad_to_multiple(x, 256, dims=-2, value=float("inf"))
    assert p.shape == (b, 768, d) and torch.isinf(p[:, 600:]).all()


def test_e2lsh_and_lsh_mapping(device):
    torch.manual_seed(4)
    e = lsh.E2LSH(n_hashes=3, n_heads=2, dim=10).to(device)
    q, k = torch.randn(2, 5000, 10), torch.randn(2, 5000, 10)
    qh, kh, shift = lsh.lsh_mapping(e, q.to(device), k.to(device))
    a = e.alpha.detach().cpu()
    want_q = np.stack([ol.project(q[i].numpy(), a[i].numpy()) for i in range(2)], axis=1)  # [n_hashes, heads, N]
    assert qh.shape == (3, 2, 5000) and np.array_equal(_np(qh), want_q)
    ref_q, ref_k = torch.bmm(q, a).permute(2, 0, 1), torch.bmm(k, a).permute(2, 0, 1)
    assert torch.allclose(qh.cpu(), ref_q, atol=1e-5)
    ref_shift = torch.max(ref_q.max(-1, keepdim=True).values, ref_k.max(-1, keepdim=True).values) - \
        torch.min(ref_q.min(-1, keepdim=True).values, ref_k.min(-1, keepdim=True).values)
    assert shift.shape == (3, 2, 1) and torch.allclose(shift.cpu(), ref_shift, atol=1e-5)
    hh, sh = lsh.lsh_mapping1(e, q.to(device))
    assert torch.equal(hh, qh) and torch.allclose(sh.cpu(), ref_q.max(-1, keepdim=True).values - ref_q.min(-1, keepdim=True).values, atol=1e-5)


def test_lsh_ordering_bit_exact_and_unsort(device):
    torch.manual_seed(5)
    B, L, D = 2, 6000, 24
    mod = lsh.LSHOrdering(input_dim=4, num_hashes=3).to(device)
    coords = torch.stack([synth.collider_event(L, seed=s)[0] for s in range(B)])
    points = torch.randn(B, L, D)
    ordered, idx = mod(points.to(device), coords.to(device))
    alpha = mod.e2lsh.alpha.detach().cpu()[0].numpy()
    for b in range(B):
        want = ol.lsh_ordering(coords[b].numpy(), alpha)
        assert np.array_equal(_np(idx[b]), want.astype(np.int64))
    assert idx.dtype == torch.int64
    assert torch.equal(ordered.cpu(), points.gather(1, idx.cpu()[..., None].expand(-1, -1, D)))
    inv = lsh.invert_permutation(idx)
    assert torch.equal(inv.cpu(), idx.cpu().argsort(dim=1))
    assert torch.equal(lsh.gather_rows(ordered, inv).cpu(), points)


def test_bucket_sort_batch_of_events_bit_exact(device):
    """A batch of padded events in one set of launches equals the events one by one (and the oracle)."""
    n_max, lens = 7000, [7000, 1, 4097, 0, 6999]
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    coords = torch.zeros(len(lens), n_max, 4)
    feats = torch.zeros(len(lens), n_max, 24)
    for e, n in enumerate(lens):
        c, f, _ = synth.collider_event(n_max, seed=10 + e)
        coords[e], feats[e] = c, f
    got = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.5, 3, 4, feats.to(device),
                              n_valid=torch.tensor(lens, dtype=torch.int32))
    for e, n in enumerate(lens):
        want = ol.bucket_sort(coords[e].numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats[e].numpy(), n_valid=n)
        for name in ("ids", "meta", "keys", "perm", "feats"):
            assert np.array_equal(_np(got[name][e]), want[name]), (name, e)
    full = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.5, 3, 4, feats.to(device))
    one = lsh.lsh_bucket_sort(coords[2].to(device), alpha.to(device), beta.to(device), 0.5, 3, 4, feats[2].to(device))
    for name in ("ids", "meta", "keys", "perm", "feats"):
        assert torch.equal(full[name][2], one[name]), name


def test_bucket_sort_batch_of_nine_events_matches_single_events(device):
    """Eight or more events take the launch forms that keep an event (and a sort segment) on one XCD."""
    n, n_events = 5000, 9
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    coords = torch.stack([synth.collider_event(n, seed=20 + e)[0] for e in range(n_events)])
    feats = torch.stack([synth.collider_event(n, seed=20 + e)[1] for e in range(n_events)])
    lens = torch.tensor([5000, 4999, 1, 0, 2048, 2049, 5000, 77, 4096], dtype=torch.int32)
    got = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.5, 3, 4, feats.to(device), n_valid=lens)
    for e in range(n_events):
        want = ol.bucket_sort(coords[e].numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats[e].numpy(),
                              n_valid=int(lens[e]))
        for name in ("ids", "meta", "keys", "perm", "feats"):
            assert np.array_equal(_np(got[name][e]), want[name]), (name, e)


def test_one_launch_and_separate_kernels_agree(device):
    """The stage has two forms: one kernel whose workgroups wait for each other (calls that fit the GPU at once) and
    separate kernels (everything else). The same event through both must give the same bits: alone (one launch), as
    one of 32 copies (96 tables: separate kernels), and with feature rows of 100 bytes (not 16-byte pieces: separate
    kernels); three calls in a row reuse the same workspace memory, whose flags the kernel never clears."""
    n = 30011
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    coords, feats, _ = synth.collider_event(n, seed=5)
    cd, fd, ad, bd = coords.to(device), feats.to(device), alpha.to(device), beta.to(device)
    want = ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats.numpy())
    for _ in range(3):
        one = lsh.lsh_bucket_sort(cd, ad, bd, 0.5, 3, 4, fd, strict=True)
        for name in ("ids", "meta", "keys", "perm", "feats"):
            assert np.array_equal(_np(one[name]), want[name]), name
    many = lsh.lsh_bucket_sort(cd[None].expand(32, -1, -1).contiguous(), ad, bd, 0.5, 3, 4,
                               fd[None].expand(32, -1, -1).contiguous(), strict=True)
    for name in ("ids", "meta", "keys", "perm", "feats"):
        assert torch.equal(many[name][0], one[name]) and torch.equal(many[name][31], one[name]), name
    f25 = torch.cat([fd, fd[:, :1]], dim=1)
    odd = lsh.lsh_bucket_sort(cd, ad, bd, 0.5, 3, 4, f25, strict=True)
    assert torch.equal(odd["perm"], one["perm"]) and torch.equal(odd["feats"][..., :24], one["feats"])
    # 12 tables of padded events: one launch of 360 workgroups of 512 threads (the library's own choice; the 768-thread
    # form does not hold 480 workgroups at once and leaves the call to the separate kernels)
    wants = [ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats.numpy(), n_valid=nv)
             for nv in [n, 17, 0, 2049]]
    try:
        for tile in (0, 768, 1024):
            lsh.one_launch_config(tile=tile)
            four = lsh.lsh_bucket_sort(cd[None].expand(4, -1, -1).contiguous(), ad, bd, 0.5, 3, 4,
                                       fd[None].expand(4, -1, -1).contiguous(), n_valid=torch.tensor([n, 17, 0, 2049]),
                                       strict=True)
            for e, w in enumerate(wants):
                for name in ("ids", "meta", "keys", "perm", "feats"):
                    assert np.array_equal(_np(four[name][e]), w[name]), (tile, name, e)
    finally:
        lsh.one_launch_config()


def test_one_launch_kernel_on_changing_sizes_shares_one_workspace(device):
    """The words that the tiles of the one-launch kernel hand to each other carry the launch and the step in their
    upper half and are never cleared: launches of different sizes, event counts and tile forms, one after the other
    on the same workspace memory, must each give the bits of the separate kernels."""
    import random

    rnd = random.Random(5)
    alpha, beta = synth.lsh_params(4, 3, 4, 1.0, 1)
    ad, bd = alpha.to(device), beta.to(device)
    sizes = [1, 63, 65, 767, 768, 769, 1023, 1025, 2048, 5000, 12345, 30000, 45000, 60000, 61234]
    try:
        for it in range(48):
            n = rnd.choice(sizes)
            ev = rnd.choice([1, 1, 2]) if n <= 45000 else 1
            gen = torch.Generator().manual_seed(it)
            coords = (torch.randn(ev, n, 4, generator=gen) * rnd.choice([0.3, 1.0, 3.0])).to(device)
            feats = torch.randn(ev, n, 24, generator=gen).to(device)
            tile = rnd.choice([0, 0, 768, 1024])
            lsh.one_launch_config(True, tile=tile)
            one = lsh.lsh_bucket_sort(coords, ad, bd, 1.0, 3, 4, feats, strict=True)
            lsh.one_launch_config(False)
            sep = lsh.lsh_bucket_sort(coords, ad, bd, 1.0, 3, 4, feats, strict=True)
            for name in ("ids", "meta", "keys", "perm", "feats"):
                assert torch.equal(one[name], sep[name]), (it, n, ev, tile, name)
    finally:
        lsh.one_launch_config()


def test_one_launch_generic_dim_and_wide_keys(device):
    """dim 3 (the generic coordinate path) and a bucket width that makes the keys need three radix passes."""
    n = 9000
    gen = torch.Generator().manual_seed(3)
    coords = torch.randn(n, 3, generator=gen) * 3
    alpha = torch.randn(3, 6, generator=gen)
    beta = torch.rand(6, generator=gen) * 0.05
    feats = torch.randn(n, 8, generator=gen)
    got = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.05, 2, 3, feats.to(device))
    want = ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.05, 2, 3, feats.numpy())
    assert int(want["meta"][:, -2].max()) > 22 and not want["meta"][:, -1].any()  # more than two 11-bit digits
    for name in ("ids", "meta", "keys", "perm", "feats"):
        assert np.array_equal(_np(got[name]), want[name]), name


@pytest.mark.parametrize("n_events", [3, 30])
def test_valid_counts_outside_the_event_are_cut(device, n_events):
    """Per-event valid counts live in device memory, so the library cannot refuse bad ones: a count beyond the event is
    taken as the event's length, a negative one as zero (both forms of the stage: 9 and 90 tables)."""
    n = 3000
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    coords = torch.stack([synth.collider_event(n, seed=40 + e)[0] for e in range(n_events)])
    feats = torch.stack([synth.collider_event(n, seed=40 + e)[1] for e in range(n_events)])
    lens = torch.tensor([n + 5000, -7, 17] * (n_events // 3), dtype=torch.int32)
    got = lsh.lsh_bucket_sort(coords.to(device), alpha.to(device), beta.to(device), 0.5, 3, 4, feats.to(device), n_valid=lens)
    for e in range(n_events):
        nv = min(n, max(0, int(lens[e])))
        want = ol.bucket_sort(coords[e].numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats[e].numpy(), n_valid=nv)
        for name in ("ids", "meta", "keys", "perm", "feats"):
            assert np.array_equal(_np(got[name][e]), want[name]), (name, e)


def test_one_launch_give_up_path_poisons_the_outputs(device):
    """The workgroups of the one-launch kernel wait for each other with a bounded number of polls. A limit of zero
    polls (set from the host; every kernel still ends normally) makes every wait give up: the tables' flag fields then
    carry bit 1, the permutations are all -1 and the sorted features all zero, ``strict=True`` raises, and the block's
    ordering step falls back to the separate kernels. Afterwards the default limit gives the exact result again."""
    from lampa_amd import block as lb
    from lampa_amd._capi import LampaError

    n = 20000
    alpha, beta = synth.lsh_params(4, 3, 4, 0.5, 1)
    coords, feats, _ = synth.collider_event(n, seed=9)
    cd, fd, ad, bd = coords.to(device), feats.to(device), alpha.to(device), beta.to(device)
    want = ol.bucket_sort(coords.numpy(), alpha.numpy(), beta.numpy(), 0.5, 3, 4, feats.numpy())
    try:
        lsh.one_launch_config(wait_limit=0)
        got = lsh.lsh_bucket_sort(cd, ad, bd, 0.5, 3, 4, fd)
        torch.cuda.synchronize()
        flags = lsh.decode_meta_flags(got["meta"])
        assert bool(flags["gave_up"].all())
        assert bool((got["perm"] == -1).all()) and bool((got["feats"] == 0).all())
        assert np.array_equal(_np(got["ids"]), want["ids"])  # the bucket ids depend on no other workgroup
        with pytest.raises(LampaError, match="gave up"):
            lsh.lsh_bucket_sort(cd, ad, bd, 0.5, 3, 4, fd, strict=True)
        # the block reads the flag once per event and sorts again with the separate kernels
        blk = lb.LshgdBlock().to(device)
        lsh.one_launch_config(wait_limit=0)
        order = blk.order(cd)
        blk_alpha, blk_beta = blk.lsh_alpha.cpu().numpy(), blk.lsh_beta.cpu().numpy()
        assert np.array_equal(_np(order), ol.bucket_sort(coords.numpy(), blk_alpha, blk_beta, 0.5, 3, 4)["perm"][0])
        # the whole block: it looks at the flags after queuing its launches and runs again with that order
        torch.manual_seed(2)
        blk16 = lb.LshgdBlock().to(device).to(torch.bfloat16)
        lsh.one_launch_config()
        want_out = blk16(fd, cd)
        lsh.one_launch_config(wait_limit=0)
        got_out = blk16(fd, cd)
        assert torch.equal(got_out, want_out) and bool(torch.isfinite(got_out.float()).all())
    finally:
        lsh.one_launch_config()
    again = lsh.lsh_bucket_sort(cd, ad, bd, 0.5, 3, 4, fd, strict=True)
    for name in ("ids", "meta", "keys", "perm", "feats"):
        assert np.array_equal(_np(again[name]), want[name]), name
