"""Host-side checks that run without a GPU: the C-ABI library loads, exports every symbol the header declares,
and its host-only planning logic is right. No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

from lampa_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_capi.LIB_PATH):
        from lampa_amd import build

        build.build(verbose=False)
    return _capi.lib()


def _declared():
    text = open(os.path.join(ROOT, "include", "lampa_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lampa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = _declared()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/lampa_amd.h but not exported"
    assert sorted(_capi.exported_symbols()) == names  # the ctypes binding covers the whole header


def test_workspace_queries_and_argument_errors(lib):
    assert lib.lampa_sort_workspace_bytes(3, 60000) > 4 * 3 * 60000 * 4
    assert lib.lampa_sort_workspace_bytes(0, 10) == -1
    assert lib.lampa_lsh_bucket_workspace_bytes(60000, 3, 4) >= 235 * 12 * 8
    assert lib.lampa_gdr_chunk_workspace_bytes(938, 60, 8, 64, 64) > 938 * 8 * 3 * 32 * 32 * 2  # three 32x32 blocks of T per chunk and head
    assert lib.lampa_gdr_chunk_workspace_bytes(938, 60, 8, 48, 64) == -4  # unsupported head size
    # null pointers / bad sizes are rejected before any launch
    assert lib.lampa_sort_pairs(None, 0, None, 1, 10, 32, None, 1, 0, None, None, 0, None) == -1
    assert lib.lampa_gather_rows(None, 1, 1, None, 4, 1, 1, 4, None, None) == -1
    assert lib.lampa_gdr_recurrent_fwd(*([None] * 9), 1, 1, 1, 1, 64, 64, 0, 1.0, 0, None) == -1


def _plan(lib, cu, cps):
    arr = (ctypes.c_int64 * len(cu))(*cu)
    size = lib.lampa_gdr_plan_size(arr, len(cu) - 1, cps)
    assert size > 0
    plan = torch.zeros(size, dtype=torch.int32)
    assert lib.lampa_gdr_plan_fill(arr, len(cu) - 1, cps, ctypes.c_void_p(plan.data_ptr())) == 0
    return plan.tolist()


def test_plan_tables(lib):
    cu = [0, 5, 69, 69, 199, 60199]
    p = _plan(lib, cu, 16)
    n_seq, chunks, segs, cps = p[0:4]
    lens = [b - a for a, b in zip(cu[:-1], cu[1:])]
    want_chunks = [(l + 63) // 64 for l in lens]
    assert (n_seq, chunks, cps) == (5, sum(want_chunks), 16)
    tok0 = p[p[4]:p[4] + chunks]
    clen = p[p[5]:p[5] + chunks]
    seg_c0, seg_nc = p[p[6]:p[6] + segs], p[p[7]:p[7] + segs]
    seg_seq, seg_flags = p[p[8]:p[8] + segs], p[p[9]:p[9] + segs]
    seq_seg0, seq_nseg = p[p[10]:p[10] + n_seq], p[p[11]:p[11] + n_seq]
    # chunks tile every sequence exactly and never straddle a boundary (index.py:69-83)
    covered = []
    for t, l in zip(tok0, clen):
        assert 1 <= l <= 64
        covered.extend(range(t, t + l))
    assert covered == list(range(cu[-1]))
    for t, l in zip(tok0, clen):
        s = max(i for i in range(n_seq) if cu[i] <= t and lens[i] > 0)
        assert t + l <= cu[s + 1] and (t - cu[s]) % 64 == 0
    # segments partition the chunks of their sequence; flags mark first / last
    assert sum(seg_nc) == chunks and seq_nseg == [max(1, (c + 15) // 16) for c in want_chunks]
    for s in range(n_seq):
        mine = [g for g in range(segs) if seg_seq[g] == s]
        assert mine == list(range(seq_seg0[s], seq_seg0[s] + seq_nseg[s]))
        assert seg_flags[mine[0]] & 1 and seg_flags[mine[-1]] & 2
        assert all(seg_nc[g] <= 16 for g in mine) and sum(seg_nc[g] for g in mine) == want_chunks[s]
    assert p[12] == cu[-1]
    # the order the segment kernels take the segments in: every segment once, the longest first, ties in plan order
    order = p[p[13]:p[13] + segs]
    assert sorted(order) == list(range(segs))
    assert order == sorted(range(segs), key=lambda g: -seg_nc[g])


def test_balanced_plan_tables(lib):
    """Segments of nearly equal length over all sequences: the greedy deal minimises the longest segment (checked
    against brute force over the segment counts), a sequence's segments differ by at most one chunk and tile it in
    order, empty sequences keep their one empty segment, and the default segmentation of a batch that needs several
    rounds of workgroups asks for a whole number of rounds."""
    import itertools
    from lampa_amd import gated_delta as gd

    def plan(cu, total):
        arr = (ctypes.c_int64 * len(cu))(*cu)
        size = lib.lampa_gdr_plan_size_balanced(arr, len(cu) - 1, total)
        assert size > 0
        p = torch.zeros(size, dtype=torch.int32)
        assert lib.lampa_gdr_plan_fill_balanced(arr, len(cu) - 1, total, ctypes.c_void_p(p.data_ptr())) == 0
        return p.tolist()

    cu = [0, 5, 69, 69, 1000, 60199, 60200]
    lens = [b - a for a, b in zip(cu[:-1], cu[1:])]
    nc = [(l + 63) // 64 for l in lens]
    for total in (1, 6, 7, 13, 40, 5000):
        p = plan(cu, total)
        n_seq, chunks, segs, cps = p[0:4]
        assert (n_seq, chunks, cps) == (6, sum(nc), 0)
        assert segs == min(max(total, n_seq), sum(max(c, 1) for c in nc))
        seg_c0, seg_nc = p[p[6]:p[6] + segs], p[p[7]:p[7] + segs]
        seg_seq, seg_flags = p[p[8]:p[8] + segs], p[p[9]:p[9] + segs]
        seq_seg0, seq_nseg = p[p[10]:p[10] + n_seq], p[p[11]:p[11] + n_seq]
        c = 0
        for s in range(n_seq):
            mine = list(range(seq_seg0[s], seq_seg0[s] + seq_nseg[s]))
            assert [g for g in range(segs) if seg_seq[g] == s] == mine
            assert seg_flags[mine[0]] & 1 and seg_flags[mine[-1]] & 2
            assert all(not (seg_flags[g] & 3) for g in mine[1:-1])
            sizes = [seg_nc[g] for g in mine]
            assert sum(sizes) == nc[s] and max(sizes) - min(sizes) <= 1 and sizes == sorted(sizes, reverse=True)
            for g in mine:  # in order, without gaps
                assert seg_c0[g] == c
                c += seg_nc[g]
        order = p[p[13]:p[13] + segs]
        assert order == sorted(range(segs), key=lambda g: -seg_nc[g])
        if segs <= 13:  # brute force: no other split of `segs` segments has a shorter longest segment
            longest = max(seg_nc)
            live = [i for i in range(n_seq) if nc[i] > 0]
            best = min(max(-(-nc[i] // k) for i, k in zip(live, ks))
                       for ks in itertools.product(range(1, segs + 1), repeat=len(live))
                       if sum(ks) + (n_seq - len(live)) == segs and all(k <= nc[i] for i, k in zip(live, ks)))
            assert longest == best
    assert lib.lampa_gdr_plan_size_balanced((ctypes.c_int64 * 2)(0, 10), 1, 0) == -1
    assert lib.lampa_gdr_plan_size_balanced((ctypes.c_int64 * 3)(0, 10, 5), 2, 4) == -1
    # default segmentation: several rounds -> whole rounds of balanced segments; one round with one workgroup per CU ->
    # one fixed length; one round with two per CU -> the first half of a sequence's segments longer than the second
    assert gd._default_segmentation([938], 8, 256, 1) == ("cps", 30)
    nc4 = [819, 830, 564, 635, 735, 659, 314, 205, 404, 189, 231, 755, 500, 434, 203, 655]
    assert gd._default_segmentation(nc4, 8, 256, 1) == ("balanced", 128)
    assert gd._default_segmentation([300] * 4, 8, 256, 1) == ("cps", 38)       # one round of 38-chunk segments holds it
    assert gd._default_segmentation([600] * 4, 8, 256, 1) == ("balanced", 64)  # 1.2 rounds of 64 chunks -> 2 of 37-38
    kind, lens = gd._default_segmentation([938], 8, 512, 2)
    assert kind == "lengths" and len(lens) == 64 and sum(lens) == 938
    assert lens[:32] == [17] * 32 and set(lens[32:]) == {12, 13} and lens[32:] == sorted(lens[32:], reverse=True)
    kind, lens = gd._default_segmentation([235, 0, 700], 8, 512, 2)
    assert kind == "lengths" and len(lens) == 64 and min(lens[:16]) > 0 and lens[16] == 0
    assert sum(lens[:16]) == 235 and sum(lens[17:]) == 700
    assert gd._default_segmentation([3, 0, 7], 8, 512, 2) == ("cps", 4)      # short sequences: 4-chunk segments


def test_plan_with_given_segment_lengths(lib):
    cu = [0, 64 * 10, 64 * 10, 64 * 10 + 1000]
    nc = [10, 0, 16]

    def plan(lens):
        arr = (ctypes.c_int64 * len(cu))(*cu)
        la = (ctypes.c_int32 * len(lens))(*lens)
        size = lib.lampa_gdr_plan_size_lengths(arr, 3, la, len(lens))
        if size < 0:
            return size
        p = torch.zeros(size, dtype=torch.int32)
        assert lib.lampa_gdr_plan_fill_lengths(arr, 3, la, len(lens), ctypes.c_void_p(p.data_ptr())) == 0
        return p.tolist()

    lens = [4, 3, 3, 0, 7, 5, 4]
    p = plan(lens)
    n_seq, chunks, segs, cps = p[0:4]
    assert (n_seq, chunks, segs, cps) == (3, 26, 7, 0)
    assert p[p[7]:p[7] + segs] == lens
    assert p[p[6]:p[6] + segs] == [0, 4, 7, 10, 10, 17, 22]
    assert p[p[8]:p[8] + segs] == [0, 0, 0, 1, 2, 2, 2]
    assert p[p[9]:p[9] + segs] == [1, 0, 2, 3, 1, 0, 2]
    assert p[p[10]:p[10] + 3] == [0, 3, 4] and p[p[11]:p[11] + 3] == [3, 1, 3]
    assert p[p[13]:p[13] + segs] == [4, 5, 0, 6, 1, 2, 3]  # longest first, ties in plan order
    # lengths that do not tile the sequences are refused
    for bad in ([4, 3, 4, 0, 7, 5, 4], [4, 3, 3, 7, 5, 4], [4, 3, 3, 0, 7, 5, 3], [4, 3, 3, 0, 7, 5, 4, 1], [10, 0, 0, 16],
                [4, 3, 3, 0, 7, -1, 10]):
        assert plan(bad) == -1, bad


def test_plan_rejects_bad_input(lib):
    bad = (ctypes.c_int64 * 3)(0, 10, 5)
    assert lib.lampa_gdr_plan_size(bad, 2, 4) == -1
    ok = (ctypes.c_int64 * 2)(0, 10)
    assert lib.lampa_gdr_plan_size(ok, 1, 0) == -1


def test_hierarchical_forward_argument_checks(lib):
    """Every check of lampa_hgdn_chunk_fwd runs on the host before the first launch (dummy, never dereferenced
    device addresses; the plan is real)."""
    # at least the chunk records (5376 B), the walk records (> 16 KiB) and two fp32 K x V tiles per chunk and head
    assert lib.lampa_hgdn_chunk_workspace_bytes(938, 30, 8, 64, 64) > 938 * 8 * (5376 + 16 * 1024 + 2 * 64 * 64 * 4)
    assert lib.lampa_hgdn_chunk_workspace_bytes(938, 30, 8, 128, 128) == -4
    assert lib.lampa_hgdn_chunk_workspace_bytes(-1, 30, 8, 64, 64) == -1
    d = ctypes.c_void_p(0x1000)  # 16-byte aligned dummy

    def call(cu, cps, L=20, K=64, V=64, q=d, ws=None, dtype=0, lam_dtype=0, states=None):
        arr = (ctypes.c_int64 * len(cu))(*cu)
        size = lib.lampa_gdr_plan_size(arr, len(cu) - 1, cps)
        plan = torch.zeros(size, dtype=torch.int32)
        assert lib.lampa_gdr_plan_fill(arr, len(cu) - 1, cps, ctypes.c_void_p(plan.data_ptr())) == 0
        return lib.lampa_hgdn_chunk_fwd(q, d, d, d, d, d, lam_dtype, 0.125, d, states, ctypes.c_void_p(plan.data_ptr()), d, 2, 2, K, V, L, dtype,
                                        0.125, 1, ws, 0, None)

    assert call([0, 4096], 8, q=None) == -1                      # null pointer
    assert call([0, 4096], 8, q=ctypes.c_void_p(0x1008)) == -1   # misaligned
    assert call([0, 4096], 8, K=128) == -4                       # head size
    assert call([0, 4096], 8, dtype=2) == -4                     # fp32 inputs
    assert call([0, 4096], 8, lam_dtype=3) == -1                 # unknown type of the level weights
    assert call([0, 4096], 12) == -1                             # split sequences need a power-of-two segment length
    assert call([0, 4096], 8, L=12) == -1                        # 64 chunks need 7 + 6 levels
    assert call([0, 4096], 8, L=13) == -2                        # all checks passed: the workspace is missing
    assert call([0, 4096], 100, L=13) == -2                      # one segment per sequence: any segment length
    assert call([0, 64 * 4097], 4096, L=32) == -4                # more than 4096 chunks in a sequence
    assert call([0, 64 * 4096], 4096, L=19) == -2
    assert call([0, 4096, 8192], 8, L=13, states=d) == -2         # level states: equal whole-chunk sequences
    assert call([0, 4096, 8000], 8, L=13, states=d) == -1
    assert call([0, 4000], 8, L=13) == -1                        # a ragged last chunk
    assert call([0, 4096, 12288], 8, L=14, states=d) == -1
    # the single-token step
    assert lib.lampa_hgdn_step(d, d, d, d, d, d, 0, 0.125, d, d, 2, 2, 2, 64, 64, 13, 13, 0, 0.125, 1, None) == -1  # z < L
    assert lib.lampa_hgdn_step(d, d, d, d, d, d, 0, 0.125, d, d, 2, 2, 2, 64, 64, 40, 1, 0, 0.125, 1, None) == -4     # more than 32 levels
    assert lib.lampa_hgdn_step(d, d, d, d, d, d, 0, 0.125, d, d, 0, 2, 2, 64, 64, 13, 0, 0, 0.125, 1, None) == 0     # empty batch


def test_operators_refuse_cpu_tensors():
    from lampa_amd import gated_delta as gd
    from lampa_amd import lsh

    x = torch.zeros(1, 64, 2, 64, dtype=torch.bfloat16)
    g = torch.zeros(1, 64, 2)
    with pytest.raises(_capi.LampaError):
        gd.chunk_gated_delta_rule(x, x, x, g, g)
    with pytest.raises(_capi.LampaError):
        lsh.stable_argsort(torch.zeros(4, dtype=torch.int32))


def test_gated_delta_shape_checks_come_before_any_gpu_work():
    # g and beta must be [B, T, HV]; the token-serial operator also takes a headwise beta [B, T, HV, V]
    # (gated_delta_rule_ori.py:444-447), the chunk operator does not (its assert on beta's rank comes first, as in the
    # reference); a CPU tensor is refused after the shape checks
    from lampa_amd import gated_delta as gd

    q = torch.zeros(1, 64, 2, 64, dtype=torch.bfloat16)
    v = torch.zeros(1, 64, 4, 64, dtype=torch.bfloat16)
    g = torch.zeros(1, 64, 4)
    with pytest.raises(_capi.LampaError):  # headwise beta passes the shape checks and reaches the device check
        gd.fused_recurrent_gated_delta_rule(q, q, v, g, torch.zeros(1, 64, 4, 64))
    with pytest.raises(ValueError, match="one value per value column"):
        gd.fused_recurrent_gated_delta_rule(q, q, v, g, torch.zeros(1, 64, 4, 32))
    with pytest.raises(AssertionError, match="beta must be of shape"):
        gd.chunk_gated_delta_rule(q, q, v, g, torch.zeros(1, 64, 4, 64))
    with pytest.raises(ValueError, match="g must have shape"):
        gd.fused_recurrent_gated_delta_rule(q, q, v, g[:, :, :2], g)
    with pytest.raises(ValueError, match="g must have shape"):
        gd.chunk_gated_delta_rule(q, q, v, g, g[:, :32])
    with pytest.raises(ValueError, match="multiple of the number"):
        gd.chunk_gated_delta_rule(q, q, v[:, :, :3], g[:, :, :3], g[:, :, :3])
    with pytest.raises(ValueError, match="expected q, k"):
        gd.chunk_gated_delta_rule(q, q[:, :32], v, g, g)


def test_static_sort_symbols_and_limit():
    lib = _capi.lib()
    assert lib.lampa_sort_pairs_static_max_bytes() == 8 << 20
    assert lib.lampa_sort_workspace_bytes(3, 60000) <= lib.lampa_sort_pairs_static_max_bytes()
    d = ctypes.c_void_p(0x1000)
    # argument and size checks run before anything touches the GPU
    assert lib.lampa_sort_pairs_static(None, 1, None, 1, 10, 32, None, 1, 0, d, None) == -1
    assert lib.lampa_sort_pairs_static(d, 7, None, 1, 10, 32, None, 1, 0, d, None) == -1
    assert lib.lampa_sort_pairs_static(d, 1, None, 3, 400000, 32, None, 1, 0, d, None) == -2
    assert lib.lampa_sort_pairs_static(d, 1, None, 3, 0, 32, None, 1, 0, d, None) == 0


def test_backward_argument_checks_and_tables(lib):
    """lampa_gdr_bwd refuses bad arguments before any GPU work; the workspace grows with its parts; the tables of the
    pass that runs backwards give every sequence one extra row and count its segments from the end."""
    from lampa_amd import gated_delta as gd
    small = lib.lampa_gdr_bwd_workspace_bytes(1024, 1, 4, 2, 64, 64)
    # maps, start states, reverse maps, end states, a state per 8 tokens, the partial dq / dk per 16-column slab
    assert small > 4 * (4 * 2 * 64 * 128 + 4 * 2 * 64 * 64 + 5 * 2 * 64 * 128 + 5 * 2 * 64 * 64
                        + 128 * 2 * 64 * 64 + 2 * 4 * 1024 * 2 * 64)
    assert lib.lampa_gdr_bwd_workspace_bytes(2048, 1, 4, 2, 64, 64) > small
    assert lib.lampa_gdr_bwd_workspace_bytes(1024, 1, 4, 2, 256, 64) == -1
    nulls = [None] * 18
    assert lib.lampa_gdr_bwd(*nulls, 16, 1, 1, 1, 1, 64, 64, 0, 1.0, 0, None, 0, None) == -1
    fake = [ctypes.c_void_p(4096)] * 18  # never dereferenced: the checks below come first
    assert lib.lampa_gdr_bwd(*fake, 16, 1, 1, 1, 1, 62, 64, 0, 1.0, 0, None, 0, None) == -4   # K not a multiple of 4
    assert lib.lampa_gdr_bwd(*fake, 16, 1, 1, 1, 1, 256, 64, 0, 1.0, 0, None, 0, None) == -4  # K > 128
    assert lib.lampa_gdr_bwd(*fake, 16, 1, 1, 3, 4, 64, 64, 0, 1.0, 0, None, 0, None) == -1   # HV not a multiple of H
    assert lib.lampa_gdr_bwd(*fake, 16, 1, 1, 1, 1, 64, 64, 0, 1.0, 3, None, 0, None) == -1   # unknown normalisation
    assert lib.lampa_gdr_bwd(*fake, 16, 1, 1, 1, 1, 64, 64, 0, 1.0, 0, None, 0, None) == -2   # no workspace
    cu_seg, seq_seg0, rev0, seg_rev, n_seg = gd._backward_tables([0, 0, 130, 194], 64, "cpu")
    assert n_seg == 5 and cu_seg.tolist() == [0, 0, 64, 128, 130, 194]
    assert seq_seg0.tolist() == [0, 1, 4, 5] and rev0.tolist() == [0, 2, 6, 8]
    assert seg_rev.tolist() == [0, 4, 3, 2, 6]  # every sequence's last segment on its first row


def test_lsh_meta_flag_decoding():
    """Bits of the last field of a table's meta row: 1 = the packed key overflowed 32 bits, 2 = a workgroup of the
    one-launch kernel gave up a wait (host-side decoding; the GPU test forces the second one)."""
    import torch

    from lampa_amd import lsh

    meta = torch.zeros(2, 3, 11, dtype=torch.int32)
    meta[0, 1, -1], meta[1, 0, -1], meta[1, 2, -1] = 1, 2, 3
    flags = lsh.decode_meta_flags(meta)
    assert flags["key_overflow"].tolist() == [[False, True, False], [False, False, True]]
    assert flags["gave_up"].tolist() == [[False, False, False], [True, False, True]]
    with pytest.raises(lsh.LampaError, match="gave up"):
        lsh._raise_on_overflow(meta, True)
    with pytest.raises(lsh.LampaError, match="overflow"):
        lsh._raise_on_overflow(meta[0], True)
    lsh._raise_on_overflow(meta, False)
    assert (lsh.META_KEY_OVERFLOW, lsh.META_GAVE_UP) == (1, 2)


def test_sequence_boundaries_are_validated_on_the_host():
    """cu_seqlens index q, k, v and the outputs inside the kernels: a list that does not start at 0, decreases or does
    not end at the number of tokens is refused before anything is launched (forward, token-serial and backward
    launchers all take their boundaries from this function)."""
    import torch

    from lampa_amd import gated_delta as gd

    assert gd._sequence_bounds(None, 2, 5) == [0, 5, 10]
    assert gd._sequence_bounds(torch.tensor([0, 3, 3, 10]), 1, 10) == [0, 3, 3, 10]
    for bad in ([1, 4, 10], [0, 4, 11], [0, 4, 9], [0, 6, 4, 10], [10], [0, -1, 10]):
        with pytest.raises(ValueError, match="cu_seqlens"):
            gd._sequence_bounds(torch.tensor(bad), 1, 10)
    import inspect
    for launcher in (gd._chunk_launch, gd._recurrent_launch, gd._backward_launch):
        assert "_sequence_bounds" in inspect.getsource(launcher)
    # the validated list is remembered per tensor object and version: the same tensor is not read again (reading a device
    # tensor drains the stream), an in-place change is seen, another token count is checked afresh
    cu = torch.tensor([0, 4, 10])
    first = gd._sequence_bounds(cu, 1, 10)
    assert gd._sequence_bounds(cu, 1, 10) is first
    with pytest.raises(ValueError, match="cu_seqlens"):
        gd._sequence_bounds(cu, 1, 12)
    cu[1] = 11
    with pytest.raises(ValueError, match="cu_seqlens"):
        gd._sequence_bounds(cu, 1, 10)
    cu[1] = 7
    assert gd._sequence_bounds(cu, 1, 10) == [0, 7, 10]


def test_bench_reads_the_traffic_table_of_the_committed_profile():
    """bench.py takes `roofline.traffic` from the counter summary under profiles/: the four kernels of the layer must
    be in its table, with a commit stamp, and every summary must say which commit it was measured at."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    table, commit = bench.measured_traffic()
    assert re.fullmatch(r"[0-9a-f]{7,40}", commit or ""), commit
    for kernel in ("gdr_local_kernel", "gdr_segment_kernel<composite>", "gdr_scan2_kernel<group>",
                   "gdr_segment_kernel<output>"):
        assert table.get(kernel, 0) > 1e6, (kernel, table)
    # the output pass moves at least its algorithmic bytes (520 B per token and head at the headline shape)
    assert table["gdr_segment_kernel<output>"] >= 520 * 60000 * 8
    prof = os.path.join(ROOT, "profiles")
    for name in sorted(os.listdir(prof)):
        if name.endswith(".md"):
            text = open(os.path.join(prof, name)).read()
            assert re.search(r"^commit: [0-9a-f]{7,40}\b", text, flags=re.M), name
            assert "rocprofv3" in text, name
