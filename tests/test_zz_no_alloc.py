"""The sort entry point that allocates nothing (``lampa_sort_pairs_static``) against ``lampa_sort_pairs``.

Both are called through the C ABI on the same device buffers; results must be bit-identical. The static variant is
called twice in a row, the second time on a smaller input, because every call on a GPU reuses one fixed array inside
the library image and that array keeps the previous call's contents.
"""
import ctypes

import pytest
import torch

from lampa_amd import _capi
from lampa_amd._capi import check, ptr, stream_of

pytestmark = pytest.mark.gpu

KEY_U32, KEY_I32, KEY_F32 = 0, 1, 2


def _sort_workspace(keys, kind, segs, n, key_bits):
    lib = _capi.lib()
    out = torch.empty((segs, n), dtype=torch.int32, device=keys.device)
    ws_bytes = check(lib.lampa_sort_workspace_bytes(segs, n), "lampa_sort_workspace_bytes")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=keys.device)
    check(lib.lampa_sort_pairs(ptr(keys), kind, None, segs, n, key_bits, None, 1, 0, ptr(out), ptr(ws), ws_bytes,
                               stream_of(keys)), "lampa_sort_pairs")
    return out


def _sort_static(keys, kind, segs, n, key_bits, out):
    check(_capi.lib().lampa_sort_pairs_static(ptr(keys), kind, None, segs, n, key_bits, None, 1, 0, ptr(out),
                                              stream_of(keys)), "lampa_sort_pairs_static")


def test_static_sort_two_calls_match_workspace_sort(device):
    lib = _capi.lib()
    assert lib.lampa_sort_pairs_static_max_bytes() == 8 << 20
    gen = torch.Generator().manual_seed(11)
    cases = [
        (KEY_F32, 3, 60000, torch.randn((3, 60000), generator=gen), 32),                    # config-1 sized, 3 passes
        (KEY_I32, 2, 5000, torch.randint(-50, 50, (2, 5000), generator=gen, dtype=torch.int32), 32),  # smaller, ties
        (KEY_U32, 5, 777, torch.randint(0, 1 << 13, (5, 777), generator=gen, dtype=torch.int32), 13),  # 2 passes
    ]
    outs = []
    for kind, segs, n, keys, bits in cases:  # the static calls back to back, outputs preallocated: nothing allocates
        keys = keys.to(device)
        out = torch.full((segs, n), -1, dtype=torch.int32, device=device)
        outs.append((kind, segs, n, keys, bits, out))
    # one warm call first (the array's address is looked up on the first call on a device), then the property the
    # entry point exists for: with the outputs already there, the calls change neither the free device memory nor
    # what the framework's allocator has reserved
    _sort_static(outs[0][3], outs[0][0], outs[0][1], outs[0][2], outs[0][4], outs[0][5])
    torch.cuda.synchronize()
    free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    for kind, segs, n, keys, bits, out in outs:
        _sort_static(keys, kind, segs, n, bits, out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    for kind, segs, n, keys, bits, out in outs:
        want = _sort_workspace(keys, kind, segs, n, bits)
        assert torch.equal(out, want), (kind, segs, n)
        if kind != KEY_U32:  # and both agree with the library sort of the framework that owns the memory
            assert torch.equal(out.long(), torch.sort(keys, dim=-1, stable=True).indices)


def test_static_sort_rejects_oversized_input(device):
    lib = _capi.lib()
    segs, n = 3, 400000
    assert lib.lampa_sort_workspace_bytes(segs, n) > lib.lampa_sort_pairs_static_max_bytes()
    keys = torch.zeros((segs, 8), dtype=torch.int32, device=device)  # never read: the size check comes first
    out = torch.zeros((segs, 8), dtype=torch.int32, device=device)
    rc = lib.lampa_sort_pairs_static(ptr(keys), KEY_I32, None, segs, n, 32, None, 1, 0, ptr(out), stream_of(keys))
    assert rc == -2
    with pytest.raises(_capi.LampaError, match="workspace"):
        check(rc, "lampa_sort_pairs_static")
