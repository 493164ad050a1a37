"""The sort entry point that allocates nothing (ha_bucket_argsort_static) against ha_bucket_argsort:
same permutations, bit for bit, on two calls in a row that share the library's built-in scratch
array, the second on a smaller input (so stale histograms of the first call lie behind it)."""
import ctypes

import numpy as np
import pytest
import torch

from hyperattention_amd import _lib

pytestmark = pytest.mark.gpu


def _sort_both(keys, seg_len, seg_stride, seg_offset, num_segments, num_keys, idx_dtype):
    L = _lib.lib()
    dev = keys.device
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    code = 0 if idx_dtype == torch.int32 else 1
    want = torch.empty((num_segments, seg_len), device=dev, dtype=idx_dtype)
    ws_bytes = L.ha_bucket_argsort_workspace_bytes(num_segments, seg_len, num_keys)
    ws = torch.empty(max(int(ws_bytes), 256), device=dev, dtype=torch.uint8)
    _lib.check(L.ha_bucket_argsort(keys.data_ptr(), want.data_ptr(), code, num_segments, seg_len, seg_stride,
                                   seg_offset, num_keys, ws.data_ptr(), ws.numel(), stream))
    got = torch.full((num_segments, seg_len), -1, device=dev, dtype=idx_dtype)
    # the first call on a device looks up the scratch array's address (and may make the runtime load it); from
    # then on neither torch's allocator nor the driver (hipMemGetInfo) may see the device's memory change
    _lib.check(L.ha_bucket_argsort_static(keys.data_ptr(), got.data_ptr(), code, num_segments, seg_len, seg_stride,
                                          seg_offset, num_keys, stream))
    got.fill_(-1)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]
    _lib.check(L.ha_bucket_argsort_static(keys.data_ptr(), got.data_ptr(), code, num_segments, seg_len, seg_stride,
                                          seg_offset, num_keys, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before, "the driver saw an allocation during the call"
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_sort_matches_the_workspace_sort_twice_in_a_row():
    g = torch.Generator().manual_seed(7)
    # first call: 24 segments of 20000 keys (5 chunks each, ragged last chunk), skewed 8-bit keys
    n1, segs1 = 20000, 24
    keys1 = (torch.randint(0, 256, (segs1, n1), generator=g) * torch.randint(0, 2, (segs1, n1), generator=g)).int()
    got, want = _sort_both(keys1.cuda(), n1, n1, 0, segs1, 256, torch.int32)
    assert np.array_equal(got, want)
    ref = np.argsort(keys1.numpy(), axis=1, kind="stable")
    assert np.array_equal(got, ref)
    # second call, smaller, two key bytes (uses the intermediate orders in the scratch array too), second
    # halves of the rows as segments, int64 output
    n2, segs2 = 9000, 3
    keys2 = torch.randint(0, 1000, (segs2, 2 * n2), generator=g).int()
    got, want = _sort_both(keys2.cuda(), n2, 2 * n2, n2, segs2, 1024, torch.int64)
    assert np.array_equal(got, want)
    ref = np.argsort(keys2.numpy()[:, n2:], axis=1, kind="stable")
    assert np.array_equal(got, ref)


def test_static_scratch_sort_rejects_what_does_not_fit():
    L = _lib.lib()
    keys = torch.zeros(16, device="cuda", dtype=torch.int32)
    st = L.ha_bucket_argsort_static(keys.data_ptr(), keys.data_ptr(), 0, 4096, 1 << 20, 1 << 20, 0, 256, None)
    assert st == -6 and b"scratch" in L.ha_last_error()
