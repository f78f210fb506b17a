"""The entry point that allocates nothing (ck_count_offsets_static) against ck_count_offsets, through the C ABI:
bit-exact counts / inclusive ends / exclusive starts on two calls in a row, the second with a smaller input, plus the
argument checks. The library's built-in workspace is shared by every call on the GPU, so the calls here are made on one
stream, one after the other."""

import numpy as np
import pytest
import torch

from cute_kernels import _C

pytestmark = pytest.mark.gpu


def _both(lib, ids, bins, dev):
    """(counts, ends, starts) from the static entry point and from the workspace one, for ids already on the device."""
    i64 = 1 if ids.dtype == torch.int64 else 0
    stream = torch.cuda.current_stream().cuda_stream
    out = []
    for static in (True, False):
        counts, ends, starts = (torch.full((bins,), 0xDEADBEEF, dtype=torch.uint32, device=dev) for _ in range(3))
        if static:
            _C.check(lib.ck_count_offsets_static(ids.data_ptr(), i64, ids.numel(), bins, counts.data_ptr(), ends.data_ptr(),
                                                 starts.data_ptr(), stream))
        else:
            ws = torch.zeros(lib.ck_count_workspace_words(bins), dtype=torch.int32, device=dev)
            _C.check(lib.ck_count_offsets(ids.data_ptr(), i64, ids.numel(), bins, counts.data_ptr(), ends.data_ptr(),
                                          starts.data_ptr(), ws.data_ptr(), stream))
        torch.cuda.synchronize()
        out.append(tuple(t.cpu().numpy().copy() for t in (counts, ends, starts)))
    return out


# two calls in a row per case, the second with a smaller input (fewer ids, and in two cases fewer bins)
@pytest.mark.parametrize(
    "first,second",
    [
        ((1 << 22, 64, torch.int32), (65536, 64, torch.int32)),       # many blocks, then the one-block baseline case
        ((3_000_001, 16384, torch.int64), (4099, 1000, torch.int64)),  # the largest bin count, then fewer bins
        ((1 << 20, 8, torch.int32), (777, 3, torch.int32)),            # register-counter path
        ((100_000, 1024, torch.int32), (0, 72, torch.int32)),          # then an empty input
    ],
)
def test_static_entry_point_matches_workspace_entry_point(device, first, second):
    lib = _C.lib()
    for n, bins, dtype in (first, second):
        g = torch.Generator().manual_seed(n + bins)
        ids = torch.randint(0, bins, (n,), generator=g, dtype=dtype)
        if n > 10:
            ids[::7] = bins + 5  # out-of-range ids are not counted by either entry point
        got, want = _both(lib, ids.to(device), bins, device)
        for a, b in zip(got, want):
            np.testing.assert_array_equal(a, b)
        # and against numpy, so that a mistake shared by the two entry points would show too
        valid = ids[(ids >= 0) & (ids < bins)].numpy()
        np.testing.assert_array_equal(got[0], np.bincount(valid, minlength=bins).astype(np.uint32))
        np.testing.assert_array_equal(got[1], np.cumsum(got[0], dtype=np.uint64).astype(np.uint32))


def test_static_entry_point_rejects_sizes_beyond_its_workspace(device):
    lib = _C.lib()
    t = torch.zeros(4, dtype=torch.int32, device=device)
    assert lib.ck_count_offsets_static(t.data_ptr(), 0, 4, 16385, t.data_ptr(), None, None, None) != 0
    assert b"16384" in lib.ck_last_error_string()
    assert lib.ck_count_offsets_static(t.data_ptr(), 0, 4, 0, t.data_ptr(), None, None, None) != 0
    assert lib.ck_count_offsets_static(t.data_ptr(), 0, -1, 4, t.data_ptr(), None, None, None) != 0
