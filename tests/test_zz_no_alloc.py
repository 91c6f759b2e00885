"""wq_delta_xor_noalloc - the entry point for callers that cannot allocate - against wq_delta_xor (the entry point
it is a variant of) and the numpy restatement of the reference, through the C ABI: two calls in a row, the second
on a smaller input, so that rows the first call left in the library's device array must not leak into the second."""

import numpy as np
import pytest
import torch

from oracle import delta_ref as D
from slime_amd import _lib

pytestmark = pytest.mark.gpu


def _pair(n, density, seed):
    rng = np.random.default_rng(seed)
    old = rng.integers(0, 256, n, dtype=np.uint8)
    new = old.copy()
    idx = rng.random(n) < density
    new[idx] = rng.integers(0, 256, int(idx.sum()), dtype=np.uint8)
    return new, old


def _run(entry, new, old, cuda, update):
    """-> (diff bytes, [changed, adler32], snapshot bytes after the call) of one call through the C ABI."""
    lib = _lib.load()
    n = new.size
    ng, og = torch.from_numpy(new).to(cuda), torch.from_numpy(old).to(cuda)
    diff = torch.empty(max(n, 1), dtype=torch.uint8, device=cuda)
    result = torch.full((2,), -1, dtype=torch.int64, device=cuda)
    st = _lib.stream_ptr(cuda)
    if entry == "noalloc":
        rc = lib.wq_delta_xor_noalloc(ng.data_ptr(), og.data_ptr(), diff.data_ptr(), n, int(update), result.data_ptr(), st)
    else:
        ws = torch.empty(lib.wq_delta_workspace_bytes(n) // 8, dtype=torch.int64, device=cuda)
        rc = lib.wq_delta_xor(ng.data_ptr(), og.data_ptr(), diff.data_ptr(), n, int(update), ws.data_ptr(),
                              result.data_ptr(), st)
    assert rc == 0, lib.wq_error_string(rc)
    torch.cuda.synchronize()
    return diff[:n].cpu().numpy(), result.tolist(), og.cpu().numpy()


def test_noalloc_equals_workspace_form_twice_second_smaller(cuda):
    # 37 chunks + a ragged tail, then 2 chunks + a tail: the second call reads only its own rows
    for call, (n, density) in enumerate([(16384 * 37 + 11, 0.05), (16384 * 2 + 5, 1.0)]):
        new, old = _pair(n, density, 100 + call)
        want_diff, want_changed = D.xor_delta_ref(new, old)
        want = [want_changed, int(D.adler32_ref(new), 16)]
        for update in (False, True):
            d0, r0, o0 = _run("workspace", new, old, cuda, update)
            d1, r1, o1 = _run("noalloc", new, old, cuda, update)
            assert r1 == r0 == want, (call, update, r1, r0, want)
            assert np.array_equal(d1, d0) and np.array_equal(d1, want_diff)
            assert np.array_equal(o1, o0) and np.array_equal(o1, new if update else old)


def test_noalloc_allocates_nothing_and_rejects_oversize(cuda):
    lib = _lib.load()
    new, old = _pair(16384 * 5, 0.5, 3)
    ng, og = torch.from_numpy(new).to(cuda), torch.from_numpy(old).to(cuda)
    diff = torch.empty_like(ng)
    result = torch.empty(2, dtype=torch.int64, device=cuda)
    st = _lib.stream_ptr(cuda)
    assert lib.wq_delta_xor_noalloc(ng.data_ptr(), og.data_ptr(), diff.data_ptr(), new.size, 0, result.data_ptr(), st) == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert lib.wq_delta_xor_noalloc(ng.data_ptr(), og.data_ptr(), diff.data_ptr(), new.size, 0, result.data_ptr(), st) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0                                   # driver-level free memory unchanged: no hipMalloc / hipFree
    assert result.tolist() == [D.xor_delta_ref(new, old)[1], int(D.adler32_ref(new), 16)]
    too_big = (4 << 30) + 1                                 # WQ_DELTA_NOALLOC_MAX_BYTES + 1; rejected before any launch
    rc = lib.wq_delta_xor_noalloc(ng.data_ptr(), og.data_ptr(), diff.data_ptr(), too_big, 0, result.data_ptr(), st)
    assert rc == -6 and b"exceeds" in lib.wq_error_string(rc)
    assert lib.wq_delta_xor_noalloc(ng.data_ptr(), og.data_ptr(), diff.data_ptr(), 0, 0, result.data_ptr(), st) == 0
    torch.cuda.synchronize()
    assert result.tolist() == [0, 1]                        # empty input: adler32 = 1
