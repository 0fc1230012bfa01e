"""The scatter-add entry point that allocates nothing (kge_scatter_add_static: its workspace is a
fixed array in device memory) against kge_scatter_add with a caller-supplied workspace: the same
kernels in the same order, so the results must be bit-identical.  Two calls in a row, the second
with a smaller input (the array still holds the first call's contents), then the size limit."""

import ctypes as C

import numpy as np
import pytest
import torch

import hip_harness as H
import kge_cases as K

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _operands(idx, g, cols):
    if len(idx) == 0:   # an empty input still needs valid pointers
        return torch.zeros(1, dtype=torch.int32, device="cuda"), torch.zeros(1, cols, device="cuda")
    return dev(idx.view(np.int32)), dev(g)


def _with_workspace(rows, cols, idx, g):
    n = len(idx)
    lib = H.lib()
    ws = torch.empty(lib.kge_scatter_add_workspace_bytes(n, rows, cols) + 16, dtype=torch.uint8, device="cuda")
    out = torch.full((rows, cols), float("nan"), device="cuda")
    ti, tg = _operands(idx, g, cols)
    assert lib.kge_scatter_add(H.dptr(out), C.c_int64(rows), C.c_int64(cols), H.dptr(ti), C.c_int64(n),
                               H.dptr(tg), H.dptr(ws), None) == 0
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _static(rows, cols, idx, g, expect=0):
    n = len(idx)
    lib = H.lib()
    out = torch.full((rows, cols), float("nan"), device="cuda")
    ti, tg = _operands(idx, g, cols)
    err = C.create_string_buffer(512)
    rc = lib.kge_scatter_add_static(H.dptr(out), C.c_int64(rows), C.c_int64(cols), H.dptr(ti), C.c_int64(n),
                                    H.dptr(tg), None, err, C.c_size_t(512))
    assert rc == expect, err.value
    torch.cuda.synchronize()
    return out.cpu().numpy(), err.value.decode()


def test_static_scatter_add_matches_the_workspace_entry_point(oracle64):
    lib = H.lib()
    lib.kge_scatter_add_static_max_bytes.restype = C.c_size_t
    limit = lib.kge_scatter_add_static_max_bytes()
    assert limit == 16 << 20
    rng = np.random.default_rng(77)
    # the second call is smaller than the first: it runs over the first one's leftovers
    for rows, cols, n in [(5000, 256, 20000), (300, 64, 700), (5000, 256, 20000), (17, 3, 0)]:
        assert lib.kge_scatter_add_workspace_bytes(n, rows, cols) <= limit
        idx = K.zipf_ids(rng, rows, n).astype(np.uint32) if n else np.zeros(0, np.uint32)
        g = rng.normal(size=(n, cols)).astype(np.float32)
        got, _ = _static(rows, cols, idx, g)
        ref = _with_workspace(rows, cols, idx, g)
        np.testing.assert_array_equal(got, ref)                 # same kernels, same order: bit for bit
        assert K.rel_l2(got, oracle64.multi_update_add(rows, idx, g)) < 1e-6


def test_static_scatter_add_rejects_what_does_not_fit():
    lib = H.lib()
    lib.kge_scatter_add_static_max_bytes.restype = C.c_size_t
    rows, cols, n = 60000, 256, 1000          # 60000 x 256 partial rows alone exceed 16 MiB
    assert lib.kge_scatter_add_workspace_bytes(n, rows, cols) > lib.kge_scatter_add_static_max_bytes()
    idx, g = np.zeros(n, np.uint32), np.zeros((n, cols), np.float32)
    _, msg = _static(rows, cols, idx, g, expect=1)
    assert "more than the 16777216 bytes of the static scratch array" in msg
    _, msg = _static(0, 4, idx[:1], g[:1, :4], expect=1)
    assert "out of range" in msg


def test_static_scatter_add_allocates_nothing_and_takes_any_stream(oracle64):
    """The entry point's claim: no device memory is allocated or freed by a call.  After a
    warm-up call (the first call on a device looks the array's address up, the first on a stream
    lets the runtime set that stream's queue up) the device's free memory is the same before and
    after a series of calls whose operands were prepared beforehand, on the null stream and on a
    stream of the caller's, whose result is bit-identical to the null stream's."""
    lib = H.lib()
    rng = np.random.default_rng(5)
    rows, cols, n = 4000, 128, 30000
    idx = K.zipf_ids(rng, rows, n).astype(np.uint32)
    g = rng.normal(size=(n, cols)).astype(np.float32)
    ti, tg = _operands(idx, g, cols)
    out = torch.full((rows, cols), float("nan"), device="cuda")
    err = C.create_string_buffer(512)

    def call(stream):
        rc = lib.kge_scatter_add_static(H.dptr(out), C.c_int64(rows), C.c_int64(cols), H.dptr(ti), C.c_int64(n),
                                        H.dptr(tg), stream, err, C.c_size_t(512))
        assert rc == 0, err.value

    call(None)                                   # warm-up
    torch.cuda.synchronize()
    first = out.cpu().numpy()
    free_before, _ = torch.cuda.mem_get_info()   # (hipMemGetInfo)
    for _ in range(5):
        call(None)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before   # nothing allocated, nothing freed
    # a stream of the caller's (default priority).  Its first call is not measured: the runtime
    # sets a new stream's queue up when kernels first run on it (among other things the scratch
    # memory for their private segments), which takes device memory once per queue.
    side = torch.cuda.Stream()
    call(C.c_void_p(side.cuda_stream))
    side.synchronize()
    out.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    call(C.c_void_p(side.cuda_stream))
    side.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    np.testing.assert_array_equal(out.cpu().numpy(), first)
    assert K.rel_l2(first, oracle64.multi_update_add(rows, idx, g)) < 1e-6
