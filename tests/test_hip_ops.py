"""GPU parity of the device ops, called through the C-ABI (ctypes) with torch
tensors as device memory, against the CPU oracle and the reference's inline
known-answer vectors."""

import ctypes as C

import numpy as np
import pytest
import torch

import hip_harness as H
import kge_cases as K

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _distance(fn, a, b):
    ta, tb = dev(a.astype(np.float32)), dev(b.astype(np.float32))
    out = torch.empty(a.shape[0], b.shape[0], dtype=torch.float32, device="cuda")
    rc = getattr(H.lib(), fn)(H.dptr(ta), H.dptr(tb), H.dptr(out), a.shape[0], b.shape[0],
                              a.shape[1], None)
    assert rc == 0
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _distance_grad(kind, a, b, g, dist=None):
    ta, tb, tg = dev(a.astype(np.float32)), dev(b.astype(np.float32)), dev(g.astype(np.float32))
    out = torch.empty_like(ta)
    if kind == "l1":
        rc = H.lib().kge_l1_distance_grad(H.dptr(ta), H.dptr(tb), H.dptr(tg), H.dptr(out),
                                          a.shape[0], b.shape[0], a.shape[1], None)
    else:
        td = dev(dist.astype(np.float32))
        rc = H.lib().kge_l2_distance_grad(H.dptr(ta), H.dptr(tb), H.dptr(td), H.dptr(tg),
                                          H.dptr(out), a.shape[0], b.shape[0], a.shape[1], None)
    assert rc == 0
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _iota():
    return (np.arange(10, dtype=np.float32).reshape(2, 5),
            np.arange(20, dtype=np.float32).reshape(4, 5))


def test_l1dist_kat():
    # tests/pag/testPag.cpp:290-319
    a, b = _iota()
    np.testing.assert_array_equal(_distance("kge_l1_distance", a, b).ravel(),
                                  [0, 25, 50, 75, 25, 0, 25, 50])
    g = np.ones((2, 4), np.float32)
    np.testing.assert_array_equal(_distance_grad("l1", a, b, g), np.repeat([[-3.0], [-1.0]], 5, 1))
    np.testing.assert_array_equal(_distance_grad("l1", b, a, g.T.copy()),
                                  np.repeat([[-1.0], [1.0], [2.0], [2.0]], 5, 1))


def test_l2dist_kat():
    # tests/pag/testPag.cpp:334-369
    a, b = _iota()
    d = _distance("kge_l2_distance", a, b)
    np.testing.assert_allclose(d.ravel(), [0, 11.1803, 22.3607, 33.5410, 11.1803, 0, 11.1803,
                                           22.3607], atol=1e-4)
    g = np.ones((2, 4), np.float32)
    np.testing.assert_allclose(_distance_grad("l2", a, b, g, d),
                               np.repeat([[-1.3416], [-0.4472]], 5, 1), atol=1e-4)
    np.testing.assert_allclose(_distance_grad("l2", b, a, g.T.copy(), d.T.copy()),
                               np.repeat([[-0.4472], [0.4472], [0.8944], [0.8944]], 5, 1),
                               atol=1e-4)


def test_l2dist_large_kat():
    # tests/pag/testPag.cpp:371-392
    a = np.array([[100, 200, 300, 400, 500]], np.float32)
    b = np.full((1, 5), 600, np.float32)
    d = _distance("kge_l2_distance", a, b)
    np.testing.assert_allclose(d, [[741.62]], atol=0.5)
    np.testing.assert_allclose(_distance_grad("l2", a, b, np.ones((1, 1), np.float32), d).ravel(),
                               [-0.6742, -0.5394, -0.4045, -0.2697, -0.1348], atol=1e-3)


def test_matmul_kat():
    # tests/pag/testPag.cpp:582-600
    np.testing.assert_array_equal(_distance("kge_dot_score", np.ones((2, 3)), np.ones((5, 3))),
                                  np.full((2, 5), 3.0))


@pytest.mark.parametrize("shape", [(7, 11, 33), (64, 64, 64), (130, 70, 256), (256, 512, 256),
                                   (1, 1, 4), (65, 129, 12)])
@pytest.mark.parametrize("kind", ["l1", "l2", "dot"])
def test_distance_vs_oracle(oracle64, kind, shape):
    M, N, D = shape
    rng = np.random.default_rng(M * 1000 + N)
    a = rng.normal(size=(M, D)).astype(np.float32)
    b = rng.normal(size=(N, D)).astype(np.float32)
    if kind != "dot" and M > 2 and N > 2:
        b[1] = a[2]  # an exact zero distance
    g = rng.normal(size=(M, N)).astype(np.float32)
    fn = {"l1": "kge_l1_distance", "l2": "kge_l2_distance", "dot": "kge_dot_score"}[kind]
    ref = getattr(oracle64, {"l1": "l1_distance", "l2": "l2_distance", "dot": "dot_score"}[kind])(a, b)
    out = _distance(fn, a, b)
    assert K.rel_l2(out, ref) < 1e-6
    # scores: 1e-5 relative; entries that cancel to near zero are held to the
    # same absolute size as a typical entry (~sqrt(D))
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-5 * np.sqrt(D))
    if kind == "l1":
        ga, ga_ref = _distance_grad("l1", a, b, g), oracle64.l1_distance_grad(a, b, g)
        gb = _distance_grad("l1", b, a, g.T.copy())
        gb_ref = oracle64.l1_distance_grad(b, a, g.T)
    elif kind == "l2":
        # the saved forward distance is the device's own, as in the reference
        ga, ga_ref = _distance_grad("l2", a, b, g, out), oracle64.l2_distance_grad(a, b, out, g)
        gb = _distance_grad("l2", b, a, g.T.copy(), out.T.copy())
        gb_ref = oracle64.l2_distance_grad(b, a, out.T, g.T)
    else:
        return
    assert K.rel_l2(ga, ga_ref) < 1e-5
    assert K.rel_l2(gb, gb_ref) < 1e-5


def test_l2_distance_near_duplicates(oracle64):
    """Rows that nearly coincide: |a|^2 + |b|^2 - 2ab would lose every digit;
    the result must still be within 1e-5 relative, and exactly 0 for equal rows."""
    rng = np.random.default_rng(9)
    M, N, D = 200, 150, 256
    a = rng.normal(size=(M, D)).astype(np.float32)
    b = rng.normal(size=(N, D)).astype(np.float32)
    for j, scale in enumerate([0.0, 1e-6, 1e-4, 1e-3, 1e-2, 0.1, 0.3, 0.5]):
        b[j::8][:M // 8 + 1] = (a[j::8][:N // 8 + 1][:len(b[j::8])] *
                                (1 + scale * rng.normal(size=(len(b[j::8]), D)))).astype(np.float32)[:len(b[j::8])]
    out = _distance("kge_l2_distance", a, b)
    ref = oracle64.l2_distance(a, b)
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=0)
    assert np.all(out[ref == 0] == 0) and np.any(ref == 0)
    g = rng.normal(size=(M, N)).astype(np.float32)
    ga, ga_ref = _distance_grad("l2", a, b, g, out), oracle64.l2_distance_grad(a, b, out, g)
    assert K.rel_l2(ga, ga_ref) < 1e-5


def test_buffer_kat():
    # tests/fructose/testFructose.cpp:121-139
    buf = torch.zeros(3, 4, device="cuda")
    data = dev(np.array([[100, 101, 102, 103], [200, 201, 202, 203], [300, 301, 302, 303]],
                        np.float32))
    widx, ridx = dev(np.array([2, 0, 1], np.uint32).view(np.int32)), dev(np.array([0, 2], np.int32))
    out = torch.zeros(2, 4, device="cuda")
    assert H.lib().kge_buffer_write(H.dptr(buf), H.dptr(widx), H.dptr(data), C.c_int64(3),
                                    C.c_int64(16), None) == 0
    assert H.lib().kge_buffer_read(H.dptr(buf), H.dptr(ridx), H.dptr(out), C.c_int64(2),
                                   C.c_int64(16), None) == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), [[200, 201, 202, 203], [100, 101, 102, 103]])


@pytest.mark.parametrize("rows,row_floats,n", [(1000, 768, 4096), (50, 30, 77), (10, 1, 5), (7, 4, 0)])
def test_buffer_read_write_bit_exact(oracle64, rows, row_floats, n):
    rng = np.random.default_rng(rows)
    table = rng.normal(size=(rows, row_floats)).astype(np.float32)
    idx = rng.integers(0, rows, n).astype(np.uint32)
    tt, ti = dev(table), dev(idx.view(np.int32))
    out = torch.zeros(max(n, 1), row_floats, device="cuda")
    assert H.lib().kge_buffer_read(H.dptr(tt), H.dptr(ti), H.dptr(out), C.c_int64(n),
                                   C.c_int64(row_floats * 4), None) == 0
    torch.cuda.synchronize()
    if n:
        np.testing.assert_array_equal(out.cpu().numpy()[:n], oracle64.buffer_read(table, idx))
    # write-back of distinct rows
    uniq = np.unique(idx)
    data = rng.normal(size=(uniq.size, row_floats)).astype(np.float32)
    ref = table.copy()
    oracle64.buffer_write(ref, uniq, data)
    if uniq.size:
        assert H.lib().kge_buffer_write(H.dptr(tt), H.dptr(dev(uniq.view(np.int32))),
                                        H.dptr(dev(data)), C.c_int64(uniq.size),
                                        C.c_int64(row_floats * 4), None) == 0
        torch.cuda.synchronize()
    np.testing.assert_array_equal(tt.cpu().numpy(), ref)


def _scatter_add(rows, cols, idx, g):
    n = len(idx)
    ws_bytes = H.lib().kge_scatter_add_workspace_bytes(n, rows, cols)
    ws = torch.empty(ws_bytes + 16, dtype=torch.uint8, device="cuda")
    out = torch.full((rows, cols), float("nan"), device="cuda")
    ti = dev(np.asarray(idx, np.uint32).view(np.int32)) if n else torch.zeros(1, dtype=torch.int32, device="cuda")
    tg = dev(np.asarray(g, np.float32)) if n else torch.zeros(1, device="cuda")
    rc = H.lib().kge_scatter_add(H.dptr(out), C.c_int64(rows), C.c_int64(cols), H.dptr(ti),
                                 C.c_int64(n), H.dptr(tg), H.dptr(ws), None)
    assert rc == 0
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_multislice_kat():
    # tests/pag/testPag.cpp:602-628 (backward = scatter-add with duplicate indices)
    g = np.array([[.1, 1], [.2, 2], [.3, 3], [.4, 4]], np.float32)
    np.testing.assert_allclose(_scatter_add(3, 2, [1, 1, 0, 1], g).ravel(), [.3, 3, .7, 7, 0, 0],
                               rtol=1e-6)


@pytest.mark.parametrize("rows,cols,n,zipf", [(100, 8, 1000, True), (5000, 256, 20000, True),
                                              (300, 64, 300, False), (17, 3, 0, False),
                                              (70000, 4, 5000, False)])
def test_scatter_add_vs_oracle_and_deterministic(oracle64, rows, cols, n, zipf):
    rng = np.random.default_rng(n + rows)
    idx = (K.zipf_ids(rng, rows, n) if zipf else rng.integers(0, rows, n)).astype(np.uint32)
    g = rng.normal(size=(n, cols)).astype(np.float32)
    out = _scatter_add(rows, cols, idx, g)
    ref = oracle64.multi_update_add(rows, idx, g)
    assert K.rel_l2(out, ref) < 1e-6
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-5)
    # untouched rows are exactly zero
    touched = np.zeros(rows, bool)
    touched[idx] = True
    assert np.all(out[~touched] == 0)
    # deterministic: bitwise equal when repeated
    np.testing.assert_array_equal(out, _scatter_add(rows, cols, idx, g))


@pytest.mark.parametrize("v_is_sqrt", [0, 1])
def test_adam_vs_oracle(oracle64, v_is_sqrt):
    rng = np.random.default_rng(3)
    n = 10007
    p0 = rng.normal(size=n).astype(np.float32)
    m0 = rng.normal(0, 0.1, n).astype(np.float32)
    v0 = np.abs(rng.normal(0, 0.3, n)).astype(np.float32)
    g = (rng.normal(size=n) * 50).astype(np.float32)
    g[::7] = 0
    p, m, v = p0.copy(), m0.copy(), v0.copy()
    oracle64.adam(p, m, v, g, 0.0123, 0.9, 0.999, 1e-8, 0.01, v_is_sqrt=bool(v_is_sqrt))
    tp, tm, tv, tg = dev(p0), dev(m0), dev(v0), dev(g)
    rc = H.lib().kge_adam(H.dptr(tp), H.dptr(tm), H.dptr(tv), H.dptr(tg), C.c_int64(n),
                          C.c_float(0.0123), C.c_float(0.9), C.c_float(0.999), C.c_float(1e-8),
                          C.c_float(0.01), v_is_sqrt, None)
    assert rc == 0
    torch.cuda.synchronize()
    np.testing.assert_allclose(tp.cpu().numpy(), p, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(tm.cpu().numpy(), m, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(tv.cpu().numpy(), v, rtol=1e-5, atol=1e-7)
    assert K.rel_l2(tp.cpu().numpy() - p0, p - p0) < 1e-5
