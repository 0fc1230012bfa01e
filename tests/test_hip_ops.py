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


# (the last case: 1.36M keys to sort = 332 sort tiles, where the histogram scan is a launch of its
# own instead of a part of the scatter)
@pytest.mark.parametrize("rows,cols,n,zipf", [(100, 8, 1000, True), (5000, 256, 20000, True),
                                              (300, 64, 300, False), (17, 3, 0, False),
                                              (70000, 4, 5000, False), (60000, 4, 1_300_000, False)])
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


# ---- loss functions as device ops ---------------------------------------------

def _log_sigmoid(x, dy=None, form=0):
    tx = dev(np.asarray(x, np.float32))
    ty, tdx = torch.empty_like(tx), torch.empty_like(tx)
    tdy = dev(np.asarray(dy, np.float32)) if dy is not None else None
    rc = H.lib().kge_log_sigmoid(H.dptr(tx), H.dptr(tdy) if tdy is not None else None, H.dptr(ty),
                                 H.dptr(tdx), C.c_int64(tx.numel()), form, None)
    assert rc == 0
    torch.cuda.synchronize()
    return ty.cpu().numpy(), tdx.cpu().numpy()


@pytest.mark.parametrize("form", [0, 1])
def test_logsigmoid_kat(form):
    # tests/pag/testPag.cpp:817-845 (margin 1e-2 as there, which tolerates the clamp)
    x = np.array([-100, -12, -1, 0, 1, 12, 100], np.float32)
    y, dx = _log_sigmoid(x, np.full(7, 10, np.float32), form)
    np.testing.assert_allclose(y, -np.log1p(np.exp(-x.astype(np.float64))), atol=1e-2)
    np.testing.assert_allclose(dx, 10.0 / (1 + np.exp(x.astype(np.float64))), atol=1e-2)


@pytest.mark.parametrize("form", [0, 1])
def test_logsigmoid_clamps_and_oracle(oracle64, form):
    """src/pag/pag.cpp:894-903: the value is x itself at x <= -11, the derivative stays at
    1 / (1 + e^11) from x = 11 on; everywhere the device agrees with the oracle to 1e-5
    relative (the bar on scores and gradients), both forms of the device function."""
    rng = np.random.default_rng(4)
    x = np.concatenate([np.array([-30, -11.5, -11, -10.9, -3, -0.0, 0.0, 0.5, 10.9, 11, 11.5, 30, 88, -88]),
                        rng.normal(0, 6, 5000), rng.uniform(-12, 12, 5000)]).astype(np.float32)
    y, dx = _log_sigmoid(x, None, form)
    np.testing.assert_array_equal(y[x <= -11], x[x <= -11])
    np.testing.assert_allclose(dx[x >= 11], 1 / (1 + np.exp(11.0)), rtol=2e-6)
    np.testing.assert_allclose(y, oracle64.log_sigmoid(x), rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(dx, oracle64.log_sigmoid_grad(x, np.ones_like(x)), rtol=1e-5)


def _log_softmax(x, dy=None):
    tx = dev(np.asarray(x, np.float32))
    rows, cols = tx.reshape(-1, tx.shape[-1]).shape
    ty = torch.empty_like(tx)
    assert H.lib().kge_log_softmax(H.dptr(tx), H.dptr(ty), C.c_int64(rows), C.c_int64(cols), None) == 0
    if dy is None:
        torch.cuda.synchronize()
        return ty.cpu().numpy()
    tdy, tdx = dev(np.asarray(dy, np.float32)), torch.empty_like(tx)
    assert H.lib().kge_log_softmax_grad(H.dptr(ty), H.dptr(tdy), H.dptr(tdx), C.c_int64(rows),
                                        C.c_int64(cols), None) == 0
    torch.cuda.synchronize()
    return ty.cpu().numpy(), tdx.cpu().numpy()


def test_logsoftmax_kat(oracle64):
    # tests/pag/testPag.cpp:775-794
    a = np.array([1, 1, 2], np.float32)
    norm = np.log(np.exp(1.0) + np.exp(1.0) + np.exp(2.0))
    y, dx = _log_softmax(a, np.array([10, 15, 5], np.float32))
    np.testing.assert_allclose(y, [1 - norm, 1 - norm, 2 - norm], rtol=1e-6)
    np.testing.assert_allclose(dx, [10 - 30 * np.exp(1 - norm), 15 - 30 * np.exp(1 - norm),
                                    5 - 30 * np.exp(2 - norm)], rtol=1e-5)
    rng = np.random.default_rng(5)
    x, dy = rng.normal(0, 4, (37, 300)).astype(np.float32), rng.normal(size=(37, 300)).astype(np.float32)
    y, dx = _log_softmax(x, dy)
    ref = oracle64.log_softmax(x)
    np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-6)
    assert K.rel_l2(dx, oracle64.log_softmax_grad(ref, dy)) < 1e-6


def _loss(loss_fn, score, label, correction=0.0, adversarial=0.0, loss_scale=1.0):
    S, B, T = score.shape
    ts, tl = dev(score.astype(np.float32)), dev(label.astype(np.uint32).view(np.int32))
    loss, rows = torch.empty(S, device="cuda"), torch.empty(S, B, device="cuda")
    ds = torch.empty_like(ts)
    rc = H.lib().kge_loss({"logsigmoid": 0, "softmax": 1}[loss_fn], H.dptr(ts), H.dptr(tl), S, B, T,
                          C.c_float(correction), C.c_float(adversarial), C.c_float(loss_scale),
                          H.dptr(loss), H.dptr(rows), H.dptr(ds), None)
    assert rc == 0
    torch.cuda.synchronize()
    return loss.cpu().numpy(), rows.cpu().numpy(), ds.cpu().numpy()


def test_softmax_xent_kat():
    # tests/fructose/testFructose.cpp:57-67: softmaxCrossEntropy([-100, 2, 2, 2, 2], 1) = log 4
    loss, rows, ds = _loss("softmax", np.array([[[-100, 2, 2, 2, 2]]], np.float32), np.array([[1]]))
    np.testing.assert_allclose(loss, [np.log(4)], rtol=1e-6)
    np.testing.assert_allclose(ds.ravel(), [0, 0.25 - 1, 0.25, 0.25, 0.25], atol=1e-7)
    # tests/pag/testPag.cpp:775-794 through the loss kernel: with label i the row's loss is
    # -logsoftmax(a)[i] and dscore = softmax(a) - onehot(i)
    a = np.broadcast_to(np.array([1, 1, 2], np.float32), (1, 3, 3)).copy()
    norm = np.log(np.exp(1.0) + np.exp(1.0) + np.exp(2.0))
    loss, rows, ds = _loss("softmax", a, np.array([[0, 1, 2]]))
    np.testing.assert_allclose(rows.ravel() * 3, [norm - 1, norm - 1, norm - 2], rtol=1e-6)
    soft = np.exp(np.array([1, 1, 2]) - norm)
    np.testing.assert_allclose(ds[0] * 3, soft[None, :] - np.eye(3), rtol=1e-5, atol=1e-7)
    grad_b = np.array([10, 15, 5])
    np.testing.assert_allclose(-(grad_b[:, None] * ds[0] * 3).sum(0), grad_b - 30 * soft, rtol=1e-5)


@pytest.mark.parametrize("variant", ["logsigmoid", "logsigmoid_saturated", "adversarial", "softmax",
                                     "softmax_corrected", "softmax_wide"])
def test_loss_vs_oracle(oracle64, variant):
    """Model::getLoss on the device (the kernel the step runs for the softmax and adversarial
    losses) against the oracle's shard_loss: per-shard loss 1e-5, d loss / d score 1e-5."""
    from oracle.kge_oracle import make_cfg

    rng = np.random.default_rng(len(variant))
    S, B, A = (2, 37, 50) if variant != "softmax_wide" else (2, 12, 1200)
    T = S * A
    loss_fn = "softmax" if variant.startswith("softmax") else "logsigmoid"
    cw = 1.0 if variant == "softmax_corrected" else 0.0
    adv = 1.5 if variant == "adversarial" else 0.0
    spread = 14.0 if variant == "logsigmoid_saturated" else 3.0   # |score| beyond the +-11 clamps
    score = rng.normal(0, spread, (S, B, T)).astype(np.float32)
    label = rng.integers(0, T, (S, B)).astype(np.uint32)
    n_entity = 5000
    cfg = make_cfg(n_shard=S, n_entity=n_entity, n_relation=4, dim=8, batch=B, a2a=A, loss_fn=loss_fn,
                   softmax_correction_weight=cw, negative_adversarial_scale=adv)
    corr = cw * float(np.float32(np.log(n_entity * S - 1) - np.log(T - 1)))
    loss_scale = 64.0
    loss, rows, ds = _loss(loss_fn, score, label, corr, adv, loss_scale)
    for s in range(S):
        ref_loss, ref_ds = oracle64.loss(cfg, score[s], label[s])
        np.testing.assert_allclose(loss[s], ref_loss, rtol=1e-5)
        np.testing.assert_allclose(rows[s].sum(dtype=np.float64), ref_loss, rtol=1e-5)
        assert K.rel_l2(ds[s], loss_scale * ref_ds) < 1e-5
        np.testing.assert_allclose(ds[s], loss_scale * ref_ds, rtol=2e-5, atol=1e-9 * loss_scale)
