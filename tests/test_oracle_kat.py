"""Pins the CPU oracle: the reference's own inline known-answer vectors, torch
cross-checks, closed forms, and an independent autograd restatement of the
whole step.  Runs on the CPU (no ``gpu`` marker)."""

import numpy as np
import pytest
import torch as T

import kge_cases as K
import torch_restatement
from oracle.kge_oracle import Oracle, make_cfg


@pytest.fixture(params=["f64", "f32"], scope="module")
def orc(request):
    return Oracle(request.param)


# ---- reference known-answer vectors --------------------------------------

def test_buffer_kat(orc):
    # tests/fructose/testFructose.cpp:121-139
    buf = np.zeros((3, 4), np.float32)
    data = np.array([[100, 101, 102, 103], [200, 201, 202, 203], [300, 301, 302, 303]], np.float32)
    orc.buffer_write(buf, [2, 0, 1], data)
    np.testing.assert_array_equal(orc.buffer_read(buf, [0, 2]),
                                  [[200, 201, 202, 203], [100, 101, 102, 103]])


def test_multislice_kat(orc):
    # tests/pag/testPag.cpp:602-628
    table = np.array([[10, 11], [20, 21], [30, 31]], np.float32)
    idx = [1, 1, 0, 1]
    np.testing.assert_array_equal(orc.multi_slice(table, idx).ravel(),
                                  [20, 21, 20, 21, 10, 11, 20, 21])
    g = np.array([[.1, 1], [.2, 2], [.3, 3], [.4, 4]], np.float32)
    np.testing.assert_allclose(orc.multi_update_add(3, idx, g).ravel(), [.3, 3, .7, 7, 0, 0],
                               rtol=1e-6)


def _iota():
    return (np.arange(10, dtype=np.float32).reshape(2, 5),
            np.arange(20, dtype=np.float32).reshape(4, 5))


def test_l1dist_kat(orc):
    # tests/pag/testPag.cpp:290-319 (zero distances included; signum(0) = 0)
    a, b = _iota()
    np.testing.assert_array_equal(orc.l1_distance(a, b).ravel(), [0, 25, 50, 75, 25, 0, 25, 50])
    g = np.ones((2, 4), np.float32)
    np.testing.assert_array_equal(orc.l1_distance_grad(a, b, g),
                                  np.repeat([[-3.0], [-1.0]], 5, 1))
    np.testing.assert_array_equal(orc.l1_distance_grad(b, a, g.T),
                                  np.repeat([[-1.0], [1.0], [2.0], [2.0]], 5, 1))


def test_l2dist_kat(orc):
    # tests/pag/testPag.cpp:334-369
    a, b = _iota()
    d = orc.l2_distance(a, b)
    np.testing.assert_allclose(d.ravel(), [0, 11.1803, 22.3607, 33.5410, 11.1803, 0, 11.1803,
                                           22.3607], atol=1e-4)
    g = np.ones((2, 4), np.float32)
    np.testing.assert_allclose(orc.l2_distance_grad(a, b, d, g),
                               np.repeat([[-1.3416], [-0.4472]], 5, 1), atol=1e-4)
    np.testing.assert_allclose(orc.l2_distance_grad(b, a, d.T, g.T),
                               np.repeat([[-0.4472], [0.4472], [0.8944], [0.8944]], 5, 1),
                               atol=1e-4)


def test_l2dist_large_kat(orc):
    # tests/pag/testPag.cpp:371-392
    a = np.array([[100, 200, 300, 400, 500]], np.float32)
    b = np.full((1, 5), 600, np.float32)
    d = orc.l2_distance(a, b)
    np.testing.assert_allclose(d, [[741.62]], atol=0.5)
    np.testing.assert_allclose(orc.l2_distance_grad(a, b, d, np.ones((1, 1), np.float32)).ravel(),
                               [-0.6742, -0.5394, -0.4045, -0.2697, -0.1348], atol=1e-3)


def test_matmul_kat(orc):
    # tests/pag/testPag.cpp:582-600: ones[2,3] x ones[3,5] = 3
    np.testing.assert_array_equal(orc.dot_score(np.ones((2, 3)), np.ones((5, 3))),
                                  np.full((2, 5), 3.0))


def test_logsoftmax_kat(orc):
    # tests/pag/testPag.cpp:775-794
    a = np.array([1, 1, 2], np.float32)
    norm = np.log(np.exp(1.0) + np.exp(1.0) + np.exp(2.0))
    y = orc.log_softmax(a)
    np.testing.assert_allclose(y, [1 - norm, 1 - norm, 2 - norm], rtol=1e-6)
    dx = orc.log_softmax_grad(y, np.array([10, 15, 5], np.float32))
    np.testing.assert_allclose(dx, [10 - 30 * np.exp(1 - norm), 15 - 30 * np.exp(1 - norm),
                                    5 - 30 * np.exp(2 - norm)], rtol=1e-5)


def test_logsigmoid_kat(orc):
    # tests/pag/testPag.cpp:817-845 (margin 1e-2 as there, which tolerates the clamp)
    x = np.array([-100, -12, -1, 0, 1, 12, 100], np.float32)
    np.testing.assert_allclose(orc.log_sigmoid(x), -np.log1p(np.exp(-x.astype(np.float64))),
                               atol=1e-2)
    np.testing.assert_allclose(orc.log_sigmoid_grad(x, np.full(7, 10, np.float32)),
                               10.0 / (1 + np.exp(x.astype(np.float64))), atol=1e-2)


def test_logsigmoid_exact_expression(orc):
    # src/pag/pag.cpp:894-903: inside (-11, 11) it is the exact logsigmoid; the
    # gradient saturates at 1/(1+e^11) above 11 and the value is x below -11.
    x = np.array([-30, -11.5, -10.9, -3, 0.5, 10.9, 11.5, 30], np.float32)
    y, dx = orc.log_sigmoid(x), orc.log_sigmoid_grad(x, np.ones_like(x))
    inside = np.abs(x) < 11
    ref = T.nn.functional.logsigmoid(T.tensor(x, dtype=T.float64)).numpy()
    np.testing.assert_allclose(y[inside], ref[inside], rtol=2e-6)
    np.testing.assert_array_equal(y[x <= -11], x[x <= -11])
    np.testing.assert_allclose(y[x >= 11], ref[x >= 11], atol=2e-5)
    np.testing.assert_allclose(dx[x >= 11], 1 / (1 + np.exp(11.0)), rtol=1e-6)
    np.testing.assert_allclose(dx[inside], 1 / (1 + np.exp(x[inside].astype(np.float64))),
                               rtol=2e-6)


def test_softmax_xent_kat(orc):
    # tests/fructose/testFructose.cpp:57-67
    np.testing.assert_allclose(orc.softmax_cross_entropy([[-100, 2, 2, 2, 2]], [1]), [np.log(4)],
                               rtol=1e-6)


def test_detached_softmax_kat(orc):
    # tests/testPoplarKge.cpp:56-72
    x = np.array([[1, 1, 2], [2, 4, 6]], np.float32)
    e = np.exp(x.astype(np.float64))
    np.testing.assert_allclose(orc.softmax(x), e / e.sum(1, keepdims=True), rtol=1e-6)


# ---- torch / closed-form cross-checks ---------------------------------------

@pytest.mark.parametrize("p", [1, 2])
def test_distance_vs_torch_cdist(orc, p):
    rng = np.random.default_rng(5)
    a = rng.normal(size=(7, 33)).astype(np.float32)
    b = rng.normal(size=(11, 33)).astype(np.float32)
    g = rng.normal(size=(7, 11)).astype(np.float32)
    ta = T.tensor(a, dtype=T.float64, requires_grad=True)
    tb = T.tensor(b, dtype=T.float64, requires_grad=True)
    d = T.cdist(ta, tb, p=p)
    d.backward(T.tensor(g, dtype=T.float64))
    tol = 1e-12 if orc.precision == "f64" else 2e-6
    if p == 1:
        mine, ga = orc.l1_distance(a, b), orc.l1_distance_grad(a, b, g)
        gb = orc.l1_distance_grad(b, a, g.T)
    else:
        mine = orc.l2_distance(a, b)
        ga = orc.l2_distance_grad(a, b, mine, g)
        gb = orc.l2_distance_grad(b, a, mine.T, g.T)
    assert K.rel_l2(mine, d.detach().numpy()) < max(tol, 1e-7)
    assert K.rel_l2(ga, ta.grad.numpy()) < max(tol, 2e-7)
    assert K.rel_l2(gb, tb.grad.numpy()) < max(tol, 2e-7)


def test_l2_grad_zero_distance_is_zero(orc):
    a = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    d = orc.l2_distance(a, a)
    ga = orc.l2_distance_grad(a, a, d, np.ones((2, 2), np.float32))
    # only the off-diagonal pair contributes: (a0-a1)/|a0-a1| and its negative
    u = (a[0] - a[1]) / np.linalg.norm(a[0] - a[1])
    np.testing.assert_allclose(ga, [u, -u], rtol=1e-6)


def test_adam_step_size_closed_form(orc):
    step, alpha = orc.adam_step_size(0, 0.1)
    assert step == 1
    # the betas are float32 constants in the reference (frnn.cpp:52-54)
    f = lambda x: float(np.float32(x))
    np.testing.assert_allclose(alpha, 0.1 * np.sqrt(1 - f(0.999)) / (1 - f(0.9)), rtol=1e-6)
    step, alpha = orc.adam_step_size(999, 1e-3, 0.8, 0.99)
    assert step == 1000
    np.testing.assert_allclose(alpha, 1e-3 * np.sqrt(1 - f(0.99)**1000) / (1 - f(0.8)**1000),
                               rtol=1e-6)


def test_adam_invariants(orc):
    rng = np.random.default_rng(1)
    p0 = rng.normal(size=64).astype(np.float32)
    # zero gradient and zero moments leave the row untouched
    p, m, v = p0.copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    orc.adam(p, m, v, np.zeros(64), alpha=0.3)
    np.testing.assert_array_equal(p, p0)
    np.testing.assert_array_equal(m, 0)
    # first step from zero state: dp = -alpha * 0.1 g / (sqrt(0.001) |g| + eps)
    g = rng.normal(size=64).astype(np.float32) * 100
    p, m, v = p0.copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    orc.adam(p, m, v, g, alpha=0.01, eps=1e-8)
    g64 = g.astype(np.float64)
    # (1 - beta) is formed in float32 from float32 betas (frnn.cpp:74-80)
    cm, cv = 1 - float(np.float32(0.9)), 1 - float(np.float32(0.999))
    np.testing.assert_allclose(p - p0, -0.01 * cm * g64 / (np.sqrt(cv) * np.abs(g64) + 1e-8),
                               rtol=2e-4, atol=1e-9)
    np.testing.assert_allclose(m, cm * g64, rtol=1e-6)
    np.testing.assert_allclose(v, cv * g64 * g64, rtol=1e-6)
    # sqrt-v storage (entity rows): same update, s = sqrt(v)
    p2, m2, s2 = p0.copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    orc.adam(p2, m2, s2, g, alpha=0.01, v_is_sqrt=True)
    np.testing.assert_allclose(p2, p, rtol=1e-6)
    np.testing.assert_allclose(s2, np.sqrt(v), rtol=1e-6)
    # weight decay term: p -= alpha * wd * p on top
    p3, m3, v3 = p0.copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    orc.adam(p3, m3, v3, g, alpha=0.01, wd=0.5)
    np.testing.assert_allclose(p3, p - 0.01 * 0.5 * p0, rtol=1e-5, atol=1e-7)


def test_adam_vs_torch_optim(orc):
    # The reference's own check is at 1e-4 (tests/python/test_poplar_kge.py:222-259):
    # torch adds eps after the bias correction, the reference before.
    rng = np.random.default_rng(2)
    p0 = rng.normal(size=(5, 16)).astype(np.float32)
    tp = T.nn.Parameter(T.tensor(p0.astype(np.float64)))
    opt = T.optim.Adam([tp], lr=0.05, betas=(0.9, 0.999), eps=1e-8)
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    step = 0
    for _ in range(6):
        g = (rng.normal(size=p0.shape) * 30).astype(np.float32)
        tp.grad = T.tensor(g.astype(np.float64))
        opt.step()
        step, alpha = orc.adam_step_size(step, 0.05)
        orc.adam(p, m, v, g, alpha)
    assert K.rel_l2(p - p0, tp.detach().numpy() - p0) < 1e-4


def test_loss_vs_reference_model_form(orc):
    # tests/python/reference_model.py:140-152: -mean(weight * logsigmoid(sign * score))
    # over [S, B, T] equals the sum over shards of the C++ per-shard loss.
    rng = np.random.default_rng(3)
    S, B, A = 3, 4, 5
    Tn = S * A
    cfg = make_cfg(n_shard=S, n_entity=50, n_relation=3, dim=4, batch=B, a2a=A)
    score = rng.normal(0, 3, (S, B, Tn)).astype(np.float32)
    label = rng.integers(0, Tn, (S, B))
    total = sum(orc.loss(cfg, score[s], label[s])[0] for s in range(S))
    ts = T.tensor(score, dtype=T.float64)
    oh = T.nn.functional.one_hot(T.tensor(label), Tn)
    w = oh * (0.5 * Tn - 0.5 * Tn / (Tn - 1)) + 0.5 * Tn / (Tn - 1)
    ref = -T.mean(w * T.nn.functional.logsigmoid((2 * oh - 1) * ts))
    np.testing.assert_allclose(total, float(ref), rtol=2e-6)


@pytest.mark.parametrize("loss_fn,extra", [
    ("logsigmoid", {}),
    ("logsigmoid", {"negative_adversarial_scale": 0.7}),
    ("softmax", {"softmax_correction_weight": 1.0}),
    ("softmax", {}),
])
def test_loss_grad_vs_autograd(orc, loss_fn, extra):
    rng = np.random.default_rng(4)
    S, B, A, NE = 2, 5, 4, 77
    Tn = S * A
    cfg = make_cfg(n_shard=S, n_entity=NE, n_relation=3, dim=4, batch=B, a2a=A, loss_fn=loss_fn,
                   **extra)
    score = rng.normal(0, 5, (B, Tn)).astype(np.float32)
    score[0, 0], score[1, 2] = 14.0, -13.0  # outside the +-11 clamp
    label = rng.integers(0, Tn, B)
    loss, ds = orc.loss(cfg, score, label)
    ts = T.tensor(score, dtype=T.float64, requires_grad=True)
    oh = T.nn.functional.one_hot(T.tensor(label), Tn).to(T.float64)
    if loss_fn == "logsigmoid":
        w = oh * (0.5 * Tn - 0.5 * Tn / (Tn - 1)) + 0.5 * Tn / (Tn - 1)
        adv = extra.get("negative_adversarial_scale", 0)
        if adv:
            w = w * (oh + (Tn - 1) * T.softmax(adv * ts.detach() - 10000 * oh, -1))
        ref = -(w * torch_restatement.log_sigmoid_clamped((2 * oh - 1) * ts)).sum() / (S * B * A * S)
    else:
        cw = extra.get("softmax_correction_weight", 0)
        corr = cw * (np.log(NE * S - 1) - np.log(S * A - 1))
        ref = -(T.log_softmax(ts + corr * (1 - oh), -1) * oh).sum() / (S * B)
    ref.backward()
    tol = 1e-6 if orc.precision == "f64" else 2e-5
    np.testing.assert_allclose(loss, float(ref.detach()), rtol=tol)
    assert K.rel_l2(ds, ts.grad.numpy()) < tol


# ---- whole step vs the independent autograd restatement --------------------

STEP_CASES = {
    "demo_l1_logsigmoid": dict(),
    "l2_logsigmoid_nofeat": dict(distance_fn="L2", feature=0, gamma=4.0),
    "l2_softmax": dict(distance_fn="L2", loss_fn="softmax", softmax_correction_weight=1.0),
    "distmult_softmax_feat": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax",
                                  softmax_correction_weight=1.0, feature=4),
    "transe_matmul": dict(distance_fn="MatMul", feature=0),
    "l1_adversarial": dict(negative_adversarial_scale=1.5),
    "l2_weight_decay": dict(distance_fn="L2", weight_decay=0.01, feature=0),
    "shared_table_l2": dict(distance_fn="L2", shared_table=True, n_shard=4, batch=8, a2a=4,
                            feature=0, n_entity=60, gamma=3.0),
    # ComplEx (src/poplar_kge.cpp:501-514): complex product of head and relation on the
    # (real | imaginary) halves, scored by the distance function's value itself
    "complex_matmul_softmax": dict(score_fn="ComplEx", distance_fn="MatMul", loss_fn="softmax",
                                   softmax_correction_weight=1.0, feature=0),
    "complex_matmul_logsigmoid_feat": dict(score_fn="ComplEx", distance_fn="MatMul", feature=4),
    "complex_l2": dict(score_fn="ComplEx", distance_fn="L2", feature=0),
    "complex_l1": dict(score_fn="ComplEx", distance_fn="L1", feature=0),
    # RotatE (src/poplar_kge.cpp:516-537): rotation of (h_re, h_im) by the relation's phases, whose
    # sine and cosine (and the phases' gradient) run in float16
    "rotate_l1": dict(score_fn="RotatE", distance_fn="L1", feature=0),
    "rotate_l2_feat": dict(score_fn="RotatE", distance_fn="L2", gamma=4.0),
    "rotate_softmax": dict(score_fn="RotatE", distance_fn="L1", loss_fn="softmax", softmax_correction_weight=1.0,
                           feature=0, dim=12),
    # TransH (src/poplar_kge.cpp:539-565): heads and tails projected onto the relation's
    # hyperplane (unit normal from relation_normal), L1 distance whatever distance_fn says
    "transh": dict(score_fn="TransH", feature=0),
    "transh_feat_softmax": dict(score_fn="TransH", distance_fn="L2", loss_fn="softmax",
                                softmax_correction_weight=1.0),
    "transh_shared_table": dict(score_fn="TransH", shared_table=True, n_shard=4, batch=8, a2a=4,
                                feature=0, n_entity=60, gamma=3.0),
    # feature MLP (src/poplar_kge.cpp:453-458): relu([embedding | feature . W] . Up) . Down
    "feature_mlp": dict(feature_mlp_size=10),
    "feature_mlp_l2_softmax_reg": dict(feature_mlp_size=6, distance_fn="L2", loss_fn="softmax",
                                       softmax_correction_weight=1.0, feature_regularisation=(3.0, 2e-2),
                                       hidden_regularisation=(2.0, 1e-2)),
    "feature_mlp_shared_distmult": dict(feature_mlp_size=8, score_fn="DistMult", distance_fn="MatMul",
                                        shared_table=True, n_shard=4, batch=8, a2a=4, feature=4, n_entity=60),
    # feature dropout (src/poplar_kge.cpp:459-461): separate masks for the head and the tail use
    "feature_dropout": dict(feature_dropout=0.3, dropout_seed=7),
    "feature_dropout_mlp_l2": dict(feature_dropout=0.5, dropout_seed=3, feature_mlp_size=6, distance_fn="L2",
                                   loss_fn="softmax", softmax_correction_weight=1.0),
    "feature_dropout_shared_distmult": dict(feature_dropout=0.2, dropout_seed=11, score_fn="DistMult",
                                            distance_fn="MatMul", shared_table=True, n_shard=4, batch=8, a2a=4,
                                            feature=4, n_entity=60),
    # separate feature networks for the head and the tail use (src/poplar_kge.cpp:268-273)
    "separate_networks": dict(share_feature_networks=False),
    "separate_networks_mlp_dropout_l2": dict(share_feature_networks=False, feature_mlp_size=6, feature_dropout=0.3,
                                             dropout_seed=5, distance_fn="L2", loss_fn="softmax",
                                             softmax_correction_weight=1.0),
    "separate_networks_shared_distmult": dict(share_feature_networks=False, score_fn="DistMult", distance_fn="MatMul",
                                              shared_table=True, n_shard=4, batch=8, a2a=4, feature=4, n_entity=60),
    # regularisers where the two entityHidden calls differ: each call's tensors once
    "regularisers_dropout": dict(feature_dropout=0.3, dropout_seed=9, embedding_regularisation=(2.0, 3e-2),
                                 feature_regularisation=(3.0, 2e-2), hidden_regularisation=(4.0, 1e-2)),
    "regularisers_separate_mlp": dict(share_feature_networks=False, feature_mlp_size=6,
                                      feature_regularisation=(3.0, 2e-2), hidden_regularisation=(2.0, 1e-2),
                                      distance_fn="L2"),
    # norm regularisers (src/poplar_kge.cpp:430-437, 463-465), the WikiKG preset's among them
    "feature_regularisation_p3": dict(feature_regularisation=(3.0, 1e-2), loss_fn="softmax",
                                      softmax_correction_weight=1.0),
    "all_regularisers": dict(embedding_regularisation=(2.0, 3e-2), feature_regularisation=(3.0, 2e-2),
                             hidden_regularisation=(4.0, 1e-2), distance_fn="L2"),
    "embedding_regularisation_nofeat": dict(embedding_regularisation=(3.0, 5e-2), feature=0,
                                            hidden_regularisation=(2.0, 1e-2)),
    # bfloat16 scoring operands (this build's option): rounding placement and the
    # straight-through gradient against autograd
    "distmult_bf16_scoring_feat": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax",
                                       softmax_correction_weight=1.0, feature=4, scoring_bf16=True),
    "distmult_bf16_scoring_logsigmoid": dict(score_fn="DistMult", distance_fn="MatMul", feature=0,
                                             scoring_bf16=True),
}


def _run_case(orc, kw, batch_fn, n_step=3, pad=0, lr=(0.1, 0.07)):
    c = K.cfg_dict(**kw)
    rng = np.random.default_rng(11)
    st0 = K.make_state(c, rng)
    batch = batch_fn(c, n_step, rng) if pad == 0 else batch_fn(c, n_step, rng, pad=pad)
    lr = np.resize(np.asarray(lr, np.float32), c["n_shard"])
    if c["shared_table"]:
        lr[:] = lr[0]
    cfg = make_cfg(**{k: v for k, v in c.items()})
    st_o = K.copy_state(st0)
    loss_o = orc.train_step_loop(cfg, st_o, lr, batch)
    st_t = K.copy_state(st0)
    losses = [torch_restatement.step(c, st_t, lr, K.step_slice(batch, i)) for i in range(n_step)]
    loss_t = np.mean(losses, 0)
    tol = 2e-6 if orc.precision == "f64" else 1e-4
    np.testing.assert_allclose(loss_o, loss_t, rtol=tol)
    assert st_o["step"] == st_t["step"] == st0["step"] + n_step
    for k in st0:
        if k == "step":
            continue
        d_o, d_t = st_o[k] - st0[k], st_t[k] - st0[k]
        assert K.rel_l2(d_o, d_t) < tol * 5, k
        assert np.any(d_t != 0), k
    return c, st0, st_o, batch


@pytest.mark.parametrize("name", ["l2_logsigmoid_nofeat", "transe_matmul", "shared_table_l2", "l1_adversarial"])
def test_gradient_tap_vs_autograd(orc, name):
    """The oracle's gradient tap (the summed gradient of every gathered row and of every relation
    row, as the updates use them) against autograd's gradients of the independent restatement."""
    c = K.cfg_dict(**dict(STEP_CASES[name], feature=0))
    rng = np.random.default_rng(4)
    st0 = K.make_state(c, rng)
    batch = K.random_batch(c, 1, rng)
    lr = np.full(c["n_shard"], 0.05, np.float32)
    n_rows = st0["entity_data"].shape[0]
    ent = np.full((n_rows, c["dim"]), np.nan)
    rel = np.full((c["n_relation"], c["dim"]), np.nan)
    orc.gradient_tap(ent, rel)
    try:
        orc.train_step_loop(make_cfg(**c), K.copy_state(st0), lr, batch)
    finally:
        orc.gradient_tap(None, None)
    grads = {}
    torch_restatement.step(c, K.copy_state(st0), lr, K.step_slice(batch, 0), grads)
    tol = 1e-9 if orc.precision == "f64" else 2e-4
    assert np.array_equal(np.flatnonzero(~np.isnan(ent[:, 0])), grads["rows"])   # exactly the gathered rows
    assert K.rel_l2(ent[grads["rows"]], grads["entity"]) < tol
    assert K.rel_l2(rel, grads["relation"]) < tol
    assert np.any(grads["entity"] != 0) and np.any(grads["relation"] != 0)


@pytest.mark.parametrize("name", list(STEP_CASES))
def test_train_step_vs_autograd(orc, name):
    _run_case(orc, STEP_CASES[name], K.random_batch)


def test_complex_score_is_real_part_of_hermitian_product(orc):
    """ComplEx with the dot product scores Re(<h r, conj t>): checked against numpy's complex
    arithmetic through the loss of a one-positive, two-tail step (softmax cross entropy of
    the two scores, closed form)."""
    c = K.cfg_dict(score_fn="ComplEx", distance_fn="MatMul", loss_fn="softmax", feature=0, n_shard=1,
                   batch=1, a2a=2, dim=6, n_entity=5, n_relation=2)
    rng = np.random.default_rng(5)
    st = K.make_state(c, rng)
    batch = dict(remote=np.array([[[1, 2, 3]]], np.uint32), a2a=np.array([[[[1, 2]]]], np.uint32),
                 head=np.array([[[0]]], np.uint32), relation=np.array([[[1]]], np.uint32),
                 tail=np.array([[[1]]], np.uint32))
    e, r = st["entity_data"][:, :6].astype(np.float64), st["relation_embedding"][1].astype(np.float64)
    z = lambda v: v[:3] + 1j * v[3:]  # noqa: E731
    scores = np.array([np.real(np.sum(z(e[1]) * z(r) * np.conj(z(e[t])))) for t in (2, 3)])
    want = -(scores[1] - np.log(np.exp(scores).sum()))
    got = orc.train_step_loop(make_cfg(**c), K.copy_state(st), 0.01, batch)
    np.testing.assert_allclose(got, [want], rtol=2e-6 if orc.precision == "f64" else 1e-5)


def test_lpnorm_closed_forms(orc):
    """One gathered row, no positives' gradient reaching it: the loss's regularisation part and the
    row's update follow from the p-norm's closed forms (p = 2: the Euclidean norm, gradient
    x / |x|; a zero row: norm 0 and, by the reference's guarded pow backward, zero gradient)."""
    c = K.cfg_dict(feature=0, n_shard=1, batch=1, a2a=2, dim=4, n_entity=6, n_relation=1,
                   embedding_regularisation=(2.0, 0.5), loss_scale=1.0)
    rng = np.random.default_rng(2)
    st = K.make_state(c, rng, warm=False)
    st["entity_data"][4, :4] = [3.0, 0.0, -4.0, 0.0]       # |x| = 5, not referenced by any slot
    st["entity_data"][5, :4] = 0.0                          # a zero row
    batch = dict(remote=np.array([[[1, 4, 5]]], np.uint32), a2a=np.array([[[[0, 0]]]], np.uint32),
                 head=np.array([[[0]]], np.uint32), relation=np.array([[[0]]], np.uint32),
                 tail=np.array([[[0]]], np.uint32))
    plain = dict(c, embedding_regularisation=(2.0, 0.0))
    st_a, st_b = K.copy_state(st), K.copy_state(st)
    loss_a = orc.train_step_loop(make_cfg(**c), st_a, 0.1, batch)
    loss_b = orc.train_step_loop(make_cfg(**plain), st_b, 0.1, batch)
    norms = np.linalg.norm(st["entity_data"][[1, 4, 5], :4].astype(np.float64), axis=1)
    np.testing.assert_allclose(loss_a - loss_b, [2 * 0.5 * norms.sum()], rtol=1e-5)
    # row 4: gradient 2 * 0.5 * x / |x| = (0.6, 0, -0.8, 0): the first Adam step moves each
    # non-zero element by lr against its sign, zero elements stay
    d4 = st_a["entity_data"][4, :4] - st["entity_data"][4, :4]
    np.testing.assert_allclose(d4, [-0.1, 0.0, 0.1, 0.0], rtol=1e-4, atol=1e-9)
    np.testing.assert_array_equal(st_a["entity_data"][5, :4], 0.0)


def test_train_step_padding_rows(orc):
    # zero-padded `remote` (src/python/poplar_kge_dataset.py:161-164): row 0 is
    # gathered several times per shard and updated once with zero gradient
    c, st0, st1, batch = _run_case(orc, dict(feature=0), K.random_batch, pad=4)
    D = c["dim"]
    for s in range(c["n_shard"]):
        r0 = s * c["n_entity"]
        # emb moves only through the decaying momentum; m and sqrt(v) decay
        np.testing.assert_allclose(st1["entity_data"][r0, D:2 * D],
                                   st0["entity_data"][r0, D:2 * D] * 0.9**3, rtol=1e-5)


def test_train_step_raw_duplicates_shared(orc):
    # raw Zipf ids with identity slots in a shared table: heavy duplicates
    _run_case(orc, dict(distance_fn="L2", shared_table=True, n_shard=4, batch=8, a2a=4, feature=0,
                        n_entity=40, gamma=3.0), K.raw_batch)


def test_untouched_rows_unchanged(orc):
    c = K.cfg_dict(feature=0)
    rng = np.random.default_rng(0)
    st0 = K.make_state(c, rng)
    batch = K.random_batch(c, 2, rng)
    st = K.copy_state(st0)
    orc.train_step_loop(make_cfg(**c), st, 0.1, batch)
    touched = np.zeros(st0["entity_data"].shape[0], bool)
    for s in range(c["n_shard"]):
        touched[s * c["n_entity"] + batch["remote"][s].ravel()] = True
    np.testing.assert_array_equal(st["entity_data"][~touched], st0["entity_data"][~touched])
    assert np.all(np.any(st["entity_data"][touched] != st0["entity_data"][touched], axis=1))


def test_storage_rounding(orc):
    x = np.array([1.0, 1.0 + 2**-9, 1.0 + 3 * 2**-9, 65519.0, 65520.0, 1e-7, -3.14159], np.float32)
    np.testing.assert_array_equal(orc.round(x, "float16"), x.astype(np.float16).astype(np.float32))
    bf = T.tensor(x).to(T.bfloat16).to(T.float32).numpy()
    np.testing.assert_array_equal(orc.round(x, "bfloat16_embedding"), bf)


# ---- predict reference ------------------------------------------------------

def test_predict_reference_by_hand():
    # two shards of three rows (row 0 padding), D = 1: scores are gamma - |h + r - t|
    from oracle.kge_oracle import predict_reference

    cfg = make_cfg(n_shard=2, n_entity=3, n_relation=2, dim=1, feature=0, batch=1, a2a=1, gamma=10.0)
    rows = np.zeros((6, 3), np.float32)
    rows[:, 0] = [99, 1.0, 2.0,      # shard 0: padding, rows 1, 2
                  99, 4.0, -1.0]     # shard 1: padding, rows 1, 2
    state = {"entity_data": rows, "relation_embedding": np.array([[0.5], [-3.0]], np.float32)}
    queries = np.array([[0, 1, 0],    # h = 1.0, r = 0.5 -> 1.5: 1.0 and 2.0 tie at 0.5, 4.0 and -1.0 at 2.5
                        [1, 1, 1]])   # h = 4.0, r = -3 -> 1.0: nearest 1.0, then 2.0, -1.0, 4.0
    idx, score = predict_reference(cfg, state, queries, [2, 2], 3)
    np.testing.assert_array_equal(idx[0], [[0, 1], [0, 2], [1, 1]])   # ties -> lower (shard, row)
    np.testing.assert_allclose(score[0], [9.5, 9.5, 7.5])
    np.testing.assert_array_equal(idx[1], [[0, 1], [0, 2], [1, 2]])
    np.testing.assert_allclose(score[1], [10.0, 9.0, 8.0])
    # rows past a shard's count never appear, nor does the padding row
    idx, score = predict_reference(cfg, state, queries, [1, 2], 3)
    np.testing.assert_array_equal(idx[1], [[0, 1], [1, 2], [1, 1]])
    np.testing.assert_allclose(score[1], [10.0, 8.0, 7.0])


def test_predict_reference_vs_torch_topk():
    # against the form of tests/python/reference_model.py:169-206: mask, broadcast score, topk
    import torch as T
    from oracle.kge_oracle import predict_reference

    rng = np.random.default_rng(5)
    S, NE, D, F, NR = 3, 40, 8, 4, 6
    for kw in (dict(distance_fn="L1"), dict(distance_fn="L2"), dict(score_fn="DistMult", distance_fn="MatMul")):
        cfg = make_cfg(n_shard=S, n_entity=NE, n_relation=NR, dim=D, feature=F, batch=2, a2a=2, gamma=3.0, **kw)
        st = {"entity_data": rng.normal(size=(S * NE, 3 * D + F)).astype(np.float32),
              "relation_embedding": rng.normal(size=(NR, D)).astype(np.float32),
              "feature_projection": rng.normal(size=(F, D)).astype(np.float32)}
        counts = [NE - 1, NE - 5, NE - 9]
        q = np.stack([rng.integers(0, S, 17), rng.integers(1, NE - 9, 17), rng.integers(0, NR, 17)], -1)
        idx, score = predict_reference(cfg, st, q, counts, 7)
        e = T.tensor(st["entity_data"], dtype=T.float64)
        hid = e[:, :D] + e[:, 3 * D:] @ T.tensor(st["feature_projection"], dtype=T.float64)
        rel = T.tensor(st["relation_embedding"], dtype=T.float64)[q[:, 2]]
        h = hid[q[:, 0] * NE + q[:, 1]]
        if kw.get("score_fn") == "DistMult":
            sc = (h * rel) @ hid.T
        else:
            sc = 3.0 - T.cdist(h + rel, hid, p=1 if kw["distance_fn"] == "L1" else 2)
        mask = T.zeros(S, NE, dtype=T.float64)
        for i, n in enumerate(counts):
            mask[i, 0] = -1e4
            mask[i, 1 + n:] = -1e4
        top = T.topk(sc + mask.reshape(-1), k=7)
        np.testing.assert_allclose(score, top.values.numpy(), rtol=1e-12, atol=1e-12)
        np.testing.assert_array_equal(idx[..., 0] * NE + idx[..., 1], top.indices.numpy())


def test_predict_reference_transh_by_hand_and_invariances():
    # D = 2, normal along x (any length): heads and tails lose their x part, so the score is
    # gamma - (|r_x| + |h_y + r_y - t_y|) with r's own x part surviving (src/poplar_kge.cpp:539-565)
    from oracle.kge_oracle import predict_reference

    cfg = make_cfg(n_shard=1, n_entity=4, n_relation=1, dim=2, feature=0, batch=1, a2a=1, gamma=10.0,
                   score_fn="TransH")
    rows = np.zeros((4, 6), np.float32)
    rows[:, :2] = [[0, 0], [5.0, 1.0], [-7.0, 2.5], [100.0, 0.0]]
    state = {"entity_data": rows, "relation_embedding": np.array([[0.25, 1.0]], np.float32),
             "relation_normal": np.array([[3.0, 0.0]], np.float32)}
    idx, score = predict_reference(cfg, state, np.array([[0, 1, 0]]), [3], 3)
    # h = (5, 1): projected (0, 1), + r = (0.25, 2); tails projected (0, 1), (0, 2.5), (0, 0)
    np.testing.assert_allclose(score[0], [10 - 0.75, 10 - 1.25, 10 - 2.25])
    np.testing.assert_array_equal(idx[0], [[0, 2], [0, 1], [0, 3]])
    # invariances on random data: the length of the raw normal, and any multiple of the normal
    # added to an entity, leave every score as it is
    rng = np.random.default_rng(3)
    NE, D, NR = 30, 6, 4
    cfg = make_cfg(n_shard=1, n_entity=NE, n_relation=NR, dim=D, feature=0, batch=1, a2a=1, gamma=2.0,
                   score_fn="TransH")
    st = {"entity_data": rng.normal(size=(NE, 3 * D)).astype(np.float32),
          "relation_embedding": rng.normal(size=(NR, D)).astype(np.float32),
          "relation_normal": rng.normal(size=(NR, D)).astype(np.float32)}
    q = np.stack([np.zeros(5, int), rng.integers(1, NE, 5), np.full(5, 2)], -1)
    idx0, score0 = predict_reference(cfg, st, q, [NE - 1], NE - 1)
    st2 = {k: v.copy() for k, v in st.items()}
    st2["relation_normal"][2] *= 4.0
    st2["entity_data"][1:, :D] += rng.normal(size=(NE - 1, 1)).astype(np.float32) * st["relation_normal"][2]
    idx1, score1 = predict_reference(cfg, st2, q, [NE - 1], NE - 1)
    np.testing.assert_allclose(score1, score0, rtol=0, atol=2e-5)


def test_dropout_mask_is_the_same_in_c_and_numpy_and_keeps_the_right_share(orc):
    import ctypes as C
    from oracle.kge_oracle import dropout_keep

    orc.lib.kge_dropout_keep.restype = C.c_int
    orc.lib.kge_dropout_keep.argtypes = [C.c_uint32] * 5 + [C.c_float]
    rng = np.random.default_rng(0)
    keys = rng.integers(0, 2**32, 200, dtype=np.uint64)
    for p in (0.1, 0.5, 0.9):
        want = [orc.lib.kge_dropout_keep(9, 12345, 1, int(k), 17, p) for k in keys]
        np.testing.assert_array_equal(dropout_keep(9, 12345, 1, keys, 17, p), np.array(want, bool))
        share = dropout_keep(9, 3, 0, np.arange(1, 4001)[:, None], np.arange(64)[None, :], p).mean()
        assert abs(share - (1 - p)) < 0.01, (p, share)
    # heads' and tails' masks, and successive steps', are different draws
    a = dropout_keep(9, 3, 0, np.arange(4000), 5, 0.5)
    assert 0.4 < (a != dropout_keep(9, 3, 1, np.arange(4000), 5, 0.5)).mean() < 0.6
    assert 0.4 < (a != dropout_keep(9, 4, 0, np.arange(4000), 5, 0.5)).mean() < 0.6
