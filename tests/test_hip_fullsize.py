"""GPU parity at the full benchmark sizes (c2: 1M-row float32 table; c3: 22.8M rows,
70 GB; c4: 4M rows with 768 float16 features, DistMult, softmax; c5: 91.2M rows
with bfloat16 embeddings, 233 GB): the table is
initialised on the device, the rows a few steps touch are read back, the CPU
oracle runs the same steps on a compacted copy of exactly those rows, and the
updated rows, the relation table and the loss are compared.  Also: rows nobody
referenced are bit-identical afterwards, and a second engine reproduces the
first bit for bit."""

import numpy as np
import pytest

import kge_cases as K
import kge_synthetic as W
from oracle.kge_oracle import Oracle, make_cfg

pytestmark = pytest.mark.gpu


def _free_gpu_bytes():
    import torch

    return torch.cuda.mem_get_info()[0]


def _close_but_for_sign_flips(got, ref, what, max_flip_fraction=5e-4, tol=1e-5):
    """Adam's first steps from zero moments move a parameter by about
    lr * sign(g): where a gradient element is an exact cancellation (common for
    L1, whose terms are +-c) its sign is decided by rounding, and float32 and
    float64 may disagree.  Such elements are allowed, rarely; all the others
    must agree to 1e-5."""
    scale = np.sqrt(np.mean(np.asarray(ref, np.float64)**2))
    bad = np.abs(got - ref) > 10 * tol * scale
    assert bad.mean() < max_flip_fraction, (what, bad.mean())
    assert K.rel_l2(np.where(bad, 0, got), np.where(bad, 0, ref)) < tol, what


def _run(workload, n_step, rng_rows=2000, **override):
    import poplar_kge as kge

    w = dict(W.WORKLOADS[workload], **override)
    need = w["n_entity"] * W.row_bytes(w) + (4 << 30)
    if _free_gpu_bytes() < need:
        pytest.skip(f"needs {need >> 30} GiB of free HBM")
    settings = W.make_settings(w, n_step, kge)
    m, d = settings.model, settings.data
    engine = kge.Engine(settings, np.full(m.n_shard, m.n_entity - 1))
    W.init_tables(engine, settings)
    batch = W.make_batch(w, n_step, kge)

    ids = np.unique(batch.remote)                       # every row the steps touch
    rng = np.random.default_rng(1)
    others = np.setdiff1d(rng.integers(1, m.n_entity, rng_rows).astype(np.uint32), ids)
    before = W.read_rows(engine, settings, ids)
    before_others = W.read_rows(engine, settings, others)
    # the generator gives N(0, init_scale / D) embeddings and zero moments
    D = m.embedding_size
    assert abs(before[:, :D].std() * np.sqrt(D) - 1.0) < 0.02 and abs(before[:, :D].mean()) < 1e-3
    assert np.all(before[:, D:3 * D] == 0)

    dense = ["relation_embedding"] + (["feature_projection"] if m.entity_feature_size else [])
    dense_before = {k + sfx: engine.read_variable(k + sfx) for k in dense for sfx in ("", "/adam_m", "/adam_v")}
    loss, _ = engine.train_step_loop(batch)
    after = W.read_rows(engine, settings, ids)
    after_others = W.read_rows(engine, settings, others)
    np.testing.assert_array_equal(after_others, before_others)

    # the oracle on a compact table: row k+1 of the copy is table row ids[k]
    compact = np.zeros((ids.size + 1, before.shape[1]), np.float32)
    compact[1:] = before
    remap = lambda a: (1 + np.searchsorted(ids, a)).astype(np.uint32)
    state = {"entity_data": compact, "step": 0}
    state.update(dense_before)
    storage = "bfloat16_embedding" if w.get("embedding_dtype") == "bfloat16" else "float32"
    softmax = w.get("loss") == "softmax"
    # the softmax correction term reads n_entity: the oracle gets the real table size for it
    cfg = make_cfg(n_shard=m.n_shard, n_entity=m.n_entity if softmax else compact.shape[0],
                   n_relation=m.n_relation_type, dim=D,
                   feature=m.entity_feature_size, batch=d.batch_size, a2a=d.a2a_size,
                   score_fn=m.score_fn, distance_fn=m.distance_fn,
                   loss_fn="softmax" if softmax else "logsigmoid",
                   softmax_correction_weight=1.0 if softmax else 0.0,
                   shared_table=True, gamma=m.gamma, loss_scale=settings.training.loss_scale,
                   scoring_bf16=w.get("scoring_dtype") == "bfloat16", storage=storage)
    ob = {k: v for k, v in vars(batch).items()}
    ob["remote"] = remap(batch.remote)
    loss_o = Oracle("f64").train_step_loop(cfg, state, settings.training.learning_rate, ob)
    # bfloat16 scoring: the oracle rounds the same operands, so the loss stays tight; the
    # coefficient matrix is a bfloat16 operand of the backward products on the device only
    # (2^-9 relative per element): gradients, and with them the moments, hold bf16's 2e-2 bar
    bf16_scoring = w.get("scoring_dtype") == "bfloat16"
    tol = 2e-2 if bf16_scoring else 1e-5
    flips = 2e-2 if bf16_scoring else 5e-4   # cold-start sign flips of near-zero gradient elements
    np.testing.assert_allclose(loss, float(np.sum(loss_o)), rtol=1e-4 if bf16_scoring else 1e-5)
    ref = state["entity_data"][1:]
    assert np.all(np.any(after != before, axis=1))       # every touched row moved
    if storage == "float32":
        _close_but_for_sign_flips(after, ref, "entity rows", flips, tol)
    else:
        assert K.rel_l2(after[:, D:], ref[:, D:]) < 1e-5          # float32 moments
        assert K.rel_l2(after[:, :D], ref[:, :D]) < 2e-3          # bfloat16 embedding (bar: 2e-2)
        assert np.mean(after[:, :D] != ref[:, :D]) < 2e-3
    for name in dense:
        _close_but_for_sign_flips(engine.read_variable(name), state[name], name, flips, tol)
        # the dense tables keep v = E[g^2]; the bar is on |g|-like quantities, as for the rows' sqrt(v)
        assert K.rel_l2(np.sqrt(engine.read_variable(name + "/adam_v")),
                        np.sqrt(state[name + "/adam_v"])) < tol, name
    return settings, batch, ids, after, loss


@pytest.mark.parametrize("scoring", ["mfma_bf16x3", "mfma", "valu"])
def test_c1_full_size_vs_oracle(scoring):
    """The smallest listed configuration (TransE-L2 D=64, 10k entities, 256 positives x 64 shared
    tails, uniform ids): one block, the smallest shape the aligned scoring tiles take, under
    every scoring path."""
    _run("c1", n_step=3, scoring=scoring)


def test_c2_full_size_vs_oracle_and_deterministic():
    import poplar_kge as kge

    import gc

    settings, batch, ids, after, loss = _run("c2", n_step=3)
    gc.collect()
    # a second engine, same seeds, same batch: bit-identical rows and loss
    m = settings.model
    engine = kge.Engine(settings, np.full(m.n_shard, m.n_entity - 1))
    W.init_tables(engine, settings)
    loss2, _ = engine.train_step_loop(batch)
    assert loss2 == loss
    np.testing.assert_array_equal(W.read_rows(engine, settings, ids), after)


def test_c3_full_size_vs_oracle():
    _run("c3", n_step=1)


def test_c3_l2_full_size_vs_oracle():
    _run("c3l2", n_step=2)


def test_c4_full_size_vs_oracle():
    # DistMult + 768 -> 512 feature projection + softmax CE, 8192 x 2048 scores,
    # bfloat16 scoring operands on the matrix cores
    _run("c4", n_step=1)


def test_c4_float32_scoring_full_size_vs_oracle():
    _run("c4", n_step=1, scoring_dtype=None)


def test_c5_full_size_vs_oracle():
    _run("c5", n_step=2)


@pytest.mark.parametrize("distance_fn", ["L2", "L1"])
def test_predict_full_size_vs_brute_force(distance_fn):
    """Engine.predict over one shard's 1M-row table (fifteen whole chunks of tails scored
    where they lie in the table, one partial chunk through the dense copy, the merge on its
    own stream) against a float64 brute force over every row, for 128 queries and the
    reference's n_best (src/python/poplar_kge.py:395-397; oracle tests/python/reference_model.py:169-206)."""
    import gc

    import poplar_kge as kge

    gc.collect()
    s = kge.Settings.create_demo()
    s.seed = 4242
    m, d, e = s.model, s.data, s.execution
    m.score_fn, m.distance_fn, m.n_shard = "TransE", distance_fn, 1
    m.n_entity, m.n_relation_type, m.embedding_size, m.entity_feature_size = 1_000_000, 1000, 256, 0
    m.gamma, m.init_scale = 10.0, 16.0
    d.batch_size, d.a2a_size = 256, 256
    e.device, e.dtype, e.shared_table, e.rw_batch_size = "hip", "float32", False, 8192
    e.train_steps_per_program_run, e.predict_hr_batch_size, e.predict_n_best = 1, 128, 100
    settings = s.prepare()
    count = m.n_entity - 12345   # the last rows of the table do not take part
    engine = kge.Engine(settings, np.full(1, count))
    W.init_tables(engine, settings)
    n = 128 + 7                  # a second, mostly empty program run
    rng = np.random.default_rng(5)
    queries = np.stack([np.zeros(n, np.uint32), rng.integers(1, count + 1, n).astype(np.uint32),
                        rng.integers(0, m.n_relation_type, n).astype(np.uint32)], axis=-1)
    found = engine.predict(queries)

    D = m.embedding_size
    table = W.read_rows(engine, settings, np.arange(0, count + 1, dtype=np.uint32))[:, :D].astype(np.float64)
    rel = engine.read_variable("relation_embedding").reshape(-1, D).astype(np.float64)
    for q in range(0, n, 9):   # fifteen of the queries, both program runs
        diff = (table[queries[q, 1]] + rel[queries[q, 2]])[None, :] - table[1:]
        dist = np.sqrt(np.einsum("nd,nd->n", diff, diff)) if distance_fn == "L2" else np.abs(diff).sum(-1)
        score = m.gamma - dist
        order = np.lexsort((np.arange(count), -score))[:e.predict_n_best]
        np.testing.assert_allclose(found.score[q], score[order], rtol=1e-5, atol=1e-5)
        agree = found.shard_idx[q, :, 1] == order + 1
        close = np.abs(found.score[q] - score[order]) <= 1e-5 * np.maximum(1.0, np.abs(score[order]))
        assert np.all(agree | close) and agree.mean() > 0.97
        assert np.all(found.shard_idx[q, :, 0] == 0)


def test_predict_shared_table_vs_brute_force():
    """`predict` with one table shared by the blocks (this build's layout for the benchmark
    shapes): the table is swept in n_shard contiguous row ranges, the returned rows are table
    rows, and the ranges' n_best pooled give the overall n_best of a float64 brute force."""
    import gc

    import poplar_kge as kge

    gc.collect()
    w = dict(W.WORKLOADS["c2"], n_entity=50_000, blocks=4, n_relation=40, dim=64, batch=32, tails=32)
    settings = W.make_settings(w, 1, kge)
    m, e = settings.model, settings.execution
    e.predict_hr_batch_size, e.predict_n_best, e.predict_chunk_rows = 16, 50, 4096
    S, Hb, nb, D = m.n_shard, 16, 50, m.embedding_size
    count = m.n_entity - 77
    engine = kge.Engine(settings, np.full(S, count))
    W.init_tables(engine, settings)
    rng = np.random.default_rng(11)
    head = rng.integers(1, count + 1, (S, Hb)).astype(np.uint32)
    relation = rng.integers(0, m.n_relation_type, (S, Hb)).astype(np.uint32)
    scores = np.full((S, S, Hb, nb), np.nan, np.float32)
    rows = np.zeros(scores.shape, np.uint32)
    engine.engine.run("predict", dict(predict_head=head, predict_relation=relation,
                                      predict_entity_count=np.full(S, count, np.uint32),
                                      predict_scores=scores, predict_indices=rows))
    table = W.read_rows(engine, settings, np.arange(0, count + 1, dtype=np.uint32))[:, :D].astype(np.float64)
    rel = engine.read_variable("relation_embedding").reshape(-1, D).astype(np.float64)
    per_range = -(-(m.n_entity - 1) // S)
    for s in range(S):
        for q in range(0, Hb, 5):
            diff = (table[head[s, q]] + rel[relation[s, q]])[None, :] - table[1:]
            score = m.gamma - np.sqrt(np.einsum("nd,nd->n", diff, diff))
            for ts in range(S):   # each range's own n_best, rows inside the range
                lo, hi = 1 + ts * per_range, min(1 + (ts + 1) * per_range, count + 1)
                assert np.all((rows[s, ts, q] >= lo) & (rows[s, ts, q] < hi))
                order = lo + np.lexsort((np.arange(hi - lo), -score[lo - 1:hi - 1]))[:nb]
                np.testing.assert_allclose(scores[s, ts, q], score[order - 1], rtol=1e-5, atol=1e-5)
                assert np.mean(rows[s, ts, q] == order) > 0.95
