"""The reference's end-to-end protocols on the HIP device, driven through the
host mirror exactly as tests/python/test_poplar_kge.py drives the IPU:
``test_engine_ops`` (:111-175, without predict) and ``test_training``
(:178-259: the S=2 demo preset, generated data, features through
``initialise_all``, three batches cycled for program_runs_per_log *
logs_per_training_run program runs).  The role of reference_model.Model is
taken by the float64 oracle started from the engine's own initial state; bars
are the reference's: loss rtol 1e-4, (final - initial) within 1e-4 relative."""

import itertools

import numpy as np
import pytest

import kge_cases as K
from oracle.kge_oracle import Oracle, make_cfg

pytestmark = pytest.mark.gpu


def _random_batch(engine):
    """Distinct non-zero sorted remote rows per (shard, step); random slots,
    relations and labels (the reference's helper, :51-91)."""
    import poplar_kge as kge

    s = engine.settings
    n_step, S = s.execution.train_steps_per_program_run, s.model.n_shard
    remote = np.stack([np.sort(engine.random.choice(np.arange(1, s.model.n_entity), s.n_remote, replace=False))
                       for _ in range(S * n_step)]).reshape(S, n_step, s.n_remote).astype(np.uint32)
    return kge.Batch(
        remote=remote,
        a2a=engine.random_integers(s.n_remote, (S, n_step, S, s.data.a2a_size)),
        head=engine.random_integers(s.n_remote, (S, n_step, s.data.batch_size)),
        relation=engine.random_integers(s.model.n_relation_type, (S, n_step, s.data.batch_size)),
        tail=engine.random_integers(s.n_tail, (S, n_step, s.data.batch_size)))


def _oracle_cfg(settings):
    m, d, t = settings.model, settings.data, settings.training
    storage = "float16" if settings.execution.dtype == "float16" else "float32"
    return make_cfg(n_shard=m.n_shard, n_entity=m.n_entity, n_relation=m.n_relation_type,
                    dim=m.embedding_size, feature=m.entity_feature_size, batch=d.batch_size,
                    a2a=d.a2a_size, score_fn=m.score_fn, distance_fn=m.distance_fn,
                    loss_fn=t.loss.type, gamma=m.gamma, beta_m=t.adam_beta_m, beta_v=t.adam_beta_v,
                    epsilon=t.adam_epsilon, weight_decay=t.weight_decay, loss_scale=t.loss_scale,
                    storage=storage, feature_mlp_size=m.feature_mlp_size,
                    share_feature_networks=m.share_feature_networks)


def _oracle_state(state):
    out = {k: np.array(v, np.float32) for k, v in state.items() if k != "step"}  # copies: the oracle works in place
    out["entity_data"] = np.array(state["entity_data"].reshape(-1, state["entity_data"].shape[-1]), np.float32)
    (out["step"],) = set(int(x) for x in np.ravel(state["step"]))
    return out


def test_engine_ops():
    import poplar_kge as kge

    settings = kge.Settings.create_demo()
    settings.seed = 100
    settings.training.learning_rate = 0.01
    settings.prepare()
    m = settings.model
    engine = kge.Engine(settings, np.full(m.n_shard, m.n_entity - 1))

    features = engine.random_normal((m.n_shard, m.n_entity, m.entity_feature_size), np.float16)
    features[:, 0, :] = 0
    engine.initialise_all(features)
    batch = _random_batch(engine)
    loss_0, _ = engine.train_step_loop(batch)
    loss_1, _ = engine.train_step_loop(batch)
    assert loss_1 < loss_0

    new_relation = engine.random_normal(engine.variable_to_shape["relation_embedding"])
    assert not np.allclose(engine.read_variable("relation_embedding"), new_relation)
    engine.write_variable("relation_embedding", new_relation)
    np.testing.assert_allclose(engine.read_variable("relation_embedding"), new_relation)

    np.testing.assert_allclose(engine.read_entity_all()[:, :, -m.entity_feature_size:], features)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_training(dtype):
    import poplar_kge as kge
    import poplar_kge_dataset as kge_data

    settings = kge.Settings.create_demo()
    settings.seed = 100
    settings.execution.dtype = dtype
    if dtype == "float16":
        settings.training.n_step = 20  # "since numerical errors compound" (the reference, :184-185)
    settings.prepare()
    data = kge_data.RawData.load(settings)
    dataset = kge_data.Dataset.load(data, settings)
    engine = kge.Engine(settings, dataset.shard_to_count)
    engine.initialise_all(dataset.entity_features(settings.model.entity_feature_size))
    initial = engine.read_all()
    cfg, oracle = _oracle_cfg(settings), Oracle("f64")
    ref = _oracle_state(initial)

    # the reference keeps 'remote' the same in every batch (its torch model updates
    # every row on every step); the protocol is kept although the oracle does not need it
    batches = [_random_batch(engine) for _ in range(3)]
    for b in batches:
        b.remote[...] = batches[0].remote[:, 0, np.newaxis, :]
    n_loop = settings.program_runs_per_log * settings.logs_per_training_run
    assert n_loop == dict(float32=20, float16=4)[dtype]

    loss, ref_loss = [], []
    for b in itertools.islice(itertools.cycle(batches), n_loop):
        step_loss, lr = engine.train_step_loop(b)
        loss.append(step_loss)
        ref_loss.append(float(np.sum(oracle.train_step_loop(cfg, ref, lr, vars(b)))))
    np.testing.assert_allclose(loss, ref_loss, rtol=dict(float16=2e-3, float32=1e-4)[dtype])

    final = engine.read_all()
    assert set(np.ravel(final.pop("step"))) == {ref["step"]} == {5 * n_loop}
    first = _oracle_state(initial)
    for key, value in final.items():
        value = value.reshape(ref[key].shape)
        delta, ref_delta = value - first[key], ref[key] - first[key]
        assert np.any(ref_delta != 0), key
        distance = K.rel_l2(delta, ref_delta)
        tolerance = dict(float16=1e-1, float32=1e-4)[dtype]   # the reference's bars (:251)
        assert distance <= tolerance, f"(final - initial) of '{key}' is {distance:.2g} away from the oracle's"


def test_training_from_sampled_batches():
    """The sampler's batches (de-duplicated, and raw ids merged on the device)
    drive the same training run to the same result."""
    import poplar_kge as kge
    import poplar_kge_dataset as kge_data

    settings = kge.Settings.create_demo()
    settings.seed = 7
    settings.prepare()
    data = kge_data.RawData.load(settings)
    results = []
    for dedup in (True, False):
        dataset = kge_data.Dataset.load(data, settings)
        engine = kge.Engine(settings, dataset.shard_to_count)
        engine.initialise_all(dataset.entity_features(settings.model.entity_feature_size))
        if not dedup:  # same rows as the first engine (write_entity draws per (seed, row, column))
            np.testing.assert_array_equal(engine.read_entity_all(), results[0][2])
        start = engine.read_entity_all()
        ref = _oracle_state(engine.read_all())
        losses = []
        for _ in range(4):
            b = dataset.sample_batch(deduplicate=dedup)
            l, lr = engine.train_step_loop(b)
            lo = float(np.sum(Oracle("f64").train_step_loop(_oracle_cfg(settings), ref, lr, vars(b))))
            np.testing.assert_allclose(l, lo, rtol=1e-4)
            losses.append(l)
        results.append((losses, engine.read_entity_all(), start))
    # raw ids visit the same entities in the same roles; rows that are gathered but carry no
    # gradient differ (padding slots do not exist in raw mode), trained rows agree
    np.testing.assert_allclose(results[0][0], results[1][0], rtol=1e-5)


def _random_queries(engine, n):
    s = engine.settings
    return np.stack([engine.random_integers(s.model.n_shard, (n,)),
                     1 + engine.random_integers(s.model.n_entity - 1, (n,)),
                     engine.random_integers(s.model.n_relation_type, (n,))], axis=-1)


@pytest.mark.parametrize("variant", ["demo_l1", "l2", "distmult", "complex", "rotate", "transh", "transh_big",
                                     "feature_mlp", "feature_dropout", "separate_networks_mlp",
                                     "no_features_big", "n_best_max", "one_chunk",
                                     "l1_big", "distmult_big", "bf16_rows_big"])
def test_predict_vs_brute_force(variant):
    """Engine.predict against a float64 brute force over every row of every shard
    (the reference checks shapes, ranges and ordering, tests/python/test_poplar_kge.py:155-175,
    and the MRR against its torch model, :214-236)."""
    import poplar_kge as kge
    from oracle.kge_oracle import predict_reference

    settings = kge.Settings.create_demo()
    settings.seed = 100
    m, ex = settings.model, settings.execution
    if variant == "l2":
        m.distance_fn = "L2"
    elif variant == "distmult":
        m.score_fn, m.distance_fn = "DistMult", "MatMul"
    elif variant == "complex":
        m.score_fn, m.distance_fn = "ComplEx", "MatMul"
    elif variant == "rotate":
        m.score_fn = "RotatE"
    elif variant == "transh":
        m.score_fn = "TransH"
    elif variant == "feature_mlp":
        m.feature_mlp_size = 24
    elif variant == "separate_networks_mlp":
        m.share_feature_networks, m.feature_mlp_size = False, 16
    elif variant == "feature_dropout":
        m.feature_dropout = 0.4   # training only (entityHidden(..., training=false), src/poplar_kge.cpp:419-422)
    elif variant in ("n_best_max", "one_chunk"):
        # the whole shard in one chunk of tails (several spans of the merge, the first ones with more
        # candidates than its list holds); the largest n_best the device keeps
        m.n_entity, m.entity_feature_size, m.embedding_size, m.n_shard = 20000, 0, 32, 2
        settings.data.batch_size, ex.rw_batch_size = 6, 4096
        ex.predict_n_best = 1024 if variant == "n_best_max" else 100
        m.distance_fn = "L2"
    elif variant in ("no_features_big", "transh_big", "l1_big", "distmult_big", "bf16_rows_big"):
        # several chunks of tails per shard, several query chunks, ragged counts
        m.n_entity, m.entity_feature_size, m.embedding_size, m.n_shard = 20000, 0, 32, 3
        settings.data.batch_size, ex.rw_batch_size, ex.predict_n_best = 6, 4096, 20
        ex.predict_chunk_rows = 8192
        m.distance_fn = "L2"
        if variant == "transh_big":
            m.score_fn = "TransH"
        elif variant == "l1_big":      # whole chunks are scored where they lie in the table: every
            m.distance_fn = "L1"       # forward kernel family reads table rows as its tail operand
        elif variant == "distmult_big":
            m.score_fn, m.distance_fn = "DistMult", "MatMul"
        elif variant == "bf16_rows_big":
            ex.embedding_dtype = "bfloat16"
    settings.prepare()
    S = m.n_shard
    counts = np.array([m.n_entity - 1 - 7 * s for s in range(S)])
    engine = kge.Engine(settings, counts)
    features = engine.random_normal((S, m.n_entity, m.entity_feature_size), np.float16)
    engine.initialise_all(features)
    state = _oracle_state(engine.read_all())

    n = ex.predict_hr_batch_size + 5
    queries = _random_queries(engine, n)
    found = engine.predict(queries)
    assert found.shard_idx.shape == (n, ex.predict_n_best, 2) and found.score.shape == (n, ex.predict_n_best)
    assert np.all(found.shard_idx[:, :, 0] < S)
    assert np.all((found.shard_idx[:, :, 1] >= 1) & (found.shard_idx[:, :, 1] <= counts[found.shard_idx[:, :, 0]]))
    assert not np.any(np.isnan(found.score))
    np.testing.assert_equal(found.score, np.sort(found.score, axis=-1)[..., ::-1])

    want_idx, want_score = predict_reference(_oracle_cfg(settings), state, queries, counts, ex.predict_n_best)
    np.testing.assert_allclose(found.score, want_score, rtol=1e-5, atol=1e-5)
    # the same entities, up to swaps between scores closer than float32 resolves
    agree = np.all(found.shard_idx == want_idx, axis=-1)
    close = np.abs(found.score - want_score) <= 1e-5 * np.maximum(1.0, np.abs(want_score))
    assert np.all(agree | close)
    assert agree.mean() > 0.99


@pytest.mark.parametrize("chunk_rows", [None, 4096])
def test_predict_ties_go_to_the_lower_row(chunk_rows):
    """All embeddings zero: every tail scores the same, so each tail shard's n_best are its
    first rows in order, however the sweep is cut into chunks (the reference leaves ties to
    the host's argsort, src/python/poplar_kge.py:806-817; this build fixes them)."""
    import poplar_kge as kge

    settings = kge.Settings.create_demo()
    m, ex = settings.model, settings.execution
    m.n_entity, m.entity_feature_size, m.embedding_size, m.n_shard = 20000, 0, 32, 2
    m.distance_fn, m.init_scale = "L2", 0.0
    settings.data.batch_size, ex.rw_batch_size, ex.predict_n_best = 6, 4096, 100
    ex.predict_chunk_rows = chunk_rows
    settings.prepare()
    S, Hb, nb = m.n_shard, ex.predict_hr_batch_size, ex.predict_n_best
    counts = np.array([m.n_entity - 1, m.n_entity - 50])
    engine = kge.Engine(settings, counts)
    engine.initialise_all(np.zeros((S, m.n_entity, 0), np.float16))
    scores = np.full((S, S, Hb, nb), np.nan, np.float32)
    rows = np.zeros(scores.shape, np.uint32)
    engine.engine.run("predict", dict(
        predict_head=engine.random_integers(m.n_entity - 60, (S, Hb)) + 1,
        predict_relation=engine.random_integers(m.n_relation_type, (S, Hb)),
        predict_entity_count=counts.astype(np.uint32), predict_scores=scores, predict_indices=rows))
    np.testing.assert_array_equal(rows, np.broadcast_to(np.arange(1, nb + 1, dtype=np.uint32), rows.shape))
    np.testing.assert_array_equal(scores, np.full(scores.shape, m.gamma, np.float32))


def test_training_mrr_matches_brute_force():
    """The reference's MRR check (tests/python/test_poplar_kge.py:214-236): after every
    program run the validation MRR from Engine.predict equals the brute-force one."""
    import poplar_kge as kge
    import poplar_kge_dataset as kge_data
    from oracle.kge_oracle import predict_reference

    settings = kge.Settings.create_demo()
    settings.seed = 100
    settings.prepare()
    data = kge_data.RawData.load(settings)
    dataset = kge_data.Dataset.load(data, settings)
    engine = kge.Engine(settings, dataset.shard_to_count)
    engine.initialise_all(dataset.entity_features(settings.model.entity_feature_size))
    cfg, n_best = _oracle_cfg(settings), settings.execution.predict_n_best

    def brute_force(queries):
        idx, score = predict_reference(cfg, _oracle_state(engine.read_all()), queries, dataset.shard_to_count, n_best)
        return kge.Predictions(shard_idx=idx.astype(np.uint32), score=score)

    seen = []
    for _ in range(6):
        engine.train_step_loop(dataset.sample_batch())
        for part in ("valid", "train"):
            got, want = dataset.mrr(part, engine.predict), dataset.mrr(part, brute_force)
            np.testing.assert_allclose(got, want, rtol=1e-4)
            seen.append(want)
    assert max(seen) > 0.05   # the training triples are being learnt: the comparison is not 0 == 0


def test_training_script_flow():
    """The reference's training script (scripts/run_training.py:12-77) step by step, without its
    logger: settings -> data -> dataset -> engine -> initialise_all -> a torch DataLoader over
    DatasetWrapper -> train_step_loop per program run, validation MRR and predictions."""
    import poplar_kge as kge
    import poplar_kge_dataset as kge_data
    import torch

    settings = kge.Settings.create_demo()
    settings.seed = 3
    settings.prepare()
    data = kge_data.RawData.load(settings)
    dataset = kge_data.Dataset.load(data, settings)
    engine = kge.Engine(settings, dataset.shard_to_count)
    engine.initialise_all(dataset.entity_features(settings.model.entity_feature_size))
    ds = kge_data.DatasetWrapper(dataset)
    dl_iter = iter(torch.utils.data.DataLoader(ds, batch_size=None, num_workers=0,
                                               worker_init_fn=ds.worker_init_fn))
    losses = []
    for n in range(settings.logs_per_training_run):
        if n % settings.logs_per_validation == 0:
            for part in ("train", "valid"):
                assert 0.0 <= dataset.mrr(part, engine.predict) <= 1.0
        loss, lr = np.mean([engine.train_step_loop(ds.tensors_to_batch(**next(dl_iter)))
                            for _ in range(settings.program_runs_per_log)], axis=0)
        assert np.isfinite(loss) and lr > 0
        losses.append(loss)
    assert losses[-1] < losses[0]
    entity, score = dataset.predict("valid", engine.predict)
    assert entity.shape == (len(data.eval_hr_["valid"]), settings.execution.predict_n_best)
    assert score.shape == entity.shape and np.all(np.diff(score, axis=1) <= 0)
    assert dataset.mrr("train", engine.predict) > 0.05
