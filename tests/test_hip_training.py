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
    return make_cfg(n_shard=m.n_shard, n_entity=m.n_entity, n_relation=m.n_relation_type,
                    dim=m.embedding_size, feature=m.entity_feature_size, batch=d.batch_size,
                    a2a=d.a2a_size, score_fn=m.score_fn, distance_fn=m.distance_fn,
                    loss_fn=t.loss.type, gamma=m.gamma, beta_m=t.adam_beta_m, beta_v=t.adam_beta_v,
                    epsilon=t.adam_epsilon, weight_decay=t.weight_decay, loss_scale=t.loss_scale)


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


def test_training():
    import poplar_kge as kge
    import poplar_kge_dataset as kge_data

    settings = kge.Settings.create_demo()
    settings.seed = 100
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
    assert n_loop == 20

    loss, ref_loss = [], []
    for b in itertools.islice(itertools.cycle(batches), n_loop):
        step_loss, lr = engine.train_step_loop(b)
        loss.append(step_loss)
        ref_loss.append(float(np.sum(oracle.train_step_loop(cfg, ref, lr, vars(b)))))
    np.testing.assert_allclose(loss, ref_loss, rtol=1e-4)

    final = engine.read_all()
    assert set(np.ravel(final.pop("step"))) == {ref["step"]} == {100}
    first = _oracle_state(initial)
    for key, value in final.items():
        value = value.reshape(ref[key].shape)
        delta, ref_delta = value - first[key], ref[key] - first[key]
        assert np.any(ref_delta != 0), key
        distance = K.rel_l2(delta, ref_delta)
        assert distance <= 1e-4, f"(final - initial) of '{key}' is {distance:.2g} away from the oracle's"


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
