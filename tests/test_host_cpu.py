"""CPU-only checks: the C-ABI library loads and exports every declared symbol,
engine construction validates settings before touching a device, and the host
mirror (settings tree, learning-rate schedule) behaves as the reference's."""

import ctypes as C
import re
import types
from pathlib import Path

import numpy as np
import pytest

import hip_harness as H
import kge_cases as K

ROOT = Path(__file__).resolve().parent.parent


def test_cabi_exports_every_declared_symbol():
    header = (ROOT / "include" / "kge_hip.h").read_text()
    declared = set(re.findall(r"\b(kge_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 15
    lib = H.lib()
    for name in sorted(declared):
        assert hasattr(lib, name), name


def test_cabi_rejects_bad_op_arguments_without_a_device():
    lib = H.lib()
    assert lib.kge_l1_distance(None, None, None, -1, 2, 3, None) == 1
    assert lib.kge_buffer_read(None, None, None, C.c_int64(3), C.c_int64(6), None) == 1
    assert lib.kge_scatter_add_workspace_bytes(0, 0, 1) == 0
    assert lib.kge_scatter_add_workspace_bytes(100, 10, 8) > 0


def test_engine_settings_validation_precedes_device_attach():
    import libpoplar_kge

    s = H.engine_settings(K.cfg_dict(feature=0), 2)
    with pytest.raises(ValueError, match="Key not found 'model.n_shard'"):
        libpoplar_kge.Engine({k: v for k, v in s.items() if k != "model.n_shard"}, "")
    with pytest.raises(ValueError, match="expected \"hip\""):
        libpoplar_kge.Engine({**s, "execution.device": "ipu"}, "")
    with pytest.raises(ValueError, match="'execution.dtype' must either be"):
        libpoplar_kge.Engine({**s, "execution.dtype": "float64"}, "")
    with pytest.raises(ValueError, match="'training.loss.type' must be one of"):
        libpoplar_kge.Engine({**s, "training.loss.type": "hinge"}, "")
    with pytest.raises(ValueError, match="unknown parameter 'nope'"):
        libpoplar_kge.Engine({**s, "training.learning_rate_modifiers": {"nope": 2.0}}, "")
    with pytest.raises(ValueError, match="holds value of unexpected type"):
        libpoplar_kge.Engine({**s, "model.gamma": 2}, "")
    # additive settings that size device tables are range-checked before anything is allocated
    for bad in (0, 16, 63, 4097):
        with pytest.raises(ValueError, match=r"'execution.reduce_chunk' must be in \[64, 4096\]"):
            libpoplar_kge.Engine({**s, "execution.reduce_chunk": bad}, "")
    with pytest.raises(ValueError, match="predict_chunk_rows"):
        libpoplar_kge.Engine({**s, "execution.predict_chunk_rows": 10}, "")


def test_settings_tree():
    import poplar_kge as kge

    s = kge.Settings.create_demo()
    s.seed = 100
    s.prepare()
    assert s.n_tail == 10 and s.n_remote == 16 and s.entity_data_r_size == 30
    assert s.training.loss_scale == 6 * 2 * 5  # batch_size * n_shard * a2a_size
    assert s.program_runs_per_log == 4 and s.logs_per_training_run == 5
    assert s.logs_per_validation == 3 and s.predict_at_log == {2}
    assert isinstance(s.model.seed, int) and isinstance(s.data.dataset.seed, int)
    # the same seed spawns the same sub-seeds
    t = kge.Settings.create_demo()
    t.seed = 100
    assert t.prepare().model.seed == s.model.seed
    flat = s.flatten()
    assert flat["model.n_shard"] == 2 and flat["training.loss.type"] == "logsigmoid"
    assert flat["data.dataset.n_train"] == 50 and flat["training.learning_rate_modifiers"] == {}
    assert flat["training.embedding_regularisation.power"] == 3.0
    w = kge.Settings.create_wikikg90mv2()
    assert w.model.n_entity == 5701915 and w.model.n_relation_type == 1392
    assert w.flatten()["training.loss.correction_weight"] == 1.0
    assert kge.Settings.create_wikikg90mv2_short().data.a2a_size == 32
    # the preset's regularisers (reference :377-380)
    assert (w.training.feature_regularisation.power, w.training.feature_regularisation.weight) == (3.0, 1e-6)
    assert w.training.embedding_regularisation.weight == 0.0 and w.training.hidden_regularisation.weight == 0.0


def _schedule(decay, n):
    import poplar_kge as kge

    eng = types.SimpleNamespace(
        settings=types.SimpleNamespace(training=types.SimpleNamespace(
            learning_rate=0.1, n_step=100, learning_rate_decay=decay)),
        step=0, current_learning_rate=0.1, decay_step=float(getattr(decay, "step", 0)))
    out = []
    for _ in range(n):
        out.append(kge.Engine._next_learning_rate(eng))
        eng.step += 10
    return out


def test_learning_rate_schedules():
    import poplar_kge as kge

    np.testing.assert_allclose(_schedule(None, 3), [0.1, 0.1, 0.1])
    np.testing.assert_allclose(_schedule(kge.LinearLearningRateDecay(), 4),
                               [0.1, 0.09, 0.08, 0.07])
    np.testing.assert_allclose(_schedule(kge.ExponentialLearningRateDecay(half_life_steps=20), 3),
                               [0.1, 0.1 * 0.5**0.5, 0.05])
    # stepped: multiply at step >= 20, then the threshold grows by 1.5x (30, 45, ...)
    np.testing.assert_allclose(
        _schedule(kge.SteppedLearningRateDecay(step=20, multiplier=0.5), 6),
        [0.1, 0.1, 0.05, 0.025, 0.025, 0.0125])


def test_predictions_topk():
    # the known-answer vector of the reference's test (tests/python/test_poplar_kge.py:15-46)
    import poplar_kge as kge

    pre = kge.Predictions(
        shard_idx=np.array([[[10, 100], [20, 200], [30, 300], [40, 400]],
                            [[50, 500], [60, 600], [70, 700], [80, 800]]]),
        score=np.array([[2, 1, 3, 0], [-4, -3, -2, -1]]))
    post = pre.topk(k=3).sort()
    assert post.shard_idx.shape == (2, 3, 2) and post.score.shape == (2, 3)
    np.testing.assert_equal(post.shard_idx, [[[30, 300], [10, 100], [20, 200]],
                                             [[80, 800], [70, 700], [60, 600]]])
    np.testing.assert_equal(post.score, [[3, 2, 1], [-1, -2, -3]])
    multi = kge.Predictions(pre.shard_idx[:, np.newaxis], pre.score[:, np.newaxis]).topk(k=3).sort()
    assert multi.shard_idx.shape == (2, 1, 3, 2) and multi.score.shape == (2, 1, 3)
    np.testing.assert_equal(multi.shard_idx[:, 0], post.shard_idx)
    np.testing.assert_equal(multi.score[:, 0], post.score)


def test_bench_reads_traffic_of_the_most_launched_kernel_variant():
    """bench.py takes `roofline.traffic` from the committed rocprofv3 summaries: every step kernel
    of a profiled workload has a figure, and where two variants of a kernel ran (the sparse update
    with and without hot rows inside) the one launched more often is taken."""
    import re
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    sys.path.insert(0, str(root))
    from bench import measured_traffic

    for workload in ("c2", "c3l2", "c3", "c5"):
        traffic, source = measured_traffic(workload)
        assert source == f"profiles/{workload}_step_hbm_traffic.md"
        for kernel in ("gather_operands", "score_fwd", "score_bwd", "adam_entity"):
            assert traffic[kernel] > 1e6, (workload, kernel)
    rows = {}
    for line in (root / "profiles" / "c2_step_hbm_traffic.md").read_text().splitlines():
        m = re.match(r"\| `(kge::k_adam_rows[^`]*)` \|[^|]*\|[^|]*\| ([0-9.]+) \| ([0-9.]+) \| (\d+) \|", line)
        if m:
            rows[m.group(1)] = ((float(m.group(2)) + float(m.group(3))) * 1e6, int(m.group(4)))
    assert len(rows) == 2
    most = max(rows.values(), key=lambda r: r[1])
    assert measured_traffic("c2")[0]["adam_entity"] == pytest.approx(most[0])
    assert measured_traffic("no_such_workload") == (None, None)
