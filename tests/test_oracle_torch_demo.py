"""The PyTorch demo-path CPU baseline (oracle/torch_demo_step.py) against the
sequential C oracle: same seeded state and batches, loss and every updated
table at the bar the reference's own PyTorch comparison uses
(tests/python/test_poplar_kge.py:222-259: loss rtol 1e-4, state 1e-4 relative L2)."""

import numpy as np
import pytest

import kge_cases as K
from oracle.kge_oracle import Oracle, make_cfg
from oracle.torch_demo_step import TorchDemoStep


@pytest.fixture(scope="module")
def oracle32():
    return Oracle("f32")


@pytest.mark.parametrize("distance_fn", ["L1", "L2"])
@pytest.mark.parametrize("shared_table", [False, True])
def test_torch_demo_step_matches_oracle(oracle32, distance_fn, shared_table):
    c = K.cfg_dict(feature=0, dim=16, distance_fn=distance_fn, shared_table=shared_table, n_entity=200)
    rng = np.random.default_rng(11)
    st_o = K.make_state(c, rng)
    st_t = K.copy_state(st_o)
    batch = K.random_batch(c, 3, rng, pad=2)
    loss_o = oracle32.train_step_loop(make_cfg(**c), st_o, 0.01, batch)
    loss_t = TorchDemoStep(c, st_t).train_step_loop(0.01, batch)
    np.testing.assert_allclose(loss_t, loss_o, rtol=1e-4)
    assert st_t["step"] == st_o["step"]
    for k in ("entity_data", "relation_embedding", "relation_embedding/adam_m", "relation_embedding/adam_v"):
        assert K.rel_l2(st_t[k], st_o[k]) < 1e-4, k


def test_torch_demo_step_bf16_embedding_rows(oracle32):
    c = K.cfg_dict(feature=0, dim=16, distance_fn="L2", shared_table=True, n_entity=200,
                   storage="bfloat16_embedding")
    rng = np.random.default_rng(12)
    st_o = K.make_state(c, rng)
    D = c["dim"]
    import torch as T
    st_o["entity_data"][:, :D] = T.from_numpy(st_o["entity_data"][:, :D].copy()).to(T.bfloat16).to(T.float32).numpy()
    st_t = K.copy_state(st_o)
    batch = K.random_batch(c, 2, rng)
    loss_o = oracle32.train_step_loop(make_cfg(**c), st_o, 0.01, batch)
    loss_t = TorchDemoStep(c, st_t).train_step_loop(0.01, batch)
    np.testing.assert_allclose(loss_t, loss_o, rtol=1e-4)
    # embeddings are stored rounded: a last-place difference before rounding moves a value by one
    # bfloat16 step (2^-8 relative) at most
    assert K.rel_l2(st_t["entity_data"], st_o["entity_data"]) < 2e-3


def test_torch_demo_step_rejects_what_the_demo_path_lacks():
    c = K.cfg_dict(feature=0, score_fn="DistMult", distance_fn="MatMul")
    with pytest.raises(ValueError):
        TorchDemoStep(c, K.make_state(c, np.random.default_rng(0)))
