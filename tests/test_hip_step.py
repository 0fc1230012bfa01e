"""GPU parity of the whole training step through the reference's engine
interface (libpoplar_kge.Engine -> C-ABI -> HIP kernels) against the CPU oracle
on the same seeded inputs.  Tolerances: loss and updated rows 1e-5 relative
(float32), state deltas 1e-4 relative L2 as the reference's own test
(tests/python/test_poplar_kge.py:222-259) -- in practice far tighter."""

import numpy as np
import pytest

import hip_harness as H
import kge_cases as K
from oracle.kge_oracle import make_cfg

pytestmark = pytest.mark.gpu

CASES = {
    "demo_l1_logsigmoid": dict(),
    "l1_nofeat": dict(feature=0),
    "l2_logsigmoid": dict(distance_fn="L2", feature=0, gamma=4.0),
    "l2_feat": dict(distance_fn="L2", gamma=4.0),
    "l2_softmax": dict(distance_fn="L2", loss_fn="softmax", softmax_correction_weight=1.0, feature=0),
    "distmult_softmax_feat": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax",
                                  softmax_correction_weight=1.0, feature=4),
    "distmult_logsigmoid": dict(score_fn="DistMult", distance_fn="MatMul", feature=0),
    "transe_matmul": dict(distance_fn="MatMul", feature=0),
    "l1_adversarial": dict(negative_adversarial_scale=1.5, feature=0),
    "l2_weight_decay": dict(distance_fn="L2", weight_decay=0.01, feature=0),
    "shared_l2": dict(distance_fn="L2", shared_table=True, n_shard=4, batch=8, a2a=4, feature=0,
                      n_entity=60, gamma=3.0),
    "odd_dim": dict(dim=10, feature=6, n_entity=41, batch=5, a2a=3, distance_fn="L2"),
    "mid_l2": dict(distance_fn="L2", n_shard=4, batch=96, a2a=40, dim=128, feature=0,
                   n_entity=3000, n_relation=40, gamma=6.0),
    "mid_l1": dict(distance_fn="L1", n_shard=2, batch=70, a2a=45, dim=64, feature=0,
                   n_entity=2000, n_relation=10, gamma=6.0),
    # tile-aligned shapes (positives % 128, tails % 128, dim % 64): the matrix-core fast path
    "aligned_l2": dict(distance_fn="L2", n_shard=2, batch=128, a2a=64, dim=64, feature=0,
                       n_entity=3000, n_relation=8, gamma=6.0),
    # L1 on whole 64 x 64 tiles and 32-column slabs: the vector forward kernel's form with the next
    # slab's loads in flight
    "aligned_l1": dict(distance_fn="L1", n_shard=2, batch=128, a2a=64, dim=64, feature=0,
                       n_entity=3000, n_relation=8, gamma=6.0),
    "aligned_l2_wide": dict(distance_fn="L2", n_shard=4, batch=256, a2a=64, dim=128, feature=0,
                            n_entity=5000, n_relation=8, gamma=6.0, shared_table=True),
    "aligned_distmult": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax",
                             softmax_correction_weight=1.0, n_shard=2, batch=128, a2a=64, dim=64,
                             feature=0, n_entity=3000, n_relation=8),
    "aligned_l2_softmax": dict(distance_fn="L2", loss_fn="softmax", softmax_correction_weight=1.0,
                               n_shard=2, batch=128, a2a=64, dim=64, feature=0, n_entity=3000,
                               n_relation=8, gamma=6.0),
    # L1 with tails split over 16 waves of 8 / 16 / 32: the one-pass backward for both sides
    "paired_l1_t128": dict(distance_fn="L1", n_shard=32, batch=16, a2a=4, dim=256, feature=0,
                           n_entity=4000, n_relation=8, gamma=6.0, shared_table=True),
    "paired_l1_t256": dict(distance_fn="L1", n_shard=32, batch=32, a2a=8, dim=256, feature=0,
                           n_entity=4000, n_relation=8, gamma=6.0, shared_table=True),
    "paired_l1_t512": dict(distance_fn="L1", n_shard=32, batch=16, a2a=16, dim=256, feature=0,
                           n_entity=4000, n_relation=8, gamma=6.0, shared_table=True),
    "bf16_embedding_l2": dict(distance_fn="L2", n_shard=2, batch=128, a2a=64, dim=64, feature=0,
                              n_entity=3000, n_relation=8, gamma=6.0, storage="bfloat16_embedding"),
    # RotatE (src/poplar_kge.cpp:516-537): rotation by the relation's D / 2 phases, sine / cosine
    # and the phases' gradient in float16
    "rotate_l1": dict(score_fn="RotatE", distance_fn="L1", feature=0),
    "rotate_l2_feat": dict(score_fn="RotatE", distance_fn="L2", gamma=4.0),
    "rotate_softmax_odd_half": dict(score_fn="RotatE", distance_fn="L1", loss_fn="softmax",
                                    softmax_correction_weight=1.0, feature=0, dim=10, n_entity=41, batch=5,
                                    a2a=3),
    "aligned_rotate_l2": dict(score_fn="RotatE", distance_fn="L2", n_shard=2, batch=128, a2a=64, dim=64,
                              feature=0, n_entity=3000, n_relation=8, gamma=6.0),
    # norm regularisers (src/poplar_kge.cpp:430-437, 463-465): the WikiKG preset's feature
    # regulariser, all three with different powers, and without features (hidden = embedding)
    "feature_regularisation_p3": dict(feature_regularisation=(3.0, 1e-2), loss_fn="softmax",
                                      softmax_correction_weight=1.0),
    "all_regularisers_l2": dict(embedding_regularisation=(2.0, 3e-2), feature_regularisation=(3.0, 2e-2),
                                hidden_regularisation=(4.0, 1e-2), distance_fn="L2"),
    "regularisers_nofeat": dict(embedding_regularisation=(3.0, 5e-2), feature=0,
                                hidden_regularisation=(2.0, 1e-2)),
    "regularisers_distmult_aligned": dict(score_fn="DistMult", distance_fn="MatMul", n_shard=2, batch=128,
                                          a2a=64, dim=64, feature=8, n_entity=3000, n_relation=8,
                                          feature_regularisation=(3.0, 1e-3),
                                          embedding_regularisation=(3.0, 1e-3)),
    # ComplEx (src/poplar_kge.cpp:501-514): complex product of head and relation on the row's
    # halves, scored by the distance function's value itself
    "complex_matmul_softmax": dict(score_fn="ComplEx", distance_fn="MatMul", loss_fn="softmax",
                                   softmax_correction_weight=1.0, feature=0),
    "complex_matmul_feat": dict(score_fn="ComplEx", distance_fn="MatMul", feature=4),
    "complex_l2": dict(score_fn="ComplEx", distance_fn="L2", feature=0),
    "complex_l1": dict(score_fn="ComplEx", distance_fn="L1", feature=0),
    "complex_odd_half": dict(score_fn="ComplEx", distance_fn="MatMul", dim=10, feature=0, n_entity=41,
                             batch=5, a2a=3),
    "aligned_complex": dict(score_fn="ComplEx", distance_fn="MatMul", loss_fn="softmax",
                            softmax_correction_weight=1.0, n_shard=2, batch=128, a2a=64, dim=64,
                            feature=0, n_entity=3000, n_relation=8),
    # TransH (src/poplar_kge.cpp:539-565): unit hyperplane normals from relation_normal, heads
    # and tails projected, L1 distance whatever distance_fn says
    "transh": dict(score_fn="TransH", feature=0),
    "transh_feat_softmax": dict(score_fn="TransH", distance_fn="L2", loss_fn="softmax",
                                softmax_correction_weight=1.0),
    "transh_shared": dict(score_fn="TransH", shared_table=True, n_shard=4, batch=8, a2a=4, feature=0,
                          n_entity=60, gamma=3.0),
    "transh_odd_adversarial": dict(score_fn="TransH", dim=10, feature=6, n_entity=41, batch=5, a2a=3,
                                   negative_adversarial_scale=1.5),
    "transh_aligned": dict(score_fn="TransH", n_shard=2, batch=128, a2a=64, dim=64, feature=0,
                           n_entity=3000, n_relation=8, gamma=6.0),
    "transh_bf16_embedding": dict(score_fn="TransH", n_shard=2, batch=128, a2a=64, dim=64, feature=0,
                                  n_entity=3000, n_relation=8, gamma=6.0, storage="bfloat16_embedding"),
    "transh_mid": dict(score_fn="TransH", n_shard=2, batch=70, a2a=45, dim=64, feature=0,
                       n_entity=2000, n_relation=10, gamma=6.0),
    # feature MLP (src/poplar_kge.cpp:453-458): hidden = value + relu([value | feature . W] . Up) . Down
    "feature_mlp": dict(feature_mlp_size=10),
    "feature_mlp_l2_softmax_reg": dict(feature_mlp_size=6, distance_fn="L2", loss_fn="softmax",
                                       softmax_correction_weight=1.0, feature_regularisation=(3.0, 2e-2),
                                       hidden_regularisation=(2.0, 1e-2)),
    "feature_mlp_shared_distmult": dict(feature_mlp_size=8, score_fn="DistMult", distance_fn="MatMul",
                                        shared_table=True, n_shard=4, batch=8, a2a=4, feature=4, n_entity=60),
    "feature_mlp_odd_dim": dict(feature_mlp_size=9, dim=10, feature=6, n_entity=41, batch=5, a2a=3,
                                distance_fn="L2", n_shard=1),
    "feature_mlp_aligned_transh": dict(feature_mlp_size=96, score_fn="TransH", n_shard=2, batch=128, a2a=64,
                                       dim=64, feature=32, n_entity=3000, n_relation=8, gamma=6.0),
    # feature dropout (src/poplar_kge.cpp:459-461): a row's head use and tail use are dropped apart
    "feature_dropout": dict(feature_dropout=0.3, dropout_seed=7),
    "feature_dropout_mlp_l2": dict(feature_dropout=0.5, dropout_seed=3, feature_mlp_size=6, distance_fn="L2",
                                   loss_fn="softmax", softmax_correction_weight=1.0),
    "feature_dropout_shared_distmult": dict(feature_dropout=0.2, dropout_seed=11, score_fn="DistMult",
                                            distance_fn="MatMul", shared_table=True, n_shard=4, batch=8, a2a=4,
                                            feature=4, n_entity=60),
    "feature_dropout_aligned_l2": dict(feature_dropout=0.4, dropout_seed=5, distance_fn="L2", n_shard=2,
                                       batch=128, a2a=64, dim=64, feature=32, n_entity=3000, n_relation=8,
                                       gamma=6.0),
    # separate feature networks for the head and the tail use (src/poplar_kge.cpp:268-273)
    "separate_networks": dict(share_feature_networks=False),
    "separate_networks_mlp_dropout_l2": dict(share_feature_networks=False, feature_mlp_size=6, feature_dropout=0.3,
                                             dropout_seed=5, distance_fn="L2", loss_fn="softmax",
                                             softmax_correction_weight=1.0),
    "separate_networks_shared_distmult": dict(share_feature_networks=False, score_fn="DistMult", distance_fn="MatMul",
                                              shared_table=True, n_shard=4, batch=8, a2a=4, feature=4, n_entity=60),
    "separate_networks_mlp_aligned": dict(share_feature_networks=False, feature_mlp_size=48, distance_fn="L2",
                                          n_shard=2, batch=128, a2a=64, dim=64, feature=32, n_entity=3000,
                                          n_relation=8, gamma=6.0),
    # regularisers where the two entityHidden calls differ: each call's tensors once
    "regularisers_dropout": dict(feature_dropout=0.3, dropout_seed=9, embedding_regularisation=(2.0, 3e-2),
                                 feature_regularisation=(3.0, 2e-2), hidden_regularisation=(4.0, 1e-2)),
    "regularisers_separate_mlp": dict(share_feature_networks=False, feature_mlp_size=6,
                                      feature_regularisation=(3.0, 2e-2), hidden_regularisation=(2.0, 1e-2),
                                      distance_fn="L2"),
    "regularisers_separate_dropout_softmax": dict(share_feature_networks=False, feature_dropout=0.25, dropout_seed=2,
                                                  embedding_regularisation=(3.0, 1e-2),
                                                  feature_regularisation=(2.0, 3e-2), loss_fn="softmax",
                                                  softmax_correction_weight=1.0),
    # 8192 contributions and more: the gather's two-rows-per-wave kernel, multiply mode and rows
    # through the feature path's index; an odd row count
    "distmult_many_rows_feat": dict(score_fn="DistMult", distance_fn="MatMul", n_shard=32, batch=128, a2a=4, dim=32,
                                    feature=8, n_entity=3000, n_relation=8, shared_table=True),
    "l1_many_rows_odd": dict(distance_fn="L1", n_shard=31, batch=129, a2a=5, dim=20, feature=0, n_entity=3000,
                             n_relation=8, shared_table=True, gamma=4.0),
    "aligned_complex_l2_shared": dict(score_fn="ComplEx", distance_fn="L2", n_shard=4, batch=128, a2a=32,
                                      dim=128, feature=0, n_entity=2000, n_relation=8, shared_table=True),
}


# bfloat16 scoring (DistMult): operands rounded to bfloat16, float32 accumulation.  The oracle
# rounds the same operands; the coefficient matrix is a bfloat16 operand of the two backward
# products on the device only (2^-9 relative per element), hence the bar of 2e-2 on the update.
BF16_SCORING_CASES = {
    "aligned": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax", softmax_correction_weight=1.0,
                    n_shard=2, batch=128, a2a=64, dim=128, feature=0, n_entity=3000, n_relation=8,
                    scoring_bf16=True),
    "aligned_logsigmoid_shared": dict(score_fn="DistMult", distance_fn="MatMul", n_shard=4, batch=128, a2a=32,
                                      dim=128, feature=0, n_entity=2000, n_relation=8, shared_table=True,
                                      scoring_bf16=True),
    "aligned_features": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax",
                             softmax_correction_weight=1.0, n_shard=1, batch=256, a2a=128, dim=128,
                             feature=64, n_entity=3000, n_relation=8, shared_table=True, scoring_bf16=True),
    "ragged_fallback": dict(score_fn="DistMult", distance_fn="MatMul", loss_fn="softmax",
                            softmax_correction_weight=1.0, n_shard=2, batch=40, a2a=30, dim=64, feature=0,
                            n_entity=1000, n_relation=8, scoring_bf16=True),
}


@pytest.mark.parametrize("name", list(BF16_SCORING_CASES))
def test_step_bf16_scoring(oracle64, name):
    import libpoplar_kge

    c = K.cfg_dict(**BF16_SCORING_CASES[name])
    rng = np.random.default_rng(21)
    st0 = K.make_state(c, rng)
    batch = K.random_batch(c, 2, rng)
    lr = np.full(c["n_shard"], 0.05, np.float32)
    engine = libpoplar_kge.Engine(H.engine_settings(c, 2), "")
    H.load_state(engine, c, st0)
    st_o = K.copy_state(st0)
    loss_o = oracle64.train_step_loop(make_cfg(**c), st_o, lr, batch)
    loss_h = H.train(engine, c, lr, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=1e-4)   # forward: same rounded operands
    st_h = H.read_state(engine, c)
    for k in st0:
        if k == "step":
            continue
        assert K.rel_l2(st_h[k] - st0[k], st_o[k] - st0[k]) < 2e-2, k
    # and the rounding is really what is compared: without it the oracle's update differs
    # from the device's by more than the device differs from the rounding oracle
    c32 = dict(c, scoring_bf16=False)
    st_f = K.copy_state(st0)
    oracle64.train_step_loop(make_cfg(**c32), st_f, lr, batch)
    k = "relation_embedding"
    assert K.rel_l2(st_f[k] - st0[k], st_o[k] - st0[k]) > 1e-4


@pytest.mark.parametrize("name", ["demo", "l2_aligned", "transh_mlp_dropout"])
def test_step_float16_table(oracle64, name):
    """execution.dtype = "float16" (src/poplar_kge.cpp:237-246): embedding, both
    moments and features stored as float16, read / write streams in float16.  The
    oracle rounds on write-back as the reference's cast does (:412-417); a float32
    difference of 1e-7 may round an element to the other float16 neighbour
    (2^-11 relative), hence the bars (the reference's own: loss 2e-3, update 1e-1)."""
    import libpoplar_kge

    kw = dict(storage="float16", feature=6) if name == "demo" else dict(
        storage="float16", distance_fn="L2", n_shard=2, batch=128, a2a=64, dim=64, feature=0,
        n_entity=3000, n_relation=8, gamma=6.0)
    if name == "transh_mlp_dropout":  # the later model options on float16 rows
        kw = dict(storage="float16", feature=6, score_fn="TransH", feature_mlp_size=8, feature_dropout=0.25,
                  dropout_seed=4, share_feature_networks=False)
    c = K.cfg_dict(**kw)
    rng = np.random.default_rng(13)
    st0 = K.make_state(c, rng)
    st0["entity_data"] = oracle64.round(st0["entity_data"], "float16")   # representable start
    batch = K.random_batch(c, 3, rng)
    engine = libpoplar_kge.Engine(H.engine_settings(c, 3), "")
    H.load_state(engine, c, st0)
    np.testing.assert_array_equal(H.read_state(engine, c)["entity_data"], st0["entity_data"])
    st_o = K.copy_state(st0)
    lr = np.full(c["n_shard"], 0.02, np.float32)
    loss_o = oracle64.train_step_loop(make_cfg(**c), st_o, lr, batch)
    loss_h = H.train(engine, c, lr, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=2e-3)
    st_h = H.read_state(engine, c)
    for k in st0:
        if k == "step":
            continue
        assert K.rel_l2(st_h[k] - st0[k], st_o[k] - st0[k]) < 2e-2, k
    assert np.mean(st_h["entity_data"] != st_o["entity_data"]) < 1e-2


def run_case(oracle, kw, n_step=3, batch_fn=K.random_batch, lr=(0.1, 0.07), n_loop=1, warm=True,
             **settings):
    import libpoplar_kge

    c = K.cfg_dict(**kw)
    rng = np.random.default_rng(11)
    st0 = K.make_state(c, rng, warm=warm)
    bf16 = c["storage"] == "bfloat16_embedding"
    if bf16:  # the table stores bfloat16 embeddings: start from representable values
        D = c["dim"]
        st0["entity_data"][:, :D] = oracle.round(st0["entity_data"][:, :D], "bfloat16_embedding")
    lr = np.resize(np.asarray(lr, np.float32), c["n_shard"])
    if c["shared_table"]:
        lr[:] = lr[0]
    engine = libpoplar_kge.Engine(H.engine_settings(c, n_step, **settings), "")
    H.load_state(engine, c, st0)
    # the state round-trips bit-exactly through write_entity_raw / read_entity
    rt = H.read_state(engine, c)
    for k in st0:
        np.testing.assert_array_equal(rt[k], st0[k], err_msg=k)
    cfg = make_cfg(**c)
    st_o = K.copy_state(st0)
    for _ in range(n_loop):
        batch = batch_fn(c, n_step, rng)
        loss_o = oracle.train_step_loop(cfg, st_o, lr, batch)
        loss_h = H.train(engine, c, lr, batch)
        np.testing.assert_allclose(loss_h, loss_o, rtol=1e-5)
    st_h = H.read_state(engine, c)
    assert st_h["step"] == st_o["step"]
    for k in st0:
        if k == "step":
            continue
        d_h, d_o = st_h[k] - st0[k], st_o[k] - st0[k]
        # updated rows: 1e-5 relative (measured ~1e-6 at lr 0.1); the update itself: the
        # reference's own 1e-4 bar on (final - initial), whose float32 storage
        # rounding alone is ~1e-5 of a small delta
        if bf16 and k == "entity_data":
            # bfloat16 rows: 2e-2 relative; a float32 difference of one part in 1e7 may
            # round an element to the other bfloat16 neighbour (2^-8 relative), so the
            # moments (float32) are held to the tight bar and the embedding to bf16's
            D = c["dim"]
            assert K.rel_l2(st_h[k][:, D:], st_o[k][:, D:]) < 1e-5
            assert K.rel_l2(st_h[k][:, :D], st_o[k][:, :D]) < 2e-3
            mism = np.mean(st_h[k][:, :D] != st_o[k][:, :D])
            assert mism < 1e-3, mism  # all but a handful of elements are bit-identical
            continue
        if c["score_fn"] == "RotatE" and k.startswith("relation_embedding"):
            # the phases' gradient is formed in float16 (as the reference forms it): where the
            # float32 value it is rounded from differs in its last bits between two implementations,
            # an element lands on the neighbouring float16 (2^-11 relative)
            assert K.rel_l2(st_h[k], st_o[k]) < 1e-3, (k, K.rel_l2(st_h[k], st_o[k]))
            assert K.rel_l2(d_h, d_o) < 5e-3, (k, K.rel_l2(d_h, d_o))
            continue
        assert K.rel_l2(st_h[k], st_o[k]) < 1e-5, (k, K.rel_l2(st_h[k], st_o[k]))
        assert K.rel_l2(d_h, d_o) < 1e-4, (k, K.rel_l2(d_h, d_o))
    return c, st0, st_h, engine


@pytest.mark.parametrize("name", list(CASES))
def test_step_vs_oracle(oracle64, name):
    run_case(oracle64, CASES[name])


@pytest.mark.parametrize("name", ["l2_logsigmoid", "l2_softmax", "distmult_softmax_feat", "mid_l2",
                                  "transe_matmul", "shared_l2", "paired_l1_t256", "aligned_l2", "aligned_l1"])
def test_step_vs_oracle_valu_scoring(oracle64, name):
    # the same cases on the VALU scoring kernels (default: matrix cores)
    run_case(oracle64, CASES[name], **{"execution.scoring": "valu"})


@pytest.mark.parametrize("scoring", ["mfma", "mfma_bf16x3"])
@pytest.mark.parametrize("name", ["aligned_l2", "aligned_l2_wide", "aligned_distmult", "aligned_l2_softmax",
                                  "bf16_embedding_l2", "l2_feat", "mid_l2"])
def test_step_vs_oracle_matrix_scoring(oracle64, name, scoring):
    # the two matrix-core forms of the float32 products, named explicitly: float32 instructions
    # ("mfma"), and six bfloat16 instructions on three-piece operands in the forward kernel
    # ("mfma_bf16x3", the default; ragged shapes fall back to the float32 instruction): same bars
    run_case(oracle64, CASES[name], **{"execution.scoring": scoring})


def test_step_l1_equal_and_signed_zero_entries(oracle64):
    # signum(0) = 0 on the one-pass L1 backward: identical rows under a zero
    # relation, zero entries of either sign, and rows that differ in a few columns
    import libpoplar_kge

    c = K.cfg_dict(distance_fn="L1", n_shard=32, batch=16, a2a=4, dim=256, feature=0, n_entity=300,
                   n_relation=4, gamma=6.0, shared_table=True)
    rng = np.random.default_rng(9)
    st0 = K.make_state(c, rng)
    D = c["dim"]
    st0["relation_embedding"][:2] = 0.0
    st0["relation_embedding"][1, ::2] = -0.0
    rows = st0["entity_data"]
    for r in range(2, rows.shape[0], 2):       # half of the rows are near-copies of row 1
        rows[r, :D] = rows[1, :D]
        rows[r, rng.integers(0, D, 5)] += 0.01
    rows[:, 3] = 0.0
    rows[::3, 3] = -0.0
    rows[:, 7] = np.where(rng.random(rows.shape[0]) < 0.5, 0.0, -0.0)
    batch = K.random_batch(c, 2, rng)
    engine = libpoplar_kge.Engine(H.engine_settings(c, 2), "")
    H.load_state(engine, c, st0)
    st_o = K.copy_state(st0)
    loss_o = oracle64.train_step_loop(make_cfg(**c), st_o, 0.05, batch)
    loss_h = H.train(engine, c, 0.05, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=1e-5)
    st_h = H.read_state(engine, c)
    for k in ("entity_data", "relation_embedding"):
        assert K.rel_l2(st_h[k] - st0[k], st_o[k] - st0[k]) < 1e-4, k


EDGE_CASES = {
    # the smallest shapes the formulas allow (T >= 2: the negative weight divides by T - 1)
    "one_shard_one_positive": dict(n_shard=1, batch=1, a2a=2, dim=4, feature=0, n_entity=5, n_relation=1),
    "one_column": dict(n_shard=2, batch=3, a2a=2, dim=1, feature=0, n_entity=9, n_relation=2),
    "one_column_l2_features": dict(n_shard=2, batch=3, a2a=2, dim=1, feature=2, n_entity=9, n_relation=2,
                                   distance_fn="L2"),
    "single_relation_distmult": dict(score_fn="DistMult", distance_fn="MatMul", n_shard=1, batch=4, a2a=3,
                                     dim=12, feature=0, n_entity=30, n_relation=1, loss_fn="softmax",
                                     softmax_correction_weight=0.5),
    "wide_rows": dict(n_shard=2, batch=4, a2a=3, dim=1027, feature=0, n_entity=20, n_relation=4,
                      distance_fn="L2"),
    "many_shards": dict(n_shard=16, batch=2, a2a=1, dim=8, feature=0, n_entity=40, n_relation=16),
}


@pytest.mark.parametrize("name", list(EDGE_CASES))
def test_step_edge_shapes(oracle64, name):
    run_case(oracle64, EDGE_CASES[name], n_step=2)


def test_step_all_padding(oracle64):
    # a batch that gathers only the padding row: every slot is row 0, which is updated once per
    # shard with the sum of all its (non-zero) gradients, as any other row would be
    import libpoplar_kge

    c = K.cfg_dict(feature=0, n_shard=2, batch=4, a2a=3, dim=8, n_entity=20, n_relation=2)
    rng = np.random.default_rng(17)
    st0 = K.make_state(c, rng)
    batch = K.random_batch(c, 2, rng)
    batch["remote"][...] = 0
    engine = libpoplar_kge.Engine(H.engine_settings(c, 2), "")
    H.load_state(engine, c, st0)
    st_o = K.copy_state(st0)
    loss_o = oracle64.train_step_loop(make_cfg(**c), st_o, 0.05, batch)
    loss_h = H.train(engine, c, 0.05, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=1e-5)
    st_h = H.read_state(engine, c)
    ne = c["n_entity"]
    for s in range(c["n_shard"]):   # only row 0 of each shard moved
        np.testing.assert_array_equal(st_h["entity_data"][s * ne + 1:(s + 1) * ne],
                                      st0["entity_data"][s * ne + 1:(s + 1) * ne])
    assert K.rel_l2(st_h["entity_data"], st_o["entity_data"]) < 1e-5


def test_step_near_duplicate_rows(oracle64):
    # head + relation almost equal to some tails: the L2 forward must not cancel
    import libpoplar_kge

    c = K.cfg_dict(distance_fn="L2", feature=0, gamma=1.0, n_shard=2, batch=40, a2a=30, dim=64,
                   n_entity=400, n_relation=4)
    rng = np.random.default_rng(3)
    st0 = K.make_state(c, rng)
    D = c["dim"]
    st0["relation_embedding"] *= 1e-3
    base = st0["entity_data"][1, :D].copy()
    for r in range(2, st0["entity_data"].shape[0], 3):  # a third of the rows cluster tightly
        st0["entity_data"][r, :D] = base * (1 + 1e-3 * rng.normal(size=D))
    st0["entity_data"][5, :D] = st0["entity_data"][8, :D]  # and two are identical
    batch = K.random_batch(c, 2, rng)
    engine = libpoplar_kge.Engine(H.engine_settings(c, 2), "")
    H.load_state(engine, c, st0)
    st_o = K.copy_state(st0)
    loss_o = oracle64.train_step_loop(make_cfg(**c), st_o, 0.05, batch)
    loss_h = H.train(engine, c, 0.05, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=1e-5)
    st_h = H.read_state(engine, c)
    for k in ("entity_data", "relation_embedding"):
        assert K.rel_l2(st_h[k] - st0[k], st_o[k] - st0[k]) < 1e-4, k


@pytest.mark.parametrize("scoring", ["mfma", "mfma_bf16x3", "valu"])
def test_step_near_duplicate_rows_aligned(oracle64, scoring):
    # the same hazard at tile-aligned shapes: the fast path flags the 32x32 score
    # sub-blocks that hold near-identical pairs and the backward treats them directly
    import libpoplar_kge

    c = K.cfg_dict(distance_fn="L2", feature=0, gamma=1.0, n_shard=2, batch=128, a2a=64, dim=64,
                   n_entity=600, n_relation=4)
    rng = np.random.default_rng(4)
    st0 = K.make_state(c, rng)
    D = c["dim"]
    st0["relation_embedding"] *= 1e-4
    base = st0["entity_data"][1, :D].copy()
    for r in range(2, st0["entity_data"].shape[0], 5):  # a fifth of the rows cluster tightly
        st0["entity_data"][r, :D] = base * (1 + 3e-4 * rng.normal(size=D))
    st0["entity_data"][7, :D] = st0["entity_data"][12, :D]
    batch = K.random_batch(c, 2, rng)
    engine = libpoplar_kge.Engine(H.engine_settings(c, 2, **{"execution.scoring": scoring}), "")
    H.load_state(engine, c, st0)
    st_o = K.copy_state(st0)
    loss_o = oracle64.train_step_loop(make_cfg(**c), st_o, 0.05, batch)
    loss_h = H.train(engine, c, 0.05, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=1e-5)
    st_h = H.read_state(engine, c)
    for k in ("entity_data", "relation_embedding"):
        assert K.rel_l2(st_h[k] - st0[k], st_o[k] - st0[k]) < 1e-4, k


def test_step_padding_rows(oracle64):
    # zero-padded `remote`: row 0 gathered several times, updated once with g = 0
    run_case(oracle64, dict(feature=0), batch_fn=lambda c, n, r: K.random_batch(c, n, r, pad=4))


def test_step_regularisers_with_padding_rows(oracle64):
    # the padding row (all zeros, gathered by several slots) has norm 0 and, by the reference's
    # guarded pow backward, zero gradient: no NaN reaches the row or the projection
    run_case(oracle64, dict(feature_regularisation=(3.0, 1e-2), hidden_regularisation=(3.0, 1e-2)),
             batch_fn=lambda c, n, r: K.random_batch(c, n, r, pad=4))


def test_regularisers_need_private_tables():
    import libpoplar_kge

    c = K.cfg_dict(feature=0, shared_table=True, n_shard=2, embedding_regularisation=(3.0, 1e-2))
    with pytest.raises(ValueError, match="private shard tables"):
        libpoplar_kge.Engine(H.engine_settings(c, 2), "")


def test_step_raw_zipf_duplicates(oracle64):
    # raw ids, identity slots, one shared table: the device does all the de-duplication
    run_case(oracle64, dict(distance_fn="L2", shared_table=True, n_shard=8, batch=64, a2a=8,
                            dim=64, feature=0, n_entity=500, n_relation=20, gamma=5.0),
             batch_fn=K.raw_batch, n_loop=2)


READBACK = {"execution.plan_readback_steps": 1}


@pytest.mark.parametrize("name", ["l2_logsigmoid", "shared_l2", "paired_l1_t256", "transh_shared", "bf16_embedding_l2",
                                  "l2_feat", "mid_l1", "feature_mlp", "distmult_logsigmoid"])
def test_step_vs_oracle_plan_readback(oracle64, name):
    # the plan's counts read back after the plan phase (what calls of eight steps and more do):
    # launches sized to the step's distinct rows and chunks, and, where the contributions are used
    # as stored, the rows with chunks summed inside the update's launch
    run_case(oracle64, CASES[name], **READBACK)


@pytest.mark.parametrize("shape", [dict(n_shard=8, batch=64, a2a=8, n_entity=500), dict(n_shard=16, batch=128, a2a=8, n_entity=40),
                                   dict(n_shard=4, batch=256, a2a=64, n_entity=3, dim=40)])
def test_step_raw_zipf_duplicates_plan_readback(oracle64, shape):
    # hot rows of a few dozen up to 2 000 contributions summed by the update's own workgroups
    # (n_entity = 3: two real rows share every contribution)
    kw = dict(distance_fn="L2", shared_table=True, dim=64, feature=0, n_relation=20, gamma=5.0)
    kw.update(shape)
    run_case(oracle64, kw, batch_fn=K.raw_batch, n_loop=2, **READBACK)


def test_step_hottest_row_above_the_in_launch_limit(oracle64):
    # 8 192 contributions for two rows, about 5 600 of them for the first: past the limit, the
    # two-level reduction runs as without the read-back
    kw = dict(distance_fn="L2", shared_table=True, n_shard=16, batch=256, a2a=16, n_entity=3, dim=32, feature=0,
              n_relation=4, gamma=5.0)
    run_case(oracle64, kw, n_step=2, batch_fn=K.raw_batch, **READBACK)


def test_step_cold_start(oracle64):
    # zero moments and step 0: the first Adam step is sign-like and the most sensitive
    run_case(oracle64, dict(distance_fn="L2", feature=0, gamma=4.0), warm=False)


def test_step_deterministic():
    import libpoplar_kge

    c = K.cfg_dict(distance_fn="L2", shared_table=True, n_shard=8, batch=128, a2a=16, dim=64,
                   feature=0, n_entity=300, n_relation=20, gamma=5.0)
    rng = np.random.default_rng(5)
    st0 = K.make_state(c, rng)
    batch = K.raw_batch(c, 2, rng)
    for extra in ({}, READBACK):  # the two-level reduction; hot rows inside the update's launch
        outs = []
        for _ in range(2):
            engine = libpoplar_kge.Engine(H.engine_settings(c, 2, **extra), "")
            H.load_state(engine, c, st0)
            loss = H.train(engine, c, 0.05, batch)
            outs.append((loss, H.read_state(engine, c)))
        np.testing.assert_array_equal(outs[0][0], outs[1][0])
        for k in ("entity_data", "relation_embedding"):
            np.testing.assert_array_equal(outs[0][1][k], outs[1][1][k])


def test_engine_errors():
    import libpoplar_kge

    c = K.cfg_dict(feature=0)
    s = H.engine_settings(c, 2)
    with pytest.raises(ValueError, match="Key not found 'model.n_shard'"):
        libpoplar_kge.Engine({k: v for k, v in s.items() if k != "model.n_shard"}, "")
    with pytest.raises(ValueError, match="score_fn"):
        libpoplar_kge.Engine({**s, "model.score_fn": "Nope"}, "")
    with pytest.raises(ValueError, match="unexpected type"):
        libpoplar_kge.Engine({**s, "model.gamma": "two"}, "")
    with pytest.raises(ValueError, match="not divisible by n_shard"):
        libpoplar_kge.Engine({**s, "model.n_relation_type": 13}, "")
    with pytest.raises(ValueError, match="predict_chunk_rows"):
        libpoplar_kge.Engine({**s, "execution.predict_chunk_rows": 10}, "")
    engine = libpoplar_kge.Engine(s, "")
    with pytest.raises(ValueError, match="Unknown command"):
        engine.run("fly", {})
    rng = np.random.default_rng(0)
    batch = K.random_batch(c, 2, rng)
    lr, loss = np.full(2, 0.1, np.float32), np.zeros(2, np.float32)
    with pytest.raises(ValueError, match="Key not found 'tail'"):
        engine.run("train_step_loop", dict(learning_rate=lr, loss=loss,
                                           **{k: v for k, v in batch.items() if k != "tail"}))
    with pytest.raises(ValueError, match="expected array of shape"):
        engine.run("train_step_loop", dict(learning_rate=lr, loss=loss,
                                           **{**batch, "head": batch["head"][:, :1].copy()}))
    with pytest.raises(ValueError, match="expected array of type"):
        engine.run("train_step_loop", dict(learning_rate=lr, loss=loss,
                                           **{**batch, "head": batch["head"].astype(np.float32)}))
    bad = {**batch, "head": batch["head"].copy()}
    bad["head"][0, 0, 0] = 10**6
    with pytest.raises(ValueError, match="out of range"):
        engine.run("train_step_loop", dict(learning_rate=lr, loss=loss, **bad))


def test_transh_relation_normal_step_size_modifier(oracle64):
    # training.learning_rate_modifiers is keyed by parameter name (src/poplar_kge.cpp:321-327):
    # relation_normal takes its own factor, with private tables (per-shard step sizes) and a
    # shared one.  One step, so that each parameter's update depends on its own step size only;
    # the oracle has one factor for the whole relation array, so it runs once per factor.
    import libpoplar_kge

    mods = {"relation_normal": 0.25, "relation_embedding": 2.0}
    for shared in (False, True):
        c = K.cfg_dict(score_fn="TransH", feature=0, shared_table=shared, n_shard=2, n_entity=90)
        rng = np.random.default_rng(31)
        st0 = K.make_state(c, rng)
        batch = K.random_batch(c, 1, rng)
        lr = np.array([0.1, 0.1 if shared else 0.04], np.float32)
        engine = libpoplar_kge.Engine(H.engine_settings(c, 1, **{"training.learning_rate_modifiers": mods}), "")
        H.load_state(engine, c, st0)
        H.train(engine, c, lr, batch)
        st_h = H.read_state(engine, c)
        for name, mod in mods.items():
            st_o = K.copy_state(st0)
            oracle64.train_step_loop(make_cfg(**c, lr_mod_relation=mod), st_o, lr, batch)
            assert K.rel_l2(st_h[name] - st0[name], st_o[name] - st0[name]) < 1e-4, (shared, name)
            for suffix in ("/adam_m", "/adam_v"):
                assert K.rel_l2(st_h[name + suffix], st_o[name + suffix]) < 1e-5, (shared, name, suffix)
        # and the two factors really differ in effect
        st_o = K.copy_state(st0)
        oracle64.train_step_loop(make_cfg(**c), st_o, lr, batch)
        assert K.rel_l2(st_h["relation_normal"] - st0["relation_normal"],
                        st_o["relation_normal"] - st0["relation_normal"]) > 0.5


def test_transh_zipf_duplicates(oracle64):
    # heavy duplicates among heads, tails and relations: hot entity rows and hot relation rows
    # (both copies) go through the chunked reduction
    kw = dict(score_fn="TransH", n_shard=4, batch=64, a2a=16, dim=32, feature=0, n_entity=500, n_relation=4,
              shared_table=True, gamma=4.0)
    run_case(oracle64, kw, n_step=2, batch_fn=K.raw_batch)


def test_dropout_masks_follow_the_optimiser_step(oracle64):
    # two calls of two steps each: the masks of the second call are those of steps 2 and 3 after
    # the state's own step count, on the device as in the oracle; and dropout really acts (the
    # same run without it ends elsewhere)
    kw = dict(feature_dropout=0.5, dropout_seed=21)
    c, st0, st_h, _ = run_case(oracle64, kw, n_step=2, n_loop=2)
    st_plain = K.copy_state(st0)
    rng = np.random.default_rng(11)
    K.make_state(c, rng)  # advance the generator as run_case did
    plain = dict(c, feature_dropout=0.0)
    for _ in range(2):
        oracle64.train_step_loop(make_cfg(**plain), st_plain, np.array([0.1, 0.07], np.float32), K.random_batch(c, 2, rng))
    k = "feature_projection"
    assert K.rel_l2(st_h[k] - st0[k], st_plain[k] - st0[k]) > 0.05


# ---- the step's gradients themselves -------------------------------------------------------------

GRADIENT_CASES = {
    # the 1M-row workload's block shape (256 positives x 256 shared tails, D = 256), raw power-law
    # ids over one shared table: hot rows, repeated tails, tile-aligned fast paths
    "c2_shaped_l2": (dict(distance_fn="L2", n_shard=4, batch=256, a2a=64, dim=256, feature=0, n_entity=20_000,
                          n_relation=40, gamma=10.0, shared_table=True), ("mfma_bf16x3", "mfma", "valu")),
    # the one-pass L1 backward (tails split over sixteen waves)
    "paired_l1": (dict(distance_fn="L1", n_shard=32, batch=32, a2a=8, dim=256, feature=0, n_entity=4000,
                       n_relation=8, gamma=6.0, shared_table=True), ("mfma_bf16x3",)),
}


@pytest.mark.parametrize("merge", [True, False])
@pytest.mark.parametrize("name,scoring", [(n, s) for n, (_, ss) in GRADIENT_CASES.items() for s in ss])
def test_step_gradients_vs_oracle(oracle64, name, scoring, merge):
    """The summed gradient of every distinct entity row and of every relation row of one step
    (what loss.backward(lossScale) and multiUpdateAdd leave, src/poplar_kge.cpp:691,
    src/pag/pag.cpp:721-743) against the float64 oracle's: 1e-5 relative as a whole, and every
    element within 1e-5 of its row's root mean square."""
    import libpoplar_kge

    c = K.cfg_dict(**GRADIENT_CASES[name][0])
    rng = np.random.default_rng(31)
    st0 = K.make_state(c, rng)
    batch = K.raw_batch(c, 1, rng)
    lr = np.full(c["n_shard"], 0.01, np.float32)
    engine = libpoplar_kge.Engine(H.engine_settings(c, 1, **{"execution.scoring": scoring,
                                                             "execution.keep_gradients": True,
                                                             "execution.merge_tails": merge}), "")
    H.load_state(engine, c, st0)
    H.train(engine, c, lr, batch)
    S, B, A, D = c["n_shard"], c["batch"], c["a2a"], c["dim"]
    R = S * (B + S * A)
    out = dict(unique_rows=np.zeros(R, np.uint32), counts=np.zeros(2, np.uint32),
               entity_gradient=np.zeros((R, D), np.float32),
               relation_gradient=np.zeros((c["n_relation"], D), np.float32))
    engine.run("grad_dump", out)
    ent = np.full((st0["entity_data"].shape[0], D), np.nan)
    rel = np.full((c["n_relation"], D), np.nan)
    oracle64.gradient_tap(ent, rel)
    try:
        oracle64.train_step_loop(make_cfg(**c), K.copy_state(st0), lr, batch)
    finally:
        oracle64.gradient_tap(None, None)
    U = int(out["counts"][0])
    rows = out["unique_rows"][:U]
    np.testing.assert_array_equal(rows, np.flatnonzero(~np.isnan(ent[:, 0])))
    for got, ref in ((out["entity_gradient"][:U], ent[rows]), (out["relation_gradient"], rel)):
        assert K.rel_l2(got, ref) < 1e-5
        rms = np.sqrt(np.mean(ref * ref, axis=1, keepdims=True))
        assert np.all(np.abs(got - ref) <= 1e-5 * rms + 1e-30), float(np.max(np.abs(got - ref) / (rms + 1e-30)))
    assert np.count_nonzero(np.any(ent[rows] != 0, axis=1)) > U // 2


# ---- merged tails: blocks whose tail lists repeat rows ---------------------------------------------

def _repeated_tail_batch(c, n_step, rng, kind):
    """Batches in the reference's layout whose tail lists repeat rows: `label_repeated` points every
    positive's label at a row that other tail positions of the block hold too; `one_row` fills a
    whole block's tails with a single row; `few_rows` draws all tails from four rows."""
    batch = K.random_batch(c, n_step, rng)
    S, A = c["n_shard"], c["a2a"]
    a2a = batch["a2a"]                      # [src shard, step, dst block, A]: slots of the source's remote
    if kind == "one_row":
        # block 0: every source sends its slot 0 only, which holds the same id everywhere (one
        # table row with a shared table, one row per source's table otherwise)
        a2a[:, :, 0, :] = 0
        batch["remote"][:, :, 0] = batch["remote"][:1, :, 0]
    elif kind == "few_rows":
        a2a[...] = rng.integers(0, 4, a2a.shape)
        batch["remote"][1:, :, :4] = batch["remote"][:1, :, :4]
    else:
        # tail position 0 of every block repeats at positions 1 and 2 (same source, same slot); labels name 0, 1 or 2
        a2a[0, :, :, 1] = a2a[0, :, :, 0]
        a2a[0, :, :, 2] = a2a[0, :, :, 0]
        batch["tail"][...] = rng.integers(0, 3, batch["tail"].shape)
    return batch


@pytest.mark.parametrize("kind", ["label_repeated", "one_row", "few_rows"])
@pytest.mark.parametrize("name", ["l2_logsigmoid", "l2_softmax", "l1_adversarial", "demo_l1_logsigmoid",
                                  "distmult_softmax_feat", "aligned_l2", "aligned_l2_softmax", "paired_l1_t256",
                                  "mid_l1"])
def test_step_repeated_tails(oracle64, name, kind):
    """One score column per distinct tail row, weighted by its multiplicity, against the oracle,
    which scores every tail position (src/poplar_kge.cpp:615-660): the label's row repeated among
    the negatives, a block whose tails are all one row, tails drawn from four rows."""
    kw = dict(CASES[name])
    run_case(oracle64, kw, n_step=2, batch_fn=lambda c, n, rng: _repeated_tail_batch(c, n, rng, kind))
    run_case(oracle64, kw, n_step=2, batch_fn=lambda c, n, rng: _repeated_tail_batch(c, n, rng, kind),
             **{"execution.merge_tails": False})


def _tails_with_distinct_counts(c, n_step, rng):
    """Raw-id batches (kge_synthetic.raw_batch) in which block d's T tail positions hold exactly
    counts[d] distinct rows: each of them once, then repeats."""
    S, A, B = c["n_shard"], c["a2a"], c["batch"]
    T = S * A
    batch = K.raw_batch(c, n_step, rng, zipf=False)
    counts = np.concatenate([[1, 20, 33, 64, 90, 100, 129, 150, 190, 200, 230, 256, 280, 300, 320, 330, 352, 370,
                              385, 400, 416, 440, 449, 470, 480, 490, 500, 512], rng.integers(1, T + 1, S)])[:S]
    for step in range(n_step):
        for d in range(S):
            n = int(min(counts[(d + step) % S], T))
            pool = rng.choice(np.arange(1, c["n_entity"]), n, replace=False).astype(np.uint32)
            rows = np.concatenate([pool, pool[rng.integers(0, n, T - n)]])
            rng.shuffle(rows)
            # block d's tails: slots B + d A .. + A - 1 of every source shard's `remote`
            batch["remote"][:, step, B + d * A:B + (d + 1) * A] = rows.reshape(S, A)
    return batch


def test_step_paired_l1_distinct_tail_counts(oracle64):
    """The paired L1 backward splits a block's distinct tails, in whole groups of 32, over its 16
    waves and has one copy of its loop per tails-per-wave count (2, 4, ... 32): blocks with 1 to
    512 distinct tails of 512 positions, against the oracle."""
    run_case(oracle64, dict(CASES["paired_l1_t512"]), n_step=2, batch_fn=_tails_with_distinct_counts)


def test_host_arrays_are_checked_chunk_by_chunk():
    """Host index arrays are checked, re-ordered and uploaded in chunks of 2, 4, 8, ... steps beside
    the device's work.  An index out of range raises as before; the chunks in front of the
    offending one have been applied by then (the reference checks shapes and types only,
    src/poplar_kge.cpp:69-106), and the engine stays usable."""
    import libpoplar_kge

    c = K.cfg_dict(feature=0, n_shard=2, batch=6, a2a=5, dim=8, n_entity=90, n_relation=12)
    rng = np.random.default_rng(5)
    st0 = K.make_state(c, rng)
    n_step = 7                                   # chunks of 2, 4 and 1 steps
    batch = K.random_batch(c, n_step, rng)
    engine = libpoplar_kge.Engine(H.engine_settings(c, n_step), "")
    H.load_state(engine, c, st0)
    bad = {k: v.copy() for k, v in batch.items()}
    bad["a2a"][1, 6, 0, 2] = 10**6               # in the last chunk
    with pytest.raises(ValueError, match=r"'a2a' holds index 1000000 out of range \[0, 16\) \(step 6\)"):
        H.train(engine, c, 0.05, bad)
    st = H.read_state(engine, c)
    assert st["step"] == st0["step"] + 6         # the first two chunks ran
    # the same six steps through the oracle, then a whole good call on top: the engine is intact
    ref = K.copy_state(st0)
    from oracle.kge_oracle import Oracle
    orc = Oracle("f64")
    orc.train_step_loop(make_cfg(**c), ref, 0.05, {k: v[:, :6] for k, v in batch.items()})
    assert K.rel_l2(st["entity_data"], ref["entity_data"]) < 1e-5
    loss_h = H.train(engine, c, 0.05, batch)
    loss_o = orc.train_step_loop(make_cfg(**c), ref, 0.05, batch)
    np.testing.assert_allclose(loss_h, loss_o, rtol=1e-5)
    assert K.rel_l2(H.read_state(engine, c)["entity_data"], ref["entity_data"]) < 1e-5
    # an index out of range in the first chunk: nothing has run
    bad = {k: v.copy() for k, v in batch.items()}
    bad["remote"][0, 1, 3] = 90
    with pytest.raises(ValueError, match="'remote' holds index 90 out of range"):
        H.train(engine, c, 0.05, bad)
    assert H.read_state(engine, c)["step"] == st0["step"] + 6 + n_step


def test_staged_batch_in_one_call_or_in_pieces():
    """A staged batch's steps run in one call or in several (`step_begin` / `step_count`: the
    plan then covers each call's steps only) must leave bit-identical tables: 40 steps in one
    call against the same 40 steps in two calls of 20 on a second engine, and both against the
    oracle."""
    import libpoplar_kge

    c = K.cfg_dict(feature=0, n_shard=4, batch=32, a2a=8, dim=16, n_entity=400, n_relation=9, shared_table=True)
    rng = np.random.default_rng(77)
    st0 = K.make_state(c, rng)
    n_step = 40
    batch = K.raw_batch(c, n_step, rng)
    lr = np.full(c["n_shard"], 0.02, np.float32)
    results = []
    for pieces in ([(0, 40)], [(0, 20), (20, 20)]):
        engine = libpoplar_kge.Engine(H.engine_settings(c, n_step), "")
        H.load_state(engine, c, st0)
        engine.run("stage_batch", {k: np.ascontiguousarray(v) for k, v in batch.items()})
        losses = []
        for begin, count in pieces:
            loss = np.full(c["n_shard"], np.nan, np.float32)
            engine.run("train_step_loop", dict(learning_rate=lr, loss=loss, staged=True,
                                               step_begin=int(begin), step_count=int(count)))
            losses.append(loss * count)
        results.append((sum(losses) / n_step, H.read_state(engine, c)))
    (loss_a, st_a), (loss_b, st_b) = results
    assert st_a["step"] == st_b["step"] == st0["step"] + n_step
    np.testing.assert_allclose(loss_a, loss_b, rtol=1e-6)   # (a mean over 40 against two means over 20)
    for name in ("entity_data", "relation_embedding", "relation_embedding/adam_m", "relation_embedding/adam_v"):
        np.testing.assert_array_equal(st_a[name], st_b[name])
    # and against the oracle
    from oracle.kge_oracle import Oracle
    ref = K.copy_state(st0)
    loss_o = Oracle("f64").train_step_loop(make_cfg(**c), ref, 0.02, batch)
    np.testing.assert_allclose(loss_a, loss_o, rtol=1e-5)
    assert K.rel_l2(st_a["entity_data"], ref["entity_data"]) < 1e-5
