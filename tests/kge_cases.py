"""Seeded synthetic states and batches shared by the oracle and GPU parity tests."""

import numpy as np


def cfg_dict(**kw):
    d = dict(n_shard=2, n_entity=90, n_relation=12, dim=8, feature=6, batch=6, a2a=5,
             score_fn="TransE", distance_fn="L1", loss_fn="logsigmoid", shared_table=False,
             storage="float32", scoring_bf16=False, gamma=2.0, beta_m=0.9, beta_v=0.999, epsilon=1e-8,
             weight_decay=0.0, loss_scale=None, softmax_correction_weight=0.0,
             negative_adversarial_scale=0.0, embedding_regularisation=(3.0, 0.0),
             feature_regularisation=(3.0, 0.0), hidden_regularisation=(3.0, 0.0), feature_mlp_size=0,
             feature_dropout=0.0, dropout_seed=0, share_feature_networks=True)
    d.update(kw)
    if d["loss_scale"] is None:
        d["loss_scale"] = float(d["batch"] * d["n_shard"] * d["a2a"])
    return d


def make_state(c, rng, warm=True, scale=None):
    """Random tables.  ``warm``: non-zero Adam moments and step, so the update
    formula is exercised away from its zero-state special case.  The second
    moments stay away from zero: m / (sqrt(v) + eps) with sqrt(v) ~ 1e-5 turns a
    float32 rounding difference in a cancelling gradient sum into a visible
    change of the parameter, in any implementation."""
    S, NE, D, F, NR = c["n_shard"], c["n_entity"], c["dim"], c["feature"], c["n_relation"]
    rows = NE if c["shared_table"] else S * NE
    scale = scale if scale is not None else 1.0 / np.sqrt(D)
    ed = np.zeros((rows, 3 * D + F), np.float32)
    ed[:, :D] = rng.normal(0, scale, (rows, D))
    if warm:
        ed[:, D:2 * D] = rng.normal(0, 0.1, (rows, D))
        ed[:, 2 * D:3 * D] = 0.05 + np.abs(rng.normal(0, 0.3, (rows, D)))
    if F:
        ed[:, 3 * D:] = rng.normal(0, 1, (rows, F)).astype(np.float16)
    rotate = c["score_fn"] == "RotatE"   # relation rows are D / 2 phases
    RD = D // 2 if rotate else D
    st = {
        "entity_data": ed,
        "relation_embedding": rng.normal(0, 1.0 if rotate else scale, (NR, RD)).astype(np.float32),
        "relation_embedding/adam_m": (rng.normal(0, 0.1, (NR, RD)) * warm).astype(np.float32),
        "relation_embedding/adam_v": ((0.05 + np.abs(rng.normal(0, 0.3, (NR, RD))))**2 * warm).astype(np.float32),
        "step": 7 if warm else 0,
    }
    if c["score_fn"] == "TransH":
        st["relation_normal"] = rng.normal(0, scale, (NR, D)).astype(np.float32)
        st["relation_normal/adam_m"] = (rng.normal(0, 0.1, (NR, D)) * warm).astype(np.float32)
        st["relation_normal/adam_v"] = ((0.05 + np.abs(rng.normal(0, 0.3, (NR, D))))**2 * warm).astype(np.float32)
    # one feature network, or a head and a tail one (src/python/poplar_kge.py:652-686)
    for pre in (("",) if c.get("share_feature_networks", True) else ("head_", "tail_")) if F else ():
        shapes = [("feature_projection", (F, D), scale / np.sqrt(F))]
        M = c.get("feature_mlp_size", 0)
        if M:
            shapes += [("mlp_up_projection", (2 * D, M), 1 / np.sqrt(2 * D)), ("mlp_down_projection", (M, D), 1 / np.sqrt(M))]
        for name, shape, sigma in shapes:
            st[pre + name] = rng.normal(0, sigma, shape).astype(np.float32)
            st[pre + name + "/adam_m"] = (rng.normal(0, 0.1, shape) * warm).astype(np.float32)
            st[pre + name + "/adam_v"] = ((0.05 + np.abs(rng.normal(0, 0.3, shape)))**2 * warm).astype(np.float32)
    return st


def copy_state(st):
    return {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in st.items()}


def random_batch(c, n_step, rng, pad=0):
    """The reference test's batch shape (tests/python/test_poplar_kge.py:51-91):
    ``remote`` sorted unique non-zero rows (the last ``pad`` entries zero
    padding), random slots for head / a2a, random relations and labels."""
    S, NE, B, A = c["n_shard"], c["n_entity"], c["batch"], c["a2a"]
    NR = B + S * A
    remote = np.zeros((S, n_step, NR), np.uint32)
    for s in range(S):
        for i in range(n_step):
            remote[s, i, :NR - pad] = np.sort(rng.choice(np.arange(1, NE), NR - pad, replace=False))
    lim = NR - pad if pad else NR
    return dict(
        remote=remote,
        a2a=rng.integers(0, lim, (S, n_step, S, A)).astype(np.uint32),
        head=rng.integers(0, lim, (S, n_step, B)).astype(np.uint32),
        relation=rng.integers(0, c["n_relation"], (S, n_step, B)).astype(np.uint32),
        tail=rng.integers(0, S * A, (S, n_step, B)).astype(np.uint32),
    )


# the raw-id batches and the power-law id sampler are the measurement workloads' own
from kge_synthetic import raw_batch, zipf_ids  # noqa: E402,F401


def step_slice(batch, i):
    return {k: v[:, i] for k, v in batch.items()}


def rel_l2(x, ref):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    den = np.sqrt(np.sum(ref * ref))
    return float(np.sqrt(np.sum((x - ref)**2)) / (den if den > 0 else 1.0))
