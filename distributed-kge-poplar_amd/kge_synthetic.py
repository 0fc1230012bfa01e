"""Seeded synthetic workloads for the training step: the table sizes, block shapes and id
distributions the measurements and the full-size parity tests run on, and the helpers that
put them on a device through the engine's own commands.

Ids are 1-based (row 0 is the padding row, as in the reference,
src/python/poplar_kge.py:420-423), drawn either uniformly or from the bounded power law
P(k) ~ k^-1.1 over k = 1 .. N-1 by inverse CDF; relations and labels are uniform.  A batch
lists raw ids with identity slot maps (every block's heads, then the tails it contributes),
so that all de-duplication happens on the device.
"""

import numpy as np

# One shared table addressed by K blocks = K virtual shards.
WORKLOADS = {
    "c1": dict(desc="TransE-L2 D=64 fp32, 10k entities, 1 block x (256 positives, 64 shared tails)",
               n_entity=10_000, n_relation=50, dim=64, blocks=1, batch=256, tails=64,
               distance_fn="L2", uniform=True),
    "c2": dict(desc="TransE-L2 D=256 fp32, 1M entities, 32 blocks x (256 positives, 256 shared tails)",
               n_entity=1_000_000, n_relation=1000, dim=256, blocks=32, batch=256, tails=256,
               distance_fn="L2"),
    "c3": dict(desc="TransE-L1 D=256 fp32, 22.8M entities, 64 blocks x (256 positives, 512 shared tails)",
               n_entity=22_800_000, n_relation=1387, dim=256, blocks=64, batch=256, tails=512,
               distance_fn="L1"),
    "c3l2": dict(desc="TransE-L2 D=256 fp32, 22.8M entities, 64 blocks x (256 positives, 512 shared tails)",
                 n_entity=22_800_000, n_relation=1387, dim=256, blocks=64, batch=256, tails=512,
                 distance_fn="L2"),
    "c4": dict(desc="DistMult D=512 + 768-dim fp16 feature projected 768->512, 4M entities, "
                    "1 block x (8192 positives, 2048 shared tails), softmax CE",
               n_entity=4_000_000, n_relation=1387, dim=512, blocks=1, batch=8192, tails=2048,
               score_fn="DistMult", distance_fn="MatMul", loss="softmax", feature=768,
               feature_dtype="float16", scoring_dtype="bfloat16"),
    "c5": dict(desc="TransE-L2 D=256 bf16 embedding + fp32 moments, 91.2M entities, "
                    "32 blocks x (512 positives, 512 shared tails)",
               n_entity=91_200_000, n_relation=1387, dim=256, blocks=32, batch=512, tails=512,
               distance_fn="L2", embedding_dtype="bfloat16"),
}

SEED = 20240611


def zipf_ids(rng, n_rows, size, s=1.1):
    """Bounded power law P(k) ~ k^-s over ids 1..n_rows-1, inverse-CDF sampled."""
    k = np.arange(1, n_rows, dtype=np.float64)
    cdf = np.cumsum(k**-s)
    cdf /= cdf[-1]
    return (1 + np.searchsorted(cdf, rng.random(size))).astype(np.uint32)


def raw_batch(c, n_step, rng, zipf=True):
    """Raw (non-deduplicated) ids with identity slot maps: ``remote`` holds
    every head id then every tail id the shard sends; duplicates allowed.
    ``c``: n_shard, n_entity, batch, a2a, n_relation."""
    S, NE, B, A = c["n_shard"], c["n_entity"], c["batch"], c["a2a"]
    T = S * A
    NR = B + T
    shape = (S, n_step, NR)
    remote = zipf_ids(rng, NE, shape) if zipf else rng.integers(1, NE, shape).astype(np.uint32)
    head = np.broadcast_to(np.arange(B, dtype=np.uint32), (S, n_step, B)).copy()
    a2a = np.broadcast_to((B + np.arange(T, dtype=np.uint32)).reshape(S, A),
                          (S, n_step, S, A)).copy()
    return dict(
        remote=remote, a2a=a2a, head=head,
        relation=rng.integers(0, c["n_relation"], (S, n_step, B)).astype(np.uint32),
        tail=rng.integers(0, T, (S, n_step, B)).astype(np.uint32),
    )


def row_bytes(w):
    """Bytes of one stacked table row [emb | m | sqrt v | feature]."""
    return ((2 if w.get("embedding_dtype") == "bfloat16" else 4) * w["dim"] + 8 * w["dim"]
            + (2 if w.get("feature_dtype") == "float16" else 4) * w.get("feature", 0))


def make_settings(w, n_step, kge):
    """The engine settings of workload ``w`` with ``n_step`` steps per program run."""
    s = kge.Settings.create_demo()
    s.seed = SEED
    m, d, t, e = s.model, s.data, s.training, s.execution
    m.score_fn, m.distance_fn = w.get("score_fn", "TransE"), w["distance_fn"]
    m.n_shard, m.n_entity, m.n_relation_type = w["blocks"], w["n_entity"], w["n_relation"]
    m.embedding_size, m.entity_feature_size, m.gamma = w["dim"], w.get("feature", 0), 10.0
    m.init_scale = float(np.sqrt(w["dim"]))  # embeddings ~ N(0, 1/sqrt(D)): sigma = init_scale / D
    d.batch_size, d.a2a_size = w["batch"], w["tails"] // w["blocks"]
    t.learning_rate = 1e-3
    t.loss = kge.SoftmaxLoss(correction_weight=1.0) if w.get("loss") == "softmax" else kge.LogSigmoidLoss()
    e.device, e.dtype, e.shared_table = "hip", "float32", True
    e.embedding_dtype, e.feature_dtype = w.get("embedding_dtype"), w.get("feature_dtype")
    e.scoring_dtype = w.get("scoring_dtype")
    if w.get("scoring"):
        e.scoring = w["scoring"]
    for key, value in w.get("execution", {}).items():  # further execution.* settings (experiments)
        setattr(e, key, value)
    e.train_steps_per_program_run = n_step
    e.rw_batch_size = 8192
    return s.prepare()


def make_batch(w, n_step, kge):
    c = dict(n_shard=w["blocks"], n_entity=w["n_entity"], batch=w["batch"],
             a2a=w["tails"] // w["blocks"], n_relation=w["n_relation"])
    rng = np.random.Generator(np.random.PCG64(SEED + 1))
    return kge.Batch(**raw_batch(c, n_step, rng, zipf=not w.get("uniform", False)))


def init_tables(engine, settings):
    """write_entity over the whole table (random-normal embeddings drawn on the
    device).  The table is shared, so each of the n_shard index rows of one call
    covers a different range of table rows."""
    engine.initialise_variables()
    m, e = settings.model, settings.execution
    per_call = m.n_shard * e.rw_batch_size
    feat = np.zeros(settings.entity_data_w_shape, np.float32)
    if m.entity_feature_size:
        # N(0, 1) features; one block of them serves every call (rows per_call apart share features)
        feat = np.random.default_rng(settings.seed + 5).normal(size=feat.shape).astype(np.float32)
    for off in range(0, m.n_entity, per_call):
        idx = np.arange(off, off + per_call, dtype=np.int64)
        idx[idx >= m.n_entity] = 0
        engine.engine.run("write_entity", dict(
            write_indices=idx.astype(np.uint32).reshape(m.n_shard, -1), write_features=feat))
    # row 0 last, so that the overflow of the final chunk does not decide its content
    idx = np.zeros(per_call, np.uint32)
    engine.engine.run("write_entity", dict(write_indices=idx.reshape(m.n_shard, -1), write_features=feat))
    engine.uninitialized_entity_data[:] = False


def read_rows(engine, settings, ids):
    """Rows `ids` of the shared table as float32 [len(ids), 3D+F] (read_entity)."""
    m, e = settings.model, settings.execution
    per_call = m.n_shard * e.rw_batch_size
    out = np.zeros((len(ids), settings.entity_data_r_size), np.float32)
    for off in range(0, len(ids), per_call):
        chunk = ids[off:off + per_call]
        idx = np.zeros(per_call, np.uint32)
        idx[:len(chunk)] = chunk
        data = np.zeros(settings.entity_data_r_shape, np.float32)
        engine.engine.run("read_entity", dict(read_indices=idx.reshape(m.n_shard, -1), read_data=data))
        out[off:off + len(chunk)] = data.reshape(per_call, -1)[:len(chunk)]
    return out
