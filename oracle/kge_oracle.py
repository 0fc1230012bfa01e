"""ctypes front end of the CPU oracle (``kge_oracle.c``).

TEST INFRASTRUCTURE ONLY.  Importable from ``tests/``, the smoke check and the
bench's ``cpu_baseline`` leg; never from the product package.  ``build()``
compiles the two libraries with the Makefile beside this file.
"""

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent

SCORE = {"TransE": 0, "DistMult": 1, "ComplEx": 2, "RotatE": 3, "TransH": 4}
DIST = {"L1": 0, "L2": 1, "MatMul": 2}
LOSS = {"logsigmoid": 0, "softmax": 1}
STORE = {"float32": 0, "float16": 1, "bfloat16_embedding": 2}


class Cfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "n_shard", "n_entity", "n_relation", "dim", "feature", "batch", "a2a", "score_fn",
        "distance_fn", "loss_fn", "shared_table", "storage", "mlp_size", "scoring_bf16")] + [(n, C.c_float) for n in (
            "gamma", "beta_m", "beta_v", "epsilon", "weight_decay", "loss_scale",
            "softmax_correction_weight", "negative_adversarial_scale", "lr_mod_entity",
            "lr_mod_relation", "lr_mod_projection", "reg_emb_power", "reg_emb_weight", "reg_feat_power",
            "reg_feat_weight", "reg_hid_power", "reg_hid_weight", "dropout")] + [
                ("dropout_seed", C.c_uint32), ("separate_networks", C.c_int32)]


def make_cfg(*, n_shard, n_entity, n_relation, dim, feature=0, batch, a2a, score_fn="TransE",
             distance_fn="L1", loss_fn="logsigmoid", shared_table=False, storage="float32",
             scoring_bf16=False, gamma=0.0, beta_m=0.9, beta_v=0.999, epsilon=1e-8, weight_decay=0.0,
             loss_scale=None, softmax_correction_weight=0.0, negative_adversarial_scale=0.0,
             lr_mod_entity=1.0, lr_mod_relation=1.0, lr_mod_projection=1.0,
             embedding_regularisation=(3.0, 0.0), feature_regularisation=(3.0, 0.0),
             hidden_regularisation=(3.0, 0.0), feature_mlp_size=0, feature_dropout=0.0, dropout_seed=0,
             share_feature_networks=True):
    """The three regularisers are (power, weight) pairs (src/python/poplar_kge.py:104-108)."""
    if loss_scale is None:  # src/python/poplar_kge.py:259-262
        loss_scale = float(batch * n_shard * a2a)
    return Cfg(n_shard, n_entity, n_relation, dim, feature, batch, a2a, SCORE[score_fn],
               DIST[distance_fn], LOSS[loss_fn], int(shared_table), STORE[storage], int(feature_mlp_size) if feature else 0,
               int(scoring_bf16),
               gamma, beta_m,
               beta_v, epsilon, weight_decay, loss_scale, softmax_correction_weight,
               negative_adversarial_scale, lr_mod_entity, lr_mod_relation, lr_mod_projection,
               *embedding_regularisation, *feature_regularisation, *hidden_regularisation,
               float(feature_dropout), int(dropout_seed), int(bool(feature) and not share_feature_networks))


def build(force=False):
    libs = [HERE / "libkge_oracle_f64.so", HERE / "libkge_oracle_f32.so"]
    src = HERE / "kge_oracle.c"
    if force or any(not p.exists() or p.stat().st_mtime < src.stat().st_mtime for p in libs):
        subprocess.run(["make", "-C", str(HERE), "-B" if force else "-s", "all"], check=True)
    return libs


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class Oracle:
    """One loaded oracle library; ``precision`` is "f64" (truth) or "f32"."""

    def __init__(self, precision="f64"):
        path = HERE / f"libkge_oracle_{precision}.so"
        if not path.exists():
            build()
        self.lib = C.CDLL(os.fspath(path))
        self.lib.kge_oracle_loss.restype = C.c_float
        self.lib.kge_oracle_adam_step_size.restype = C.c_float
        self.lib.kge_oracle_round.restype = C.c_float
        self.lib.kge_oracle_round.argtypes = [C.c_float, C.c_int]
        self.precision = precision

    # -- ops ---------------------------------------------------------------
    def buffer_read(self, buf, idx):
        buf, idx = _f32(buf), _u32(idx)
        out = np.empty((idx.size, buf.shape[1]), np.float32)
        self.lib.kge_oracle_buffer_read(_p(buf), C.c_int64(buf.shape[1]), _p(idx),
                                        C.c_int64(idx.size), _p(out))
        return out

    def buffer_write(self, buf, idx, data):
        assert buf.dtype == np.float32 and buf.flags.c_contiguous
        idx, data = _u32(idx), _f32(data)
        self.lib.kge_oracle_buffer_write(_p(buf), C.c_int64(buf.shape[1]), _p(idx),
                                         C.c_int64(idx.size), _p(data))

    def multi_slice(self, t, idx):
        t, idx = _f32(t), _u32(idx)
        out = np.empty((idx.size, t.shape[1]), np.float32)
        self.lib.kge_oracle_multi_slice(_p(t), C.c_int64(t.shape[1]), _p(idx),
                                        C.c_int64(idx.size), _p(out))
        return out

    def multi_update_add(self, rows, idx, grad_out):
        idx, grad_out = _u32(idx), _f32(grad_out)
        out = np.empty((rows, grad_out.shape[1]), np.float32)
        self.lib.kge_oracle_multi_update_add(_p(out), C.c_int64(rows),
                                             C.c_int64(grad_out.shape[1]), _p(idx),
                                             C.c_int64(idx.size), _p(grad_out))
        return out

    def _dist(self, fn, a, b):
        a, b = _f32(a), _f32(b)
        out = np.empty((a.shape[0], b.shape[0]), np.float32)
        fn(_p(a), _p(b), C.c_int64(a.shape[0]), C.c_int64(b.shape[0]), C.c_int64(a.shape[1]),
           _p(out))
        return out

    def l1_distance(self, a, b):
        return self._dist(self.lib.kge_oracle_l1_distance, a, b)

    def l2_distance(self, a, b):
        return self._dist(self.lib.kge_oracle_l2_distance, a, b)

    def dot_score(self, a, b):
        return self._dist(self.lib.kge_oracle_dot_score, a, b)

    def l1_distance_grad(self, a, b, g):
        """Gradient of the first operand; call with (b, a, g.T) for the second."""
        a, b, g = _f32(a), _f32(b), _f32(g)
        out = np.empty_like(a)
        self.lib.kge_oracle_l1_distance_grad(_p(a), _p(b), _p(g), C.c_int64(a.shape[0]),
                                             C.c_int64(b.shape[0]), C.c_int64(a.shape[1]), _p(out))
        return out

    def l2_distance_grad(self, a, b, dist, g):
        a, b, dist, g = _f32(a), _f32(b), _f32(dist), _f32(g)
        out = np.empty_like(a)
        self.lib.kge_oracle_l2_distance_grad(_p(a), _p(b), _p(dist), _p(g),
                                             C.c_int64(a.shape[0]), C.c_int64(b.shape[0]),
                                             C.c_int64(a.shape[1]), _p(out))
        return out

    def log_sigmoid(self, x):
        x = _f32(x)
        y = np.empty_like(x)
        self.lib.kge_oracle_log_sigmoid(_p(x), C.c_int64(x.size), _p(y))
        return y

    def log_sigmoid_grad(self, x, dy):
        x, dy = _f32(x), _f32(dy)
        dx = np.empty_like(x)
        self.lib.kge_oracle_log_sigmoid_grad(_p(x), _p(dy), C.c_int64(x.size), _p(dx))
        return dx

    def log_softmax(self, x):
        x = _f32(x)
        x2 = x.reshape(-1, x.shape[-1])
        y = np.empty_like(x2)
        self.lib.kge_oracle_log_softmax(_p(x2), C.c_int64(x2.shape[0]), C.c_int64(x2.shape[1]),
                                        _p(y))
        return y.reshape(x.shape)

    def log_softmax_grad(self, y, dy):
        y, dy = _f32(y), _f32(dy)
        y2, dy2 = y.reshape(-1, y.shape[-1]), dy.reshape(-1, y.shape[-1])
        dx = np.empty_like(y2)
        self.lib.kge_oracle_log_softmax_grad(_p(y2), _p(dy2), C.c_int64(y2.shape[0]),
                                             C.c_int64(y2.shape[1]), _p(dx))
        return dx.reshape(y.shape)

    def softmax_cross_entropy(self, logits, labels):
        logits, labels = _f32(logits), _u32(labels)
        l2 = logits.reshape(-1, logits.shape[-1])
        out = np.empty(l2.shape[0], np.float32)
        self.lib.kge_oracle_softmax_cross_entropy(_p(l2), _p(labels), C.c_int64(l2.shape[0]),
                                                  C.c_int64(l2.shape[1]), _p(out))
        return out

    def softmax(self, x):
        x = _f32(x)
        x2 = x.reshape(-1, x.shape[-1])
        y = np.empty_like(x2)
        self.lib.kge_oracle_softmax(_p(x2), C.c_int64(x2.shape[0]), C.c_int64(x2.shape[1]), _p(y))
        return y.reshape(x.shape)

    def adam_step_size(self, step, lr, beta_m=0.9, beta_v=0.999):
        """Returns (new_step, alpha)."""
        st = C.c_uint32(step)
        alpha = self.lib.kge_oracle_adam_step_size(C.byref(st), C.c_float(lr), C.c_float(beta_m),
                                                   C.c_float(beta_v))
        return st.value, alpha

    def adam(self, p, m, v, g, alpha, beta_m=0.9, beta_v=0.999, eps=1e-8, wd=0.0,
             v_is_sqrt=False):
        """In-place on float32 contiguous p, m, v."""
        for a in (p, m, v):
            assert a.dtype == np.float32 and a.flags.c_contiguous
        g = _f32(g)
        self.lib.kge_oracle_adam(_p(p), _p(m), _p(v), _p(g), C.c_int64(p.size), C.c_float(alpha),
                                 C.c_float(beta_m), C.c_float(beta_v), C.c_float(eps),
                                 C.c_float(wd), C.c_int(int(v_is_sqrt)))

    def round(self, x, storage):
        return np.array([self.lib.kge_oracle_round(float(v), STORE[storage])
                         for v in np.asarray(x, np.float32).ravel()],
                        np.float32).reshape(np.shape(x))

    def loss(self, cfg, score, label):
        """Shard loss and d(loss)/d(score) (before the loss scale)."""
        score, label = _f32(score), _u32(label)
        ds = np.empty_like(score)
        loss = self.lib.kge_oracle_loss(C.byref(cfg), _p(score), _p(label), _p(ds))
        return loss, ds

    def gradient_tap(self, ent=None, rel=None):
        """Test hook: float64 arrays [table rows, D] and [relation rows, D] that every following
        training step fills with the summed gradients its updates are made from (None: off)."""
        for a in (ent, rel):
            assert a is None or (a.dtype == np.float64 and a.flags.c_contiguous)
        self._tap = (ent, rel)   # keeps the arrays alive while the C side writes to them
        self.lib.kge_oracle_gradient_tap(_p(ent) if ent is not None else None,
                                         _p(rel) if rel is not None else None)

    # -- whole step --------------------------------------------------------
    def train_step_loop(self, cfg, state, lr, batch):
        """Runs n_step steps in place on ``state`` and returns loss f32[S].

        state: dict with float32 C-contiguous arrays ``entity_data``
        [n_tables*n_entity, 3D+F], ``relation_embedding`` (+ ``/adam_m``,
        ``/adam_v``), ``feature_projection`` (+ moments; may be absent when
        F == 0) and an int ``step``.  batch: dict of uint32 arrays laid out
        [S, n_step, ...] as the host passes them.
        """
        S = cfg.n_shard
        remote = _u32(batch["remote"])
        n_step = remote.shape[1]
        a2a, head = _u32(batch["a2a"]), _u32(batch["head"])
        relation, tail = _u32(batch["relation"]), _u32(batch["tail"])
        lr = _f32(np.broadcast_to(np.asarray(lr, np.float32), (S,)))
        for k in ("entity_data", "relation_embedding", "relation_embedding/adam_m",
                  "relation_embedding/adam_v"):
            assert state[k].dtype == np.float32 and state[k].flags.c_contiguous, k
        mlp = ("mlp_up_projection", "mlp_down_projection") if cfg.feature and cfg.mlp_size else ()
        # the feature networks' parameters: one network, or the head's then the tail's
        # (src/poplar_kge.cpp:268-273), each W then the MLP's Up and Down
        net_names = [pre + n for pre in (("head_", "tail_") if cfg.separate_networks else ("",))
                     for n in ("feature_projection",) + mlp]
        if cfg.feature:
            # the C side takes them back to back
            proj_arrays = [np.concatenate([_f32(state[n + x]).reshape(-1) for n in net_names])
                           if len(net_names) > 1 else state["feature_projection" + x]
                           for x in ("", "/adam_m", "/adam_v")]
            for a in proj_arrays:
                assert a.dtype == np.float32 and a.flags.c_contiguous
            proj = [_p(a) for a in proj_arrays]
        else:
            proj = [None, None, None]
        step = C.c_uint32(int(state["step"]))
        loss = np.zeros(S, np.float32)
        suffixes = ("", "/adam_m", "/adam_v")
        if cfg.score_fn == SCORE["TransH"]:
            # the C side takes the hyperplane normals as rows [n_relation, 2 n_relation) of the
            # relation arrays
            rel = [np.concatenate([_f32(state["relation_embedding" + x]), _f32(state["relation_normal" + x])])
                   for x in suffixes]
        else:
            rel = [state["relation_embedding" + x] for x in suffixes]
        rc = self.lib.kge_oracle_train_step_loop(
            C.byref(cfg), C.c_int32(n_step), _p(state["entity_data"]),
            _p(rel[0]), _p(rel[1]), _p(rel[2]), *proj, C.byref(step), _p(lr), _p(remote),
            _p(a2a), _p(head), _p(relation), _p(tail), _p(loss))
        assert rc == 0
        if cfg.score_fn == SCORE["TransH"]:
            n = cfg.n_relation
            for x, a in zip(suffixes, rel):
                state["relation_embedding" + x][...] = a[:n]
                state["relation_normal" + x][...] = a[n:]
        if cfg.feature and len(net_names) > 1:
            for x, a in zip(("", "/adam_m", "/adam_v"), proj_arrays):
                o = 0
                for n in net_names:
                    state[n + x][...] = a[o:o + state[n + x].size].reshape(state[n + x].shape)
                    o += state[n + x].size
        state["step"] = step.value
        return loss


def predict_reference(cfg, state, queries, shard_to_count, n_best):
    """Brute-force tail prediction in float64 (tests/python/reference_model.py:169-206):
    score every (head shard, head row, relation) query against every real row of
    every shard's table and return the n_best best as (shard, row) and score,
    best first, ties to the lower (shard, row).

    state as for ``train_step_loop`` with private tables (``entity_data``
    [n_shard * n_entity, 3D+F]); queries int[n, 3]."""
    S, NE, D, F = cfg.n_shard, cfg.n_entity, cfg.dim, cfg.feature
    rows = np.asarray(state["entity_data"], np.float64).reshape(S * NE, -1)
    value = rows[:, :D]

    def hidden_of(prefix):  # entityHidden for the part whose network has this prefix (:439-467)
        if not F:
            return value.copy()
        fh = rows[:, 3 * D:3 * D + F] @ np.asarray(state[prefix + "feature_projection"], np.float64)
        if cfg.mlp_size:  # :453-458
            boom = np.maximum(np.concatenate([value, fh], 1)
                              @ np.asarray(state[prefix + "mlp_up_projection"], np.float64), 0)
            fh = boom @ np.asarray(state[prefix + "mlp_down_projection"], np.float64)
        return value + fh

    # the candidates are tails, the queries heads (:811-855)
    hidden = hidden_of("tail_" if cfg.separate_networks else "")
    rel = np.asarray(state["relation_embedding"], np.float64)
    q = np.asarray(queries, np.int64)
    h = (hidden_of("head_") if cfg.separate_networks else hidden)[q[:, 0] * NE + q[:, 1]]
    dot = cfg.score_fn == SCORE["DistMult"] or cfg.distance_fn == DIST["MatMul"]
    r = rel[q[:, 2]]
    if cfg.score_fn == SCORE["RotatE"]:  # src/poplar_kge.cpp:516-530: phases, sine, cosine in float16
        H = D // 2
        th = r[:, :H].astype(np.float32).astype(np.float16)
        sn = np.sin(th.astype(np.float64)).astype(np.float16).astype(np.float64)
        cs = np.cos(th.astype(np.float64)).astype(np.float16).astype(np.float64)
        p = np.concatenate([h[:, :H] * cs - h[:, H:] * sn, h[:, H:] * cs + h[:, :H] * sn], axis=1)
    elif cfg.score_fn == SCORE["ComplEx"]:  # src/poplar_kge.cpp:501-510
        H = D // 2
        p = np.concatenate([h[:, :H] * r[:, :H] - h[:, H:] * r[:, H:],
                            h[:, :H] * r[:, H:] + h[:, H:] * r[:, :H]], axis=1)
    elif cfg.score_fn == SCORE["TransH"]:  # src/poplar_kge.cpp:539-565
        w = np.asarray(state["relation_normal"], np.float64)[q[:, 2]]
        n = w / np.sqrt((w * w).sum(-1, keepdims=True))
        p = h - n * (n * h).sum(-1, keepdims=True) + r
    else:
        p = h * r if cfg.score_fn == SCORE["DistMult"] else h + r
    if cfg.score_fn == SCORE["TransH"]:
        dist = np.stack([np.abs(x[None, :] - (hidden - nn[None, :] * (hidden @ nn)[:, None])).sum(-1)
                         for x, nn in zip(p, n)])
    elif dot:
        dist = p @ hidden.T
    elif cfg.distance_fn == DIST["L1"]:
        dist = np.stack([np.abs(x[None, :] - hidden).sum(-1) for x in p])
    else:
        dist = np.stack([np.sqrt(((x[None, :] - hidden) ** 2).sum(-1)) for x in p])
    score = cfg.gamma - dist if cfg.score_fn in (SCORE["TransE"], SCORE["RotatE"], SCORE["TransH"]) else dist
    live = np.zeros((S, NE), bool)
    for s, n in enumerate(shard_to_count):
        live[s, 1:1 + int(n)] = True
    score = np.where(live.reshape(-1)[None, :], score, -np.inf)
    order = np.argsort(-score, axis=1, kind="stable")[:, :n_best]
    best = np.take_along_axis(score, order, axis=1)
    return np.stack(np.divmod(order, NE), axis=-1), best


def dropout_keep(seed, step, role, key, k, p):
    """The oracle's dropout mask (kge_dropout_keep in kge_oracle.c) on NumPy arrays: True = keep."""
    u = lambda v: np.asarray(v, np.uint64)
    x = (u(key) * 0x9E3779B1 + u(k) * 0x85EBCA77 + u(role) * 0xC2B2AE3D + u(step) * 0x27D4EB2F
         + u(seed) * 0x165667B1) & 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x >= np.uint64(int(np.float64(np.float32(p)) * 4294967296.0))
