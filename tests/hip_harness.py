"""Test plumbing for the HIP library: ctypes bindings of the device ops (torch
supplies device memory only) and helpers that move a whole state dict in and
out of a ``libpoplar_kge.Engine`` through the reference's own commands."""

import ctypes as C
import os
from pathlib import Path

import numpy as np

PKG = Path(__file__).resolve().parent.parent / "distributed-kge-poplar_amd"
LIB_PATH = PKG / "libkge_hip.so"

_lib = None


def lib():
    """The C-ABI library.  Fails loudly if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(f"{LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(os.fspath(LIB_PATH))
        _lib.kge_scatter_add_workspace_bytes.restype = C.c_size_t
        _lib.kge_scatter_add_workspace_bytes.argtypes = [C.c_int64] * 3
    return _lib


def dptr(t):
    return C.c_void_p(t.data_ptr())


def engine_settings(c, n_step, rw_batch=64, **extra):
    """Flattened settings as src/python/poplar_kge.py:487-496 hands them over."""
    loss = {"training.loss.type": c["loss_fn"]}
    if c["loss_fn"] == "softmax":
        loss["training.loss.correction_weight"] = float(c["softmax_correction_weight"])
    s = {
        "seed": 1, "model.seed": int(c.get("dropout_seed") or 1234),
        "model.score_fn": c["score_fn"], "model.distance_fn": c["distance_fn"],
        "model.n_shard": c["n_shard"], "model.n_entity": c["n_entity"],
        "model.n_relation_type": c["n_relation"], "model.embedding_size": c["dim"],
        "model.entity_feature_size": c["feature"], "model.feature_mlp_size": int(c.get("feature_mlp_size", 0)),
        "model.feature_dropout": float(c.get("feature_dropout", 0.0)),
        "model.negative_adversarial_scale": float(c["negative_adversarial_scale"]),
        "model.share_feature_networks": bool(c.get("share_feature_networks", True)), "model.gamma": float(c["gamma"]),
        "model.init_scale": 1.0,
        "data.seed": 5, "data.batch_size": c["batch"], "data.a2a_size": c["a2a"],
        "data.entity_feature_mapping": "full",
        "training.n_step": 100, "training.validation_interval": 50,
        **loss,
        "training.embedding_regularisation.power": float(c.get("embedding_regularisation", (3.0, 0.0))[0]),
        "training.embedding_regularisation.weight": float(c.get("embedding_regularisation", (3.0, 0.0))[1]),
        "training.feature_regularisation.power": float(c.get("feature_regularisation", (3.0, 0.0))[0]),
        "training.feature_regularisation.weight": float(c.get("feature_regularisation", (3.0, 0.0))[1]),
        "training.hidden_regularisation.power": float(c.get("hidden_regularisation", (3.0, 0.0))[0]),
        "training.hidden_regularisation.weight": float(c.get("hidden_regularisation", (3.0, 0.0))[1]),
        "training.learning_rate": 0.1, "training.learning_rate_modifiers": {},
        "training.adam_beta_m": float(c["beta_m"]), "training.adam_beta_v": float(c["beta_v"]),
        "training.adam_epsilon": float(c["epsilon"]),
        "training.weight_decay": float(c["weight_decay"]),
        "training.loss_scale": float(c["loss_scale"]),
        "execution.device": "hip", "execution.dtype": "float32",
        "execution.train_steps_per_program_run": n_step, "execution.rw_batch_size": rw_batch,
        "execution.predict_hr_batch_size": 8, "execution.predict_tail_batch_size": 8,
        "execution.predict_n_best": 4,
        "logging.wandb": False, "logging.steps_per_log": 20,
        "execution.shared_table": bool(c["shared_table"]),
    }
    if c.get("storage") == "bfloat16_embedding":
        s["execution.embedding_dtype"] = "bfloat16"
    if c.get("storage") == "float16":
        s["execution.dtype"] = "float16"
    if c.get("scoring_bf16"):
        s["execution.scoring_dtype"] = "bfloat16"
    s.update(extra)
    return s


def _chunks(c, rw):
    S, NE = c["n_shard"], c["n_entity"]
    for off in range(0, NE, rw):
        idx = np.arange(off, off + rw, dtype=np.uint32)
        idx *= idx < NE  # overflow goes to row 0 (src/python/poplar_kge.py:546-552)
        yield off, np.tile(idx[None], (S, 1))


def load_state(engine, c, state, rw=64):
    """Writes every table row (write_entity_raw) and variable ("write")."""
    S, NE, D, F = c["n_shard"], c["n_entity"], c["dim"], c["feature"]
    ed = state["entity_data"].reshape(-1, NE, 3 * D + F)  # [n_tables, NE, W]
    # descending offsets: the overflow of the last chunk lands on row 0 first
    # and is then overwritten by the real row 0
    for off, idx in reversed(list(_chunks(c, rw))):
        data = np.zeros((S, rw, 3 * D + F), np.float32)
        for s in range(S):
            data[s] = ed[0 if c["shared_table"] else s][idx[s]]
        engine.run("write_entity_raw", dict(write_indices=idx, write_data=data))
    for k, v in state.items():
        if k == "entity_data":
            continue
        if k == "step":
            engine.run("write", dict(name="step", value=np.full(S, v, np.uint32)))
        else:
            engine.run("write", dict(name=k, value=np.ascontiguousarray(v, np.float32)))


def read_state(engine, c, rw=64):
    S, NE, D, F = c["n_shard"], c["n_entity"], c["dim"], c["feature"]
    n_tables = 1 if c["shared_table"] else S
    ed = np.zeros((n_tables, NE, 3 * D + F), np.float32)
    half = c.get("storage") == "float16"   # the read stream carries execution.dtype, float16 as int16 bits
    for off, idx in _chunks(c, rw):
        out = np.zeros((S, rw, 3 * D + F), np.float16 if half else np.float32)
        engine.run("read_entity", dict(read_indices=idx, read_data=out.view(np.int16) if half else out))
        n = min(rw, NE - off)
        ed[:, off:off + n] = out[:n_tables, :n]
    st = {"entity_data": ed.reshape(-1, 3 * D + F)}
    shapes = dict(engine.run("variables", {})["variables"])
    for name, shape in shapes.items():
        if name == "step":
            v = np.zeros(S, np.uint32)
            engine.run("read", dict(name=name, value=v))
            assert len(set(v.tolist())) == 1
            st["step"] = int(v[0])
        elif shape[0] > 0:
            v = np.full(shape, np.nan, np.float32)
            engine.run("read", dict(name=name, value=v))
            st[name] = v
    return st


def train(engine, c, lr, batch):
    S = c["n_shard"]
    loss = np.full(S, np.nan, np.float32)
    lr = np.ascontiguousarray(np.broadcast_to(np.asarray(lr, np.float32), (S,)))
    engine.run("train_step_loop", dict(learning_rate=lr, loss=loss,
                                       **{k: np.ascontiguousarray(v) for k, v in batch.items()}))
    return loss
