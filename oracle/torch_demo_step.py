"""The reference's PyTorch CPU path for one training step, as a timing baseline.

Test and benchmark infrastructure, not part of the product: only the tests and
the benchmark's CPU-baseline leg may import it.

Structure of the reference's demo (doc/pytorch_demo/kge_training.py:353-380:
fancy-index gather of heads and tails, the all-to-all as ``permute(1, 0, 2, 3)``,
``torch.cdist`` for the distance, :211-221; ``loss.backward()`` then an
optimiser step, :521-542), with the pieces the demo does not have taken from
the reference's own PyTorch oracle and C++:

* TransE score ``gamma - dist(h + r, t)`` with L1 or L2 distance
  (src/poplar_kge.cpp:469-499) instead of the demo's L1 only;
* the weighted logsigmoid loss of tests/python/reference_model.py:126-152
  (``torch.nn.functional.logsigmoid``, as that oracle uses; it differs from the
  device's clamped form by at most 1.7e-5 beyond |z| > 11);
* the reference's Adam (src/fructose/frnn.cpp:42-90: bias correction folded into
  the step size, ``sqrt(v) + eps``, ``sqrt(v)`` stored) applied to the gathered
  distinct rows only, as src/poplar_kge.cpp:695-703 does, instead of the demo's
  dense ``AdamW`` over the whole table, which is meaningless on a 70 GB table.

Everything is float32 torch on all host threads.  Pinned by
tests/test_oracle_torch_demo.py against the sequential C oracle on seeded steps.
"""

import numpy as np
import torch as T


class TorchDemoStep:
    """cfg: the keyword arguments of kge_oracle.make_cfg, as a dict; state: the C
    oracle's state dict (float32 arrays, updated in place)."""

    def __init__(self, cfg, state, threads=None):
        if cfg["score_fn"] != "TransE" or cfg["loss_fn"] != "logsigmoid" or cfg["feature"]:
            raise ValueError("the PyTorch demo path covers TransE with the logsigmoid loss and no features")
        if cfg.get("storage", "float32") not in ("float32", "bfloat16_embedding"):
            raise ValueError("float32 rows, or bfloat16 embeddings with float32 moments")
        if threads:
            T.set_num_threads(threads)
        # make_cfg's defaults for what the caller leaves out
        cfg = {**dict(shared_table=False, storage="float32", beta_m=0.9, beta_v=0.999, epsilon=1e-8,
                      weight_decay=0.0), **cfg}
        if cfg.get("loss_scale") is None:
            cfg["loss_scale"] = float(cfg["batch"] * cfg["n_shard"] * cfg["a2a"])
        self.cfg, self.state = cfg, state
        self.table = T.from_numpy(state["entity_data"])  # shares the array's memory
        self.rel = [T.from_numpy(state["relation_embedding" + s]) for s in ("", "/adam_m", "/adam_v")]
        self.p = {"L1": 1.0, "L2": 2.0}[cfg["distance_fn"]]
        self.bf16_rows = cfg.get("storage") == "bfloat16_embedding"

    def _adam(self, p, m, v, g, alpha):
        c = self.cfg
        bm, bv = float(np.float32(c["beta_m"])), float(np.float32(c["beta_v"]))
        m.mul_(bm).add_(g, alpha=1 - bm)
        v.mul_(bv).addcmul_(g, g, value=1 - bv)
        upd = m / (v.sqrt() + float(np.float32(c["epsilon"])))
        if c["weight_decay"]:
            upd.add_(p, alpha=float(np.float32(c["weight_decay"])))
        p.sub_(alpha * upd)

    def step(self, lr, b):
        """b: one step's index arrays remote[S, B+T], a2a[S, S, A], head / relation / tail[S, B].
        Returns loss[S]."""
        c = self.cfg
        S, NE, D, B, A = c["n_shard"], c["n_entity"], c["dim"], c["batch"], c["a2a"]
        Tn = S * A
        remote, a2a, head, relation, tail = (T.from_numpy(np.asarray(b[k]).astype(np.int64))
                                             for k in ("remote", "a2a", "head", "relation", "tail"))
        shards = T.arange(S)
        keys = remote if c["shared_table"] else remote + (shards * NE)[:, None]
        uniq, inverse = T.unique(keys.reshape(-1), return_inverse=True)
        rows = self.table[uniq]  # the gather: distinct stacked rows [U, 3D]
        emb = rows[:, :D].clone().requires_grad_(True)
        rel = self.rel[0].clone().requires_grad_(True)
        hidden = emb[inverse].view(S, -1, D)
        heads = hidden[shards[:, None], head]
        tails = hidden[shards[:, None, None], a2a].permute(1, 0, 2, 3).reshape(S, Tn, D)
        score = c["gamma"] - T.cdist(heads + rel[relation], tails, p=self.p)
        onehot = T.nn.functional.one_hot(tail, Tn).to(T.float32)
        w_pos, w_neg = 0.5 * Tn, 0.5 * Tn / (Tn - 1)
        weight = onehot * (w_pos - w_neg) + w_neg
        loss = -(weight * T.nn.functional.logsigmoid((2 * onehot - 1) * score)).sum((1, 2)) / (S * B * A * S)
        loss.sum().backward(T.tensor(float(c["loss_scale"])))

        self.state["step"] = st = int(self.state["step"]) + 1
        bm, bv = float(np.float32(c["beta_m"])), float(np.float32(c["beta_v"]))
        lr = np.broadcast_to(np.asarray(lr, np.float64), (S,))
        if np.any(lr != lr[0]):
            raise ValueError("one learning rate for all shards")
        alpha = float(lr[0] * np.sqrt(1 - bv**st) / (1 - bm**st))
        with T.no_grad():
            p, m = emb.detach(), rows[:, D:2 * D]
            v = rows[:, 2 * D:3 * D].square()
            self._adam(p, m, v, emb.grad, alpha)
            if self.bf16_rows:
                p = p.to(T.bfloat16).to(T.float32)
            self.table[uniq] = T.cat([p, m, v.sqrt()], 1)  # the write-back
            self._adam(self.rel[0], self.rel[1], self.rel[2], rel.grad, alpha)
        return loss.detach().numpy()

    def train_step_loop(self, lr, batch):
        """batch: arrays with a step axis after the shard axis (remote[S, n_step, ...]);
        returns the mean loss per shard like the device's train_step_loop."""
        n_step = batch["remote"].shape[1]
        total = np.zeros(self.cfg["n_shard"], np.float64)
        for i in range(n_step):
            total += self.step(lr, {k: v[:, i] for k, v in batch.items()})
        return (total / n_step).astype(np.float32)
