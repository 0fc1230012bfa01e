"""An independent torch-autograd restatement of one training step.

Test infrastructure.  It follows the structure of the reference's own PyTorch
oracle (tests/python/reference_model.py:113-152: gather by ``remote``, heads by
``head``, tails by ``a2a`` then all-to-all as ``transpose(0, 1)``, broadcast
score, weighted logsigmoid) generalised to the distance / score / loss
variants of src/poplar_kge.cpp:469-499, 567-573, 615-660, and uses autograd
for every gradient, so it shares no hand-derived backward with the C oracle.
The optimiser is the reference formula (src/fructose/frnn.cpp:42-90) in
float64 NumPy.  Everything runs in float64.
"""

import numpy as np
import torch as T


def log_sigmoid_clamped(x):
    """src/pag/pag.cpp:888-910, forward and backward as the reference defines them."""

    class Fn(T.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            ctx.save_for_backward(x)
            return T.where(x > -11, -T.log1p(T.exp(-T.clamp(x, min=-11))), x)

        @staticmethod
        def backward(ctx, g):
            (x,) = ctx.saved_tensors
            return g / (1 + T.exp(T.clamp(x, max=11)))

    return Fn.apply(x)


def safe_pow(x, e):
    """pow with the reference's backward, g * e * pow(x, e) / (x + (x == 0)), which is 0 at
    x = 0 where torch's own gives inf or nan (src/pag/pag.cpp:483-503).  Elsewhere the two
    agree, so torch's autograd still checks the formula."""

    class Fn(T.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            y = T.pow(x, e)
            ctx.save_for_backward(x, y)
            return y

        @staticmethod
        def backward(ctx, g):
            x, y = ctx.saved_tensors
            return g * e * y / (x + (x == 0).to(x.dtype))

    return Fn.apply(x)


def lpnorm(a, p):
    """src/poplar_kge.cpp:389-391, per row."""
    return safe_pow(safe_pow(a, p).abs().sum(-1), 1.0 / p)


def round_bf16_ste(x):
    """x rounded to bfloat16 (nearest even) in the forward pass, identity in the
    backward pass: how the bfloat16 scoring mode treats its operands."""
    return x + (x.detach().to(T.float32).to(T.bfloat16).to(T.float64) - x.detach())


def step(cfg, state, lr, batch_step, grads=None):
    """One step in place on ``state`` (float32 arrays); returns loss[S].  ``grads`` (a dict):
    receives autograd's gradients of the step, ``rows`` (distinct table rows, ascending),
    ``entity`` [rows, D] and ``relation`` [n_relation, D].

    cfg: dict(n_shard, n_entity, n_relation, dim, feature, batch, a2a,
    score_fn, distance_fn, loss_fn, shared_table, gamma, beta_m, beta_v,
    epsilon, weight_decay, loss_scale, softmax_correction_weight,
    negative_adversarial_scale).  batch_step: dict of int arrays for ONE step:
    remote[S,B+T], a2a[S,S,A], head/relation/tail[S,B].
    """
    S, NE, D, F = cfg["n_shard"], cfg["n_entity"], cfg["dim"], cfg["feature"]
    B, A = cfg["batch"], cfg["a2a"]
    Tn = S * A
    remote = T.tensor(batch_step["remote"].astype(np.int64))
    a2a = T.tensor(batch_step["a2a"].astype(np.int64))
    head = T.tensor(batch_step["head"].astype(np.int64))
    relation = T.tensor(batch_step["relation"].astype(np.int64))
    tail = T.tensor(batch_step["tail"].astype(np.int64))
    shards = T.arange(S)

    table = T.tensor(state["entity_data"].astype(np.float64))
    base = T.zeros(S, dtype=T.int64) if cfg["shared_table"] else shards * NE
    keys = base[:, None] + remote  # [S, NR] global row ids
    # one leaf per distinct row so that duplicates share a gradient
    uniq, inverse = T.unique(keys.reshape(-1), return_inverse=True)
    emb = table[uniq, :D].clone().requires_grad_(True)
    feat = table[uniq, 3 * D:]
    rel = T.tensor(state["relation_embedding"].astype(np.float64), requires_grad=True)
    params = [emb, rel]
    if cfg["score_fn"] == "TransH":
        normal = T.tensor(state["relation_normal"].astype(np.float64), requires_grad=True)
        params.append(normal)
    # feature networks (src/poplar_kge.cpp:256-273, 439-458): one, or one for a row's use as a
    # head and one for its use as a tail
    prefixes = ("",) if cfg.get("share_feature_networks", True) or not F else ("head_", "tail_")
    nets = {}

    def feature_hidden(prefix):
        if not F:
            return emb
        leaf = lambda n: nets.setdefault(prefix + n, T.tensor(state[prefix + n].astype(np.float64), requires_grad=True))
        proj = leaf("feature_projection")
        if cfg.get("scoring_bf16"):
            return emb + round_bf16_ste(feat) @ round_bf16_ste(proj)
        if cfg.get("feature_mlp_size"):
            # :453-458; max(x, 0) whose gradient passes where input == output, so also at exactly 0
            # (src/pag/pag.cpp:650-658), which `where` reproduces
            pre = T.cat([emb, feat @ proj], 1) @ leaf("mlp_up_projection")
            return emb + T.where(pre >= 0, pre, T.zeros_like(pre)) @ leaf("mlp_down_projection")
        return emb + feat @ proj

    hidden_u = feature_hidden(prefixes[0])
    hidden_tail_u = feature_hidden(prefixes[-1]) if len(prefixes) == 2 else hidden_u
    drop = cfg.get("feature_dropout", 0.0)
    if F and drop > 0:
        # src/poplar_kge.cpp:459-461, src/pag/pag.cpp:596-617: keep mask / (1 - p) on the feature part,
        # drawn once for the rows' use as heads and once for their use as tails (the oracle's hash
        # stands in for the device's random stream); the backward passes where the OUTPUT is
        # non-zero, which differs from the mask where a kept input is exactly 0
        from oracle.kge_oracle import dropout_keep
        cols = np.arange(D)[None, :]

        def dropped(role, hid):
            fh = hid - emb
            keep = dropout_keep(cfg.get("dropout_seed", 0), int(state["step"]), role, uniq.numpy()[:, None], cols,
                                drop)
            live = T.tensor(keep) & (fh.detach() != 0)
            return emb + fh * live.to(T.float64) / (1 - float(np.float32(drop)))

        hidden_u, hidden_tail_u = dropped(0, hidden_u), dropped(1, hidden_tail_u)
    hidden = hidden_u[inverse].reshape(S, -1, D)  # [S, NR, D]
    hidden_tail = hidden_tail_u[inverse].reshape(S, -1, D)
    # norm regularisers over every gathered slot, once for the heads' and once for the tails'
    # entityHidden call (src/poplar_kge.cpp:463-465, 676-678)
    reg = T.zeros(S, dtype=T.float64)
    value = emb[inverse].reshape(S, -1, D)
    for hid in (hidden, hidden_tail):  # the two calls (the same tensors unless dropout / separate networks)
        for key, tensor in (("embedding_regularisation", value), ("feature_regularisation", hid - value),
                            ("hidden_regularisation", hid)):
            power, weight = cfg.get(key, (3.0, 0.0))
            if weight > 0:
                reg = reg + weight * lpnorm(tensor, float(power)).sum(-1)

    heads = hidden[shards[:, None], head]  # [S, B, D]
    tails = hidden_tail[shards[:, None, None], a2a]  # [S(src), S(dst), A, D]
    tails = tails.transpose(0, 1).reshape(S, Tn, D)  # all-to-all
    r = rel[relation]
    if cfg["score_fn"] == "TransH":
        # src/poplar_kge.cpp:539-565 as written there: unit normal, head and tails projected
        # onto the relation's hyperplane, L1 distance
        n = normal[relation]
        n = n / T.sqrt((n * n).sum(-1, keepdim=True))
        pred = heads - n * (n * heads).sum(-1, keepdim=True) + r
        tails_norm = n @ tails.transpose(1, 2)  # [S, B, T]
        projected = tails[:, None, :, :] - n[:, :, None, :] * tails_norm[..., None]
        score = cfg["gamma"] - (pred[:, :, None, :] - projected).abs().sum(-1)
    elif cfg["score_fn"] in ("TransE", "ComplEx", "RotatE"):
        if cfg["score_fn"] == "RotatE":
            # the phases, their sine and cosine and the phases' gradient in float16 (torch's own
            # float16 kernels and autograd), the rotation in float64
            theta = r.to(T.float32).to(T.float16)
            sn, cs = T.sin(theta).to(T.float64), T.cos(theta).to(T.float64)
            h_re, h_im = heads[..., :D // 2], heads[..., D // 2:]
            pred = T.cat([h_re * cs - h_im * sn, h_im * cs + h_re * sn], -1)
        elif cfg["score_fn"] == "ComplEx":  # complex product on (real | imaginary) halves
            hc = T.complex(heads[..., :D // 2], heads[..., D // 2:]) * T.complex(r[..., :D // 2], r[..., D // 2:])
            pred = T.cat([hc.real, hc.imag], -1)
        else:
            pred = heads + r
        if cfg["distance_fn"] == "L1":
            dist = (pred[:, :, None, :] - tails[:, None, :, :]).abs().sum(-1)
        elif cfg["distance_fn"] == "L2":
            diff = pred[:, :, None, :] - tails[:, None, :, :]
            sq = (diff * diff).sum(-1)
            # the reference's L2 gradient is 0 at zero distance
            safe = T.where(sq > 0, sq, T.ones_like(sq))
            dist = T.where(sq > 0, T.sqrt(safe), T.zeros_like(sq))
        else:
            dist = pred @ tails.transpose(1, 2)
        score = dist if cfg["score_fn"] == "ComplEx" else cfg["gamma"] - dist
    else:
        pred = heads * r
        if cfg.get("scoring_bf16"):
            pred, tails = round_bf16_ste(pred), round_bf16_ste(tails)
        score = pred @ tails.transpose(1, 2)

    onehot = T.nn.functional.one_hot(tail, Tn).to(T.float64)
    if cfg["loss_fn"] == "logsigmoid":
        w_pos, w_neg = 0.5 * Tn, 0.5 * Tn / (Tn - 1)
        weight = onehot * (w_pos - w_neg) + w_neg
        adv = cfg.get("negative_adversarial_scale", 0.0)
        if adv > 0:
            sm = T.softmax(adv * score.detach() - 10000.0 * onehot, dim=-1)
            weight = weight * (onehot + (Tn - 1) * sm)
        per_shard = -(weight * log_sigmoid_clamped((2 * onehot - 1) * score)).sum((1, 2)) / (
            S * B * A * S)
    else:
        cw = cfg.get("softmax_correction_weight", 0.0)
        corr = cw * np.float32(np.log(NE * S - 1) - np.log(S * A - 1)) if cw else 0.0
        z = score + float(corr) * (1 - onehot)
        per_shard = -(T.log_softmax(z, -1) * onehot).sum((1, 2)) / (S * B)
    per_shard = per_shard + reg  # src/poplar_kge.cpp:688
    per_shard.sum().backward(T.tensor(float(cfg["loss_scale"]), dtype=T.float64))

    # optimiser (float64 restatement of frnn.cpp:42-90)
    state["step"] = int(state["step"]) + 1
    st = state["step"]
    # the hyper-parameters are float32 constants in the reference
    bm, bv, eps, wd = (float(np.float32(cfg[k]))
                       for k in ("beta_m", "beta_v", "epsilon", "weight_decay"))
    lr = np.broadcast_to(np.asarray(lr, np.float64), (S,))
    alpha = lr * np.sqrt(1 - bv**st) / (1 - bm**st)

    def adam(p, m, v, g, a):
        m[...] = bm * m + (1 - bm) * g
        v[...] = bv * v + (1 - bv) * g * g
        p[...] = p - a * (m / (np.sqrt(v) + eps) + wd * p)

    g = emb.grad.numpy()
    rows = uniq.numpy()
    if grads is not None:
        grads.update(rows=rows.copy(), entity=g.copy(), relation=rel.grad.numpy().copy())
    ed = state["entity_data"]
    p = ed[rows, :D].astype(np.float64)
    m = ed[rows, D:2 * D].astype(np.float64)
    v = ed[rows, 2 * D:3 * D].astype(np.float64) ** 2
    a_rows = alpha[0] if cfg["shared_table"] else alpha[rows // NE][:, None]
    adam(p, m, v, g, a_rows)
    ed[rows, :D] = p
    ed[rows, D:2 * D] = m
    ed[rows, 2 * D:3 * D] = np.sqrt(v)

    def dense(name, grad):
        n = state[name].shape[0]
        a = alpha[0] if cfg["shared_table"] else alpha[np.arange(n) // (n // S)][:, None]
        p = state[name].astype(np.float64)
        m = state[name + "/adam_m"].astype(np.float64)
        v = state[name + "/adam_v"].astype(np.float64)
        adam(p, m, v, grad, a)
        state[name][...] = p
        state[name + "/adam_m"][...] = m
        state[name + "/adam_v"][...] = v

    dense("relation_embedding", rel.grad.numpy())
    if cfg["score_fn"] == "TransH":
        dense("relation_normal", normal.grad.numpy())
    for name, leaf in nets.items():
        dense(name, leaf.grad.numpy())
    return per_shard.detach().numpy().astype(np.float32)
