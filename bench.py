#!/usr/bin/env python3
"""Throughput of the per-shard KGE training step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]

One "step" is one training step over one batch: gather -> BESS scoring ->
loss forward/backward -> deterministic scatter-add -> sparse Adam write-back.
The index arrays of all W + K steps (fresh ids every step) are resident in HBM
before the timed region, which runs exactly K steps through the engine's
``train_step_loop`` (device plan phase included) and ends with the loss copied
back and the stream synchronised.  Prints ONE JSON line.

Extra objects in that line:
  roofline      the kernel with the largest share of the step time: algorithmic
                bytes or flops per launch over its mean launch duration, measured
                with HIP events on the engine's stream in a second (untimed) pass;
                `traffic` = its HBM-side bytes per launch from the committed counter
                summary named in `traffic_source` (null without one)
  kernels       the same figures for every kernel of the step
  cpu_baseline  the reference's CPU path (its PyTorch demo step: fancy-index gather,
                torch.cdist, autograd, Adam on the gathered rows) on the first steps of
                the same workload, all of this host's threads, a bounded sample
  cpu_baseline_port  the sequential float32 C port of the step (1 thread), ~15 s
  workloads     the same measurement on the 22.8M-row (L2 and L1) and 91.2M-row tables
  host_batches  the same steps with the index arrays handed over as host buffers
                every call (PCIe-inclusive; never the headline value)
  copy_calibration  one plain row copy much larger than the caches, whose known
                size scales the FETCH_SIZE / WRITE_SIZE counters of a profiler run
"""

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
for p in (ROOT, ROOT / "distributed-kge-poplar_amd"):
    sys.path.insert(0, os.fspath(p))

from kge_synthetic import WORKLOADS, init_tables, make_batch, make_settings, read_rows, row_bytes  # noqa: E402

PEAK_HBM_GBPS = 8000.0
PEAK_FP32_TFLOPS = 157.3
PEAK_BF16_TFLOPS = 2500.0

# kernels of the step by the names the profiler summaries list them under
KERNEL_SYMBOLS = {"gather_operands": "k_gather_operands", "score_fwd": "k_score_fwd", "score_bwd": "k_score_bwd",
                  "reduce_entity": "k_reduce_chunks", "adam_entity": "k_adam_rows", "loss_rows": "k_loss_rows"}


def measured_traffic(workload):
    """HBM-side bytes per launch (fetched + written) of every step kernel, read from the committed
    summary of two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE, each scaled
    by what the same counter reads for the calibration copy).  Counters cannot be read from inside
    this process; the summary names the command it came from.  None when there is no summary."""
    path = ROOT / "profiles" / f"{workload}_step_hbm_traffic.md"
    if not path.exists():
        return None, None
    table = {}
    for line in path.read_text().splitlines():
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) in (5, 6) and cells[0].startswith("`"):
            try:
                launches = float(cells[5]) if len(cells) == 6 else 1.0
                table[cells[0].strip("`")] = (launches, (float(cells[3]) + float(cells[4])) * 1e6)
            except ValueError:
                pass
    out = {}
    for name, symbol in KERNEL_SYMBOLS.items():
        hits = [v for k, v in table.items() if symbol in k]
        if hits:
            out[name] = max(hits)[1]  # variants of one kernel (with and without hot rows): the one launched most
    return out, f"profiles/{path.name}"


def cpu_start_state(engine, settings, w, sub):
    """The oracle-side state and configuration for the steps in `sub`, from the device's own
    initial rows (only the rows those steps touch are read back; the rest of the host table
    stays untouched virtual memory)."""
    m, d = settings.model, settings.data
    ids = np.unique(sub["remote"])
    rows = read_rows(engine, settings, ids)
    table = np.zeros((m.n_entity, settings.entity_data_r_size), np.float32)  # untouched pages stay virtual
    table[ids] = rows
    state = {"entity_data": table, "step": 0}
    names = ["relation_embedding"] + (["feature_projection"] if m.entity_feature_size else [])
    for name in names:
        for suffix in ("", "/adam_m", "/adam_v"):
            state[name + suffix] = engine.read_variable(name + suffix)
    softmax = w.get("loss") == "softmax"
    cfg = dict(n_shard=m.n_shard, n_entity=m.n_entity, n_relation=m.n_relation_type,
               dim=m.embedding_size, feature=m.entity_feature_size, batch=d.batch_size, a2a=d.a2a_size,
               score_fn=m.score_fn, distance_fn=m.distance_fn,
               loss_fn="softmax" if softmax else "logsigmoid",
               softmax_correction_weight=1.0 if softmax else 0.0,
               shared_table=True, gamma=m.gamma, loss_scale=settings.training.loss_scale,
               scoring_bf16=settings.execution.scoring_dtype == "bfloat16",
               storage="bfloat16_embedding" if w.get("embedding_dtype") == "bfloat16" else "float32")
    return cfg, state


def cpu_port_prepare(engine, settings, w, batch, n_cpu_steps):
    """The sequential float32 oracle's configuration and start state (the device's own initial
    rows) for the first `n_cpu_steps` steps.  Called before the device runs a step; timed by
    cpu_port_run after the device's timed regions, so that the device is not left idle for the
    oracle's ~15 s right before them."""
    from oracle.kge_oracle import make_cfg

    sub = {k: np.ascontiguousarray(v[:, :n_cpu_steps]) for k, v in vars(batch).items()}
    cfg, state = cpu_start_state(engine, settings, w, sub)
    return make_cfg(**cfg), state, sub


def cpu_port_run(prepared, settings, n_check):
    """Times the oracle on the prepared steps.  The first `n_check` of them are run as a separate
    call so that their mean loss can be compared with the GPU's.  Returns (json object, loss of
    the first call)."""
    from oracle.kge_oracle import Oracle

    cfg, state, sub = prepared
    m, d = settings.model, settings.data
    n_cpu_steps = sub["remote"].shape[1]
    oracle = Oracle("f32")
    lr = settings.training.learning_rate
    t0 = time.perf_counter()
    first = {k: np.ascontiguousarray(v[:, :n_check]) for k, v in sub.items()}
    loss = oracle.train_step_loop(cfg, state, lr, first)
    if n_cpu_steps > n_check:
        rest = {k: np.ascontiguousarray(v[:, n_check:]) for k, v in sub.items()}
        oracle.train_step_loop(cfg, state, lr, rest)
    dt = time.perf_counter() - t0
    triples = n_cpu_steps * m.n_shard * d.batch_size
    return dict(value=triples / dt, unit="triples/s", cores=1, kind="port",
                sample=f"{n_cpu_steps} step(s) of the same workload ({triples} triples) in {dt:.1f} s, "
                       f"sequential float32 C oracle, 1 thread of {os.cpu_count()} host cpus"), loss


def cpu_torch_prepare(engine, settings, w, batch, n_max, threads):
    """The reference's PyTorch CPU path (oracle/torch_demo_step.py: fancy-index gather,
    torch.cdist, autograd, the reference's Adam on the gathered rows) set up on the device's own
    initial rows for the first `n_max` steps of the workload; None for a workload that path does
    not cover.  Called before the device runs a step; timed by cpu_torch_run after the device's
    timed regions, because its worker threads would compete with the thread that launches kernels."""
    from oracle.torch_demo_step import TorchDemoStep

    sub = {k: np.ascontiguousarray(v[:, :n_max]) for k, v in vars(batch).items()}
    cfg, state = cpu_start_state(engine, settings, w, sub)
    try:
        return TorchDemoStep(cfg, state, threads=threads), sub, threads
    except ValueError:
        return None


def cpu_torch_run(prepared, settings, n_check, budget_s=10.0):
    """One untimed step to start the thread pool, then steps until `budget_s` seconds have gone,
    going round the prepared steps as often as that takes (the state keeps evolving; only the
    first pass's losses are compared).  Returns (json object, mean loss of the first n_check steps)."""
    path, sub, threads = prepared
    m, d = settings.model, settings.data
    lr = settings.training.learning_rate
    n_prepared = sub["remote"].shape[1]
    losses, dt, n, i = [], 0.0, 0, 0
    while dt <= budget_s and n < 100000:
        t0 = time.perf_counter()
        loss = path.step(lr, {k: v[:, i % n_prepared] for k, v in sub.items()})
        if i > 0:
            dt += time.perf_counter() - t0
            n += 1
        if i < n_prepared:
            losses.append(loss)
        i += 1
    triples = n * m.n_shard * d.batch_size
    loss = np.mean(losses[:n_check], axis=0) if len(losses) >= n_check else None
    return dict(value=triples / dt, unit="triples/s", cores=threads, kind="port",
                sample=f"{n} step(s) of the same workload ({triples} triples; the first {n_prepared} steps' "
                       f"index arrays, repeated) in {dt:.1f} s after one untimed step, float32 PyTorch demo "
                       f"path, {threads} threads of {os.cpu_count()} host cpus"), loss


def split_forward(w):
    """Whether the forward kernel takes the three-piece bfloat16 path: the engine's default for
    L2 / dot scoring on float32 operands at shapes aligned to its tiles."""
    return (w.get("scoring") in (None, "mfma_bf16x3") and w.get("distance_fn", "L2") != "L1"
            and w.get("scoring_dtype") != "bfloat16"
            and w["batch"] % 128 == 0 and w["tails"] % 64 == 0 and w["dim"] % 64 == 0)


def split_backward(w):
    """The same for the backward kernel (its tiles are 128 rows on either side)."""
    return split_forward(w) and w["tails"] % 128 == 0


# kernels whose working set (a few tens of MB, just written by the kernel before) is served by the
# memory-side caches: their rate is no HBM figure
CACHE_SERVED = ("gather_operands", "reduce_entity")


def kernel_table(w, timing, n_steps, uniq_rows, contributions):
    """Algorithmic bytes / flops per launch and achieved rates of every kernel.  `contributions`:
    gradient rows the sparse update sums per step (heads + the blocks' distinct tails)."""
    K_, B, T, D = w["blocks"], w["batch"], w["tails"], w["dim"]
    R = K_ * (B + T)
    U = float(np.mean(uniq_rows))
    emb_bytes = 2 if w.get("embedding_dtype") == "bfloat16" else 4
    row_state = D * emb_bytes + 2 * D * 4           # emb + m + sqrt v, read and written
    pair_dims = K_ * B * T * D
    work = {
        # flops: 3 per pair-dim forward (sub, abs|mul, add); backward = 2x forward
        "score_fwd": ("flops", 3.0 * pair_dims),
        "score_bwd": ("flops", 6.0 * pair_dims),
        # bytes: contributions in, one summed row out per distinct row
        # one wave per contribution: row in (from the table), float32 operand row out
        "gather_operands": ("bytes", R * D * (emb_bytes + 4)),
        # the two launches below each serve the entity rows and the relation table:
        # contributions in, one summed row out per distinct row; rows read + written
        "reduce_entity": ("bytes", (R + K_ * B) * D * 4 + (U + w["n_relation"]) * D * 4),
        # scatter-add + Adam in one launch: the contributions in (scatter-add's input), the
        # distinct rows in and out, the relation table in and out
        "adam_entity": ("bytes", contributions * D * 4 + U * 2 * row_state + 2 * 3 * w["n_relation"] * D * 4),
        "plan": ("bytes", 4.0 * (R + 2 * K_ * B) + 4 * U),
    }
    F = w.get("feature", 0)
    if F:
        work["hidden_fwd"] = ("flops", 2.0 * U * F * D)
        work["proj_grad"] = ("flops", 2.0 * U * F * D)
        work["loss_rows"] = ("bytes", 2.0 * K_ * B * T * 4)
    if w.get("score_fn") == "DistMult":  # 2 flop per pair-dim forward (mul, add); backward = 2x
        work["score_fwd"] = ("flops", 2.0 * pair_dims)
        work["score_bwd"] = ("flops", 4.0 * pair_dims)
    out = {}
    for name, rec in timing["kernels"].items():
        if rec["calls"] == 0 or name not in work:
            continue
        kind, amount = work[name]
        ms = rec["ms"] / n_steps  # per step (plan: one launch group per call, shared by its steps)
        entry = dict(ms_per_step=ms, launches_per_step=rec["calls"] / n_steps)
        if kind == "bytes":
            entry.update(bound="cache" if name in CACHE_SERVED else "hbm", achieved=amount / (ms * 1e-3) / 1e9,
                         peak=PEAK_HBM_GBPS, unit="GB/s")
        else:
            # the published peak of the instruction the kernel issues: float32 matrix / vector
            # instructions 157.3; bfloat16 matrix instructions 2500, of which the float32-product
            # kernels issue six per product (three-piece operands)
            peak, instr = PEAK_FP32_TFLOPS, "f32"
            if w.get("scoring_dtype") == "bfloat16":
                peak, instr = PEAK_BF16_TFLOPS, "bf16"
            elif (name == "score_fwd" and split_forward(w)) or (name == "score_bwd" and split_backward(w)):
                peak, instr = PEAK_BF16_TFLOPS / 6.0, "bf16 x6 (float32 products)"
            entry.update(bound="mfma", achieved=amount / (ms * 1e-3) / 1e12, peak=peak, unit="TFLOP/s",
                         instructions=instr)
        entry["frac"] = entry["achieved"] / entry["peak"]
        entry["algorithmic_per_step"] = amount
        out[name] = {k: (float(f"{v:.4g}") if isinstance(v, float) else v) for k, v in entry.items()}
    return out


def predict_bench(args, w, kge, torch):
    """`--mode predict`: the all-entity scoring sweep with the running n_best
    (reference src/poplar_kge.cpp:743-855 behind Engine.predict,
    src/python/poplar_kge.py:781-861).  One "step" is one `predict` program
    run: predict_hr_batch_size queries against every row of one shard's table,
    query batch and n_best as in the reference's large configuration
    (src/python/poplar_kge.py:395-397).  Prints one JSON line of its own."""
    Q, n_best = 128, 100
    s = kge.Settings.create_demo()
    s.seed = 20240611
    m, d, e = s.model, s.data, s.execution
    m.score_fn, m.distance_fn = w.get("score_fn", "TransE"), w["distance_fn"]
    m.n_shard, m.n_entity, m.n_relation_type = 1, w["n_entity"], w["n_relation"]
    m.embedding_size, m.entity_feature_size, m.gamma = w["dim"], 0, 10.0
    m.init_scale = float(np.sqrt(w["dim"]))
    d.batch_size, d.a2a_size = 256, 256
    e.device, e.dtype, e.shared_table = "hip", "float32", False
    e.embedding_dtype = w.get("embedding_dtype")
    e.train_steps_per_program_run, e.rw_batch_size = 1, 8192
    e.predict_hr_batch_size, e.predict_n_best = Q, n_best
    e.predict_chunk_rows = args.predict_chunk_rows
    if args.scoring:
        e.scoring = args.scoring
    settings = s.prepare()
    engine = kge.Engine(settings, np.full(1, m.n_entity - 1))
    init_tables(engine, settings)
    rng = np.random.default_rng(7)
    head = rng.integers(1, m.n_entity, (1, Q)).astype(np.uint32)
    relation = rng.integers(0, m.n_relation_type, (1, Q)).astype(np.uint32)
    scores = np.zeros((1, 1, Q, n_best), np.float32)
    rows = np.zeros(scores.shape, np.uint32)
    call = dict(predict_head=head, predict_relation=relation,
                predict_entity_count=np.full(1, m.n_entity - 1, np.uint32),
                predict_scores=scores, predict_indices=rows)
    for _ in range(args.warmup):
        engine.engine.run("predict", call)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        engine.engine.run("predict", call)   # synchronous: the n_best are on the host when it returns
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps

    # check: ranks sorted, rows valid, and every returned score recomputed in float64 from the
    # returned row, the head's row and the relation's (TransE: gamma - |h + r - t|)
    sc, ix = scores[0, 0], rows[0, 0]
    assert np.all(sc[:, :-1] >= sc[:, 1:]) and ix.min() >= 1 and ix.max() < m.n_entity
    D = m.embedding_size
    rel = engine.read_variable("relation_embedding").reshape(-1, D).astype(np.float64)
    nq = 8
    t_rows = read_rows(engine, settings, ix[:nq].reshape(-1))[:, :D].astype(np.float64).reshape(nq, n_best, D)
    h_rows = read_rows(engine, settings, head[0, :nq])[:, :D].astype(np.float64)
    diff = (h_rows + rel[relation[0, :nq]])[:, None, :] - t_rows
    dist = np.sqrt((diff ** 2).sum(-1)) if m.distance_fn == "L2" else np.abs(diff).sum(-1)
    err = float(np.max(np.abs((m.gamma - dist) - sc[:nq]) / np.maximum(1.0, np.abs(sc[:nq]))))
    assert err < 1e-5, err

    # CPU baseline: the same sweep in NumPy float32 over a bounded sample of the table
    # (the product form for L2, |a - b| summed in slabs for L1), one thread
    n_cpu = min(m.n_entity - 1, 200_000 if m.distance_fn == "L2" else 20_000)
    cand = read_rows(engine, settings, np.arange(1, n_cpu + 1, dtype=np.uint32))[:, :D]
    q32 = (read_rows(engine, settings, head[0])[:, :D] + rel[relation[0]].astype(np.float32)).astype(np.float32)
    torch.set_num_threads(1)
    t1 = time.perf_counter()
    if m.distance_fn == "L2":
        d2 = (q32 ** 2).sum(1)[:, None] + (cand ** 2).sum(1)[None, :] - 2.0 * (q32 @ cand.T)
        sc_cpu = m.gamma - np.sqrt(np.maximum(d2, 0.0))
    else:
        sc_cpu = np.stack([m.gamma - np.abs(q[None, :] - cand).sum(1) for q in q32])
    top = np.argpartition(-sc_cpu, n_best, axis=1)[:, :n_best]
    cpu_dt = time.perf_counter() - t1
    del top

    pairs = float(Q) * (m.n_entity - 1)
    flop = 3.0 * pairs * D
    emb_bytes = 2 if w.get("embedding_dtype") == "bfloat16" else 4
    table_bytes = float(m.n_entity - 1) * D * emb_bytes
    # L2 with the default scoring runs as six bfloat16 matrix products per float32 product
    # (12 executed flop per pair-dim, priced against the bfloat16 peak); L1 is float32 vector work
    # (3 flop per pair-dim against the float32 peak)
    pieces = m.distance_fn == "L2" and (args.scoring or "mfma_bf16x3") == "mfma_bf16x3"
    peak = PEAK_BF16_TFLOPS if pieces else PEAK_FP32_TFLOPS
    done = (12.0 if pieces else 3.0) * pairs * D
    frac_flop, frac_hbm = done / dt / 1e12 / peak, table_bytes / dt / 1e9 / PEAK_HBM_GBPS
    roof = (dict(bound="mfma", achieved=done / dt / 1e12, peak=peak, unit="TFLOP/s", frac=frac_flop)
            if frac_flop >= frac_hbm else
            dict(bound="hbm", achieved=table_bytes / dt / 1e9, peak=PEAK_HBM_GBPS, unit="GB/s", frac=frac_hbm))
    roof.update(traffic=None, kernel="predict sweep (score + n_best merge), whole program run",
                launch_ms=dt * 1e3, algorithmic_tflops=flop / dt / 1e12,
                table_read_gbps=table_bytes / dt / 1e9)
    print(json.dumps(dict(
        metric="predict_candidate_scores_per_s", value=pairs / dt, unit="scores/s", n_gpus=1,
        steps=args.steps, warmup=args.warmup, ms_per_step=dt * 1e3, higher_is_better=True,
        scaling="weak", vs_baseline=None, dtype="f32", data="synthetic",
        config=dict(workload=f"predict over {w['desc'].split(',')[0]}, {m.n_entity} rows of one shard, "
                             f"{Q} queries per run, n_best {n_best}"),
        roofline=roof,
        cpu_baseline=dict(value=float(Q) * n_cpu / cpu_dt, unit="scores/s", cores=1, kind="port",
                          sample=f"{Q} queries against the first {n_cpu} rows, NumPy float32, "
                                 f"scores and n_best selection, {cpu_dt:.2f} s"),
        check=dict(recomputed_score_rel_err=err, queries_checked=nq))))


def measure(name, args, kge, torch, full):
    """One workload: W untimed warm-up steps, exactly K timed steps (one `train_step_loop` call over
    index arrays resident in HBM, plan phase included, device idle on both sides), then the same K
    steps once more with an event pair around every kernel.  With `full` also the CPU baselines,
    the stand-alone gather, the calibration copy and the host-buffer variant."""
    w = dict(WORKLOADS[name])
    if args.n_entity and full:
        w["n_entity"] = args.n_entity
        w["desc"] += f" [table size overridden: {args.n_entity}]"
    if args.scoring:
        w["scoring"] = args.scoring
    if args.execution:
        w["execution"] = {k: json.loads(v) for k, v in (kv.split("=", 1) for kv in args.execution)}
    n_total = args.warmup + args.steps
    settings = make_settings(w, n_total, kge)
    m, d = settings.model, settings.data
    batch = make_batch(w, n_total, kge)  # host work first: the device goes from initialisation straight to the steps
    engine = kge.Engine(settings, np.full(m.n_shard, m.n_entity - 1))
    init_tables(engine, settings)
    engine.stage_batch(batch)

    # CPU baselines on the first steps, from the same initial state the GPU starts from.  The C
    # port: about 15 s of work on one core (~2e9 pair-dims per second for the whole step).
    pair_dims = m.n_shard * d.batch_size * settings.n_tail * m.embedding_size
    n_cpu = args.cpu_steps or int(np.clip(round(15 * 2e9 / pair_dims), 1, n_total))
    n_cpu = min(n_cpu, n_total)
    n_check = max(1, min(n_cpu, args.warmup))
    with_cpu = not args.no_cpu and (full or name in args.cpu_workloads)
    port_prepared = cpu_port_prepare(engine, settings, w, batch, n_cpu) if with_cpu and full else None
    # the worker threads this process may use: the host's share for one GPU, not the node's core count
    threads = int(os.environ.get("OMP_NUM_THREADS") or min(16, os.cpu_count()))
    torch_path = cpu_torch_prepare(engine, settings, w, batch, n_total, threads) if with_cpu else None

    # warm-up: W untimed steps; the first n_check of them double as the parity check
    check = None
    done = 0
    if args.warmup > 0:
        first = n_check if with_cpu else args.warmup
        loss, _ = engine.train_step_loop(None, step_begin=0, step_count=first)
        done = first
        if with_cpu:
            check = dict(gpu_loss=loss)
        if args.warmup > done:
            engine.train_step_loop(None, step_begin=done, step_count=args.warmup - done)

    # timed region: exactly K steps, device idle on both sides
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loss, _ = engine.train_step_loop(None, step_begin=args.warmup, step_count=args.steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timing = engine.timing()
    uniq_rows = timing["unique_entity_rows"][args.warmup:args.warmup + args.steps].astype(np.float64)

    # second pass over the same steps with an event pair around every kernel
    engine.train_step_loop(None, step_begin=args.warmup, step_count=args.steps, profile_kernels=True)
    prof = engine.timing()
    # merged tails: how many score columns a block keeps (distinct tail rows), from the plan of the
    # first timed step
    R_all = m.n_shard * settings.n_remote
    contributions, tails_scored = float(R_all), None
    try:
        tc = np.zeros(m.n_shard, np.uint32)
        engine.engine.run("plan_dump", dict(step=args.warmup, tail_count=tc))
        contributions = float(m.n_shard * d.batch_size + tc.sum())
        tails_scored = dict(distinct_per_block=float(tc.mean()), of=int(settings.n_tail))
    except ValueError:
        pass   # the engine scores every tail position for this configuration
    kernels = kernel_table(w, prof, args.steps, uniq_rows, contributions)
    traffic, traffic_source = measured_traffic(name)
    for k, v in kernels.items():
        v["traffic"] = traffic.get(k) if traffic else None
    step_kernels = {k: v for k, v in kernels.items() if k != "plan"}
    dominant = max(step_kernels, key=lambda k: step_kernels[k]["ms_per_step"])
    dom = kernels[dominant]
    roofline = dict(kernel=dominant, bound=dom["bound"], achieved=dom["achieved"], peak=dom["peak"],
                    unit=dom["unit"], frac=dom["frac"], traffic=dom["traffic"], traffic_source=traffic_source,
                    launch_ms=dom["ms_per_step"] / dom["launches_per_step"])

    triples = args.steps * m.n_shard * d.batch_size
    U = float(np.mean(uniq_rows))
    R = m.n_shard * settings.n_remote
    rb = row_bytes(w)
    step_bytes = (U * 2 * rb + 4 * (R + 2 * m.n_shard * d.batch_size) + 4 * U
                  + 2 * 3 * m.n_relation_type * m.embedding_size * 4)
    step_traffic = sum(v for k, v in traffic.items() if k in step_kernels) if traffic else None
    out = {
        "value": triples / dt,
        "unit": "triples/s",
        "ms_per_step": dt / args.steps * 1e3,
        "dtype": ("bf16 scoring operands / f32 accumulate" if w.get("scoring_dtype") == "bfloat16" else
                  "bf16 rows / f32 math" if w.get("embedding_dtype") == "bfloat16" else "f32"),
        "config": {"workload": f"{name}: {w['desc']}; {'uniform' if w.get('uniform') else 'Zipf s=1.1'} ids, "
                               f"{w.get('loss', 'logsigmoid')} loss, "
                               f"Adam lr 1e-3, raw ids de-duplicated on the device",
                   "positives_per_step": m.n_shard * d.batch_size, "row_refs_per_step": R,
                   "unique_rows_per_step": U, "gradient_rows_per_step": contributions,
                   "tail_columns": tails_scored},
        "step_hbm": {"algorithmic_bytes_per_step": step_bytes,
                     "achieved": step_bytes / (dt / args.steps) / 1e9, "unit": "GB/s",
                     "traffic_per_step": step_traffic,
                     "traffic_over_algorithmic": step_traffic / step_bytes if step_traffic else None,
                     "traffic_source": traffic_source},
        "device_ms": {"plan_per_step": timing["plan_ms"] / args.steps,
                      "kernels_per_step": timing["steps_ms"] / args.steps},
        "loss": loss,
        "roofline": roofline,
        "kernels": kernels,
    }
    # the same steps with the index arrays handed over as host buffers, as the reference's
    # interface takes them (checked, re-ordered and uploaded inside the timed call, chunk by chunk
    # beside the device's work): one call over the K timed steps' worth of a fresh W + K step batch
    host_times = []
    for _ in range(3):   # the median of three calls: a single call's host side is at the mercy of the scheduler
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        engine.train_step_loop(batch)
        torch.cuda.synchronize()
        host_times.append((time.perf_counter() - t1) / n_total)
    dt_host = float(np.median(host_times))
    out["host_batches"] = {"value": m.n_shard * d.batch_size / dt_host, "unit": "triples/s",
                           "ms_per_step": dt_host * 1e3, "over_resident": dt_host / (dt / args.steps),
                           "note": f"median of three calls over {n_total} steps each, index arrays checked and "
                                   "uploaded from host memory inside the timed call"}
    if full:
        # stand-alone row gather (fr::Buffer::read) over one step's distinct rows
        ids = np.unique(batch.remote[:, args.warmup]).astype(np.uint32)
        gms = np.zeros(1, np.float32)
        engine.engine.run("gather_benchmark", dict(indices=ids, ms=gms, repeats=20))
        out["row_gather"] = dict(rows=int(ids.size), ms=float(gms[0]),
                                 achieved=2 * ids.size * rb / (gms[0] * 1e-3) / 1e9, unit="GB/s (read + write)",
                                 note="working set of a few tens of MB: served by the caches, not an HBM figure")
        # one large plain copy (distinct rows, > 1 GB each way): scales the profiler's byte counters,
        # and is the HBM bandwidth a plain streaming kernel reaches on this device
        n_cal = min(m.n_entity - 1, 400_000)
        cal_ids = (1 + np.random.default_rng(5).permutation(m.n_entity - 1)[:n_cal]).astype(np.uint32)
        engine.engine.run("gather_benchmark", dict(indices=cal_ids, ms=gms, repeats=1))
        out["copy_calibration"] = dict(kernel="k_rows_copy", rows=int(n_cal), bytes_read=int(n_cal * rb),
                                       bytes_written=int(n_cal * rb), ms=float(gms[0]),
                                       achieved=2 * n_cal * rb / (gms[0] * 1e-3) / 1e9, unit="GB/s (read + write)")
    # the CPU paths last: nothing of this workload's device work is timed after them
    port = None
    if port_prepared is not None:
        port, port_loss = cpu_port_run(port_prepared, settings, n_check)
        if check is not None:
            check.update(cpu_port_loss=float(np.sum(port_loss)),
                         cpu_port_rel_err=abs(check["gpu_loss"] - float(np.sum(port_loss))) / abs(float(np.sum(port_loss))))
    cpu_torch, cpu_torch_loss = (cpu_torch_run(torch_path, settings, n_check, args.cpu_torch_seconds)
                                 if torch_path else (None, None))
    if check is not None and cpu_torch_loss is not None:
        check["cpu_loss"] = float(np.sum(cpu_torch_loss))
        check["cpu_rel_err"] = abs(check["gpu_loss"] - check["cpu_loss"]) / abs(check["cpu_loss"])
    # the reference's own CPU path (PyTorch, all host threads) where it covers the workload; the
    # sequential C port beside it
    out["cpu_baseline"] = cpu_torch if cpu_torch is not None else port
    if with_cpu and full:
        out["cpu_baseline_port"] = port
    if out["cpu_baseline"]:
        out["speedup_over_cpu_baseline"] = out["value"] / out["cpu_baseline"]["value"]
    out["check"] = check
    del engine
    import gc
    gc.collect()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--mode", default="train", choices=["train", "predict"],
                    help="train: the training step (the headline metric); predict: the all-entity scoring sweep")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3l2", choices=sorted(WORKLOADS),
                    help="the headline workload (default c3l2: TransE-L2 D=256 on the 22.8M-row table, the "
                         "configuration the performance target is quoted on)")
    ap.add_argument("--also", default=None,
                    help="comma-separated workloads measured after the headline one and reported under "
                         "`workloads` (default with --workload c3l2: c2,c3,c5,c4 - the 1M-row table, the L1 "
                         "configuration, the 91.2M-row table and the DistMult + feature configuration; "
                         "'none' to skip)")
    ap.add_argument("--cpu-steps", type=int, default=None,
                    help="steps the sequential CPU port times (default: sized for ~15 s)")
    ap.add_argument("--cpu-torch-seconds", type=float, default=8.0, help="time budget of the PyTorch CPU path")
    ap.add_argument("--cpu-workloads", default="",
                    help="workloads of --also that also time the PyTorch CPU path (comma-separated)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--n-entity", type=int, default=None, help="override the table size (experiments)")
    ap.add_argument("--predict-chunk-rows", type=int, default=None,
                    help="--mode predict: tails scored per launch (experiments; default: the engine's)")
    ap.add_argument("--execution", action="append", default=[], metavar="KEY=JSON",
                    help="further execution.* settings, e.g. merge_tails=false (experiments)")
    ap.add_argument("--scoring", default=None, choices=["mfma", "mfma_bf16x3", "valu"], help="scoring kernels (default mfma_bf16x3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU holding one shard's whole table: --gpus must be 1 "
                 "(the step has no collectives; nothing here uses a second GPU)")
    if args.steps < 1 or args.warmup < 0:
        sys.exit("--steps must be >= 1 and --warmup >= 0")
    args.cpu_workloads = [x for x in args.cpu_workloads.split(",") if x]

    import torch  # device discovery only; all device memory is the engine's own

    if not torch.cuda.is_available():
        sys.exit("no HIP device visible")
    import poplar_kge as kge

    if args.mode == "predict":
        w = dict(WORKLOADS[args.workload])
        if args.n_entity:
            w["n_entity"] = args.n_entity
            w["desc"] += f" [table size overridden: {args.n_entity}]"
        if w.get("feature") or w.get("score_fn", "TransE") != "TransE":
            sys.exit("--mode predict covers the TransE workloads without features")
        return predict_bench(args, w, kge, torch)

    also = args.also if args.also is not None else ("c2,c3,c5,c4" if args.workload == "c3l2" and not args.n_entity else "none")
    also = [x for x in also.split(",") if x and x != "none"]
    for x in also:
        if x not in WORKLOADS:
            sys.exit(f"unknown workload '{x}' in --also")

    head = measure(args.workload, args, kge, torch, full=True)
    out = {
        "metric": "train triples/sec (fwd+bwd+sparse Adam) at dim 256; achieved HBM GB/s",
        "value": head.pop("value"),
        "unit": head.pop("unit"),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head.pop("ms_per_step"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head.pop("dtype"),
        "data": "synthetic",
    }
    # the other table sizes, same protocol (W warm-up, K timed steps, kernel pass), one after the other
    extra = {}
    for x in also:
        need = WORKLOADS[x]["n_entity"] * row_bytes(WORKLOADS[x]) + (6 << 30)
        if torch.cuda.mem_get_info()[0] < need:
            extra[x] = {"skipped": f"needs {need >> 30} GiB of free HBM"}
            continue
        extra[x] = measure(x, args, kge, torch, full=False)
    if extra:
        out["workloads"] = extra
    # the headline workload's details behind the other workloads, its workload description, roofline
    # and CPU baseline last: whoever reads only the end of this one long line still sees them
    last = ("config", "roofline", "cpu_baseline", "speedup_over_cpu_baseline")
    out.update({k: v for k, v in head.items() if k not in last})
    out.update({k: head[k] for k in last if k in head})

    def plain(o):  # numpy scalars -> Python numbers
        if isinstance(o, np.generic):
            return o.item()
        raise TypeError(type(o))

    print(json.dumps(out, default=plain))


if __name__ == "__main__":
    main()
