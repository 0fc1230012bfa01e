"""Host-side driver of the MI355X KGE training step.

This module plays the part ``src/python/poplar_kge.py`` plays in
graphcore/distributed-kge-poplar: a settings tree that flattens to the dotted
keys the native engine reads (reference :36-278), the ``Batch`` layout contract
(:416-433) and an ``Engine`` wrapper with initialisation, variable / entity
read-write and ``train_step_loop`` including the host learning-rate schedule
(:471-777).  It is written against ``libpoplar_kge`` from this package, whose
``Engine(settings, gp_folder)`` / ``run(command, data)`` keep the reference's
signatures, so a script written for the reference (scripts/run_training.py)
drives it with ``execution.device = "hip"``.

Additions that the reference does not have are marked "additive".
"""

import dataclasses
from pathlib import Path
from typing import Any, Callable, Dict, Optional, Tuple, Union

import numpy as np

import libpoplar_kge

Shape = Tuple[int, ...]


def _record(cls_name: str, spec: str, /, **defaults: Any) -> type:
    """A plain mutable dataclass from a 'field:type' spec string."""
    fields = []
    for item in spec.split():
        fname, _, ftype = item.partition(":")
        entry = (fname, {"int": int, "float": float, "str": str, "bool": bool}.get(ftype, Any))
        if fname in defaults:
            entry += (dataclasses.field(default=defaults[fname]),)
        fields.append(entry)
    return dataclasses.make_dataclass(cls_name, fields)


# The settings tree.  Field names and nesting are the engine's dotted keys
# (src/poplar_kge.cpp:198-236); n_entity, batch_size, a2a_size and the rw /
# predict sizes are per shard.
ModelSettings = _record(
    "ModelSettings",
    "seed:int score_fn:str distance_fn:str n_shard:int n_entity:int n_relation_type:int "
    "embedding_size:int entity_feature_size:int feature_mlp_size:int feature_dropout:float "
    "negative_adversarial_scale:float share_feature_networks:bool gamma:float init_scale:float")
WikiKg90Mv2Settings = _record("WikiKg90Mv2Settings", "name:str", name="wikikg90mv2")
GeneratedDataSettings = _record("GeneratedDataSettings", "n_train:int n_eval:int seed:int name:str",
                                name="generated")
CubicRootRelationSampling = _record("CubicRootRelationSampling", "type:str", type="cubic_root")
DataSettings = _record(
    "DataSettings",
    "seed:int dataset batch_size:int a2a_size:int entity_feature_mapping:str sampling_strategy")
LinearLearningRateDecay = _record("LinearLearningRateDecay", "type:str", type="linear")
SteppedLearningRateDecay = _record("SteppedLearningRateDecay", "step:int multiplier:float type:str",
                                   type="stepped")
ExponentialLearningRateDecay = _record("ExponentialLearningRateDecay", "half_life_steps:int type:str",
                                       type="exponential")
LogSigmoidLoss = _record("LogSigmoidLoss", "type:str", type="logsigmoid")
SoftmaxLoss = _record("SoftmaxLoss", "correction_weight:float type:str", type="softmax")
NormRegularisation = _record("NormRegularisation", "power:float weight:float")
TrainingSettings = _record(
    "TrainingSettings",
    "n_step:int validation_interval:int loss embedding_regularisation feature_regularisation "
    "hidden_regularisation learning_rate:float learning_rate_decay learning_rate_modifiers "
    "adam_beta_m:float adam_beta_v:float adam_epsilon:float weight_decay:float loss_scale:float")
# additive fields: shared_table, embedding_dtype, feature_dtype, profile_kernels, scoring, scoring_dtype,
# predict_chunk_rows, merge_tails, keep_gradients
ExecutionSettings = _record(
    "ExecutionSettings",
    "device:str dtype:str train_steps_per_program_run:int rw_batch_size:int "
    "predict_hr_batch_size:int predict_tail_batch_size:int predict_n_best:int shared_table:bool "
    "embedding_dtype feature_dtype profile_kernels:bool scoring scoring_dtype predict_chunk_rows "
    "merge_tails keep_gradients",
    shared_table=False, embedding_dtype=None, feature_dtype=None, profile_kernels=False, scoring=None,
    scoring_dtype=None, predict_chunk_rows=None, merge_tails=None, keep_gradients=None)
LogSettings = _record("LogSettings", "path wandb:bool steps_per_log:int predict_at")

CODE_CHANGES: Tuple[str, ...] = ("HIP-device",)


@dataclasses.dataclass
class Settings:
    seed: int
    model: Any
    data: Any
    training: Any
    execution: Any
    logging: Any
    code_changes: Tuple[str, ...] = CODE_CHANGES

    # derived sizes ---------------------------------------------------------
    @property
    def program_runs_per_log(self) -> int:
        return -(-self.logging.steps_per_log // self.execution.train_steps_per_program_run)

    @property
    def logs_per_training_run(self) -> int:
        per_log = self.execution.train_steps_per_program_run * self.program_runs_per_log
        return -(-self.training.n_step // per_log)

    @property
    def logs_per_validation(self) -> int:
        per_log = self.execution.train_steps_per_program_run * self.program_runs_per_log
        return -(-self.training.validation_interval // per_log)

    @property
    def n_tail(self) -> int:
        return self.model.n_shard * self.data.a2a_size

    @property
    def n_remote(self) -> int:
        return self.data.batch_size + self.n_tail

    @property
    def entity_data_r_size(self) -> int:
        return 3 * self.model.embedding_size + self.model.entity_feature_size

    @property
    def entity_data_r_shape(self) -> Shape:
        return (self.model.n_shard, self.execution.rw_batch_size, self.entity_data_r_size)

    @property
    def entity_data_w_shape(self) -> Shape:
        return (self.model.n_shard, self.execution.rw_batch_size, self.model.entity_feature_size)

    @property
    def predict_at_log(self) -> set:
        per_log = self.execution.train_steps_per_program_run * self.program_runs_per_log
        return {int(round(t * self.training.n_step / per_log)) for t in self.logging.predict_at}

    @property
    def relation_embedding_size(self) -> int:
        half = self.model.score_fn == "RotatE"
        return self.model.embedding_size // 2 if half else self.model.embedding_size

    # seeds and defaults ------------------------------------------------------
    def prepare(self) -> "Settings":
        """Fill in unset seeds (spawned from ``seed``) and the default loss
        scale batch_size * n_shard * a2a_size (reference :241-263)."""
        if self.seed is None:
            self.seed = int(np.random.randint(1 << 30))
        spawned = [int(s.generate_state(1)[0]) for s in np.random.SeedSequence(self.seed).spawn(3)]
        if self.model.seed is None:
            self.model.seed = spawned[0]
        if self.data.seed is None:
            self.data.seed = spawned[1]
        dataset = self.data.dataset
        if isinstance(dataset, GeneratedDataSettings) and dataset.seed is None:
            dataset.seed = spawned[2]
        if isinstance(self.logging.path, str):
            self.logging.path = Path(self.logging.path)
        if self.training.loss_scale is None:
            self.training.loss_scale = float(self.data.batch_size * self.n_tail)
        return self

    def flatten(self) -> Dict[str, Any]:
        """{'model.n_shard': 16, ...}: every leaf under its dotted path."""
        out: Dict[str, Any] = {}

        def walk(node: Any, path: Tuple[str, ...]) -> None:
            if dataclasses.is_dataclass(node):
                for key, child in vars(node).items():
                    walk(child, path + (key,))
            else:
                out[".".join(path)] = node

        walk(self, ())
        return out

    # presets ---------------------------------------------------------------
    @classmethod
    def _preset(cls, model: Dict[str, Any], data: Dict[str, Any], training: Dict[str, Any],
                execution: Dict[str, Any], logging: Dict[str, Any]) -> "Settings":
        no_reg = lambda: NormRegularisation(power=3.0, weight=0.0)  # noqa: E731
        training = dict(dict(
            embedding_regularisation=no_reg(), feature_regularisation=no_reg(),
            hidden_regularisation=no_reg(), learning_rate_modifiers={}, adam_beta_m=0.9,
            adam_beta_v=0.999, adam_epsilon=1e-8, weight_decay=0.0, loss_scale=None), **training)
        model = dict(dict(seed=None, feature_mlp_size=0, feature_dropout=0.0,
                          negative_adversarial_scale=0.0, share_feature_networks=True,
                          init_scale=1.0), **model)
        data = dict(dict(seed=None, entity_feature_mapping="full",
                         sampling_strategy=CubicRootRelationSampling()), **data)
        return cls(seed=None, model=ModelSettings(**model), data=DataSettings(**data),
                   training=TrainingSettings(**training), execution=ExecutionSettings(**execution),
                   logging=LogSettings(**logging))

    @classmethod
    def create_demo(cls) -> "Settings":
        """The small TransE-L1 preset the reference tests run (reference :280-343)."""
        return cls._preset(
            model=dict(score_fn="TransE", distance_fn="L1", n_shard=2, n_entity=90,
                       n_relation_type=12, embedding_size=8, entity_feature_size=6, gamma=2.0),
            data=dict(batch_size=6, a2a_size=5,
                      dataset=GeneratedDataSettings(n_train=50, n_eval=50, seed=None)),
            training=dict(n_step=100, validation_interval=50, loss=LogSigmoidLoss(),
                          learning_rate=0.1, learning_rate_decay=None),
            execution=dict(device="hip", dtype="float32", train_steps_per_program_run=5,
                           rw_batch_size=50, predict_hr_batch_size=30, predict_tail_batch_size=50,
                           predict_n_best=11),
            logging=dict(path=None, wandb=False, steps_per_log=20, predict_at=(0.5,)))

    @classmethod
    def create_wikikg90mv2(cls) -> "Settings":
        """WikiKG90Mv2 over 16 shards (reference :345-405); the HIP device keeps
        float32 optimiser state, so the table dtype here is float32 with a
        float16 feature block."""
        n_shard = 16
        settings = cls._preset(
            model=dict(score_fn="TransE", distance_fn="L1", n_shard=n_shard,
                       n_entity=int(np.ceil(91230610 / n_shard) + 1),
                       n_relation_type=int(n_shard * np.ceil(1387 / n_shard)), embedding_size=256,
                       entity_feature_size=768, gamma=10.0),
            data=dict(batch_size=512, a2a_size=96, dataset=WikiKg90Mv2Settings()),
            training=dict(n_step=int(5e6), validation_interval=int(2.5e5),
                          loss=SoftmaxLoss(correction_weight=1.0), learning_rate=1e-3,
                          learning_rate_decay=LinearLearningRateDecay(),
                          feature_regularisation=NormRegularisation(power=3.0, weight=1e-6)),
            execution=dict(device="hip", dtype="float32", feature_dtype="float16",
                           train_steps_per_program_run=20, rw_batch_size=512,
                           predict_hr_batch_size=128, predict_tail_batch_size=1024,
                           predict_n_best=100),
            logging=dict(path=None, wandb=True, steps_per_log=int(1e3), predict_at=(0.8, 0.9)))
        return settings

    @classmethod
    def create_wikikg90mv2_short(cls) -> "Settings":
        settings = cls.create_wikikg90mv2()
        settings.data.batch_size, settings.data.a2a_size = 256, 32
        settings.execution.train_steps_per_program_run = 100
        return settings


@dataclasses.dataclass
class Batch:
    """Index arrays of ``train_steps_per_program_run`` steps (reference :416-433).

    remote   uint32[n_shard, steps, batch_size + n_shard*a2a_size]  table rows to gather;
             0 is the padding row.  The reference requires them distinct within a
             shard; this engine also accepts repeats (it de-duplicates on the device).
    a2a      uint32[n_shard, steps, n_shard, a2a_size]  slots of ``remote`` sent to each shard
    head     uint32[n_shard, steps, batch_size]         slots of ``remote``
    relation uint32[n_shard, steps, batch_size]
    tail     uint32[n_shard, steps, batch_size]         position of the true tail among the
             n_shard*a2a_size tails the shard receives (sender-major)
    """

    remote: np.ndarray
    a2a: np.ndarray
    head: np.ndarray
    relation: np.ndarray
    tail: np.ndarray


@dataclasses.dataclass
class Predictions:
    """Best tails per query, as (shard, row) pairs (reference :435-470).

    shard_idx  uint32[..., n_best, 2]
    score      float32[..., n_best]
    """

    shard_idx: np.ndarray
    score: np.ndarray

    def _take(self, order: np.ndarray) -> "Predictions":
        # order: int[..., k] positions along the n_best axis
        return Predictions(shard_idx=np.take_along_axis(self.shard_idx, order[..., None], axis=-2),
                           score=np.take_along_axis(self.score, order, axis=-1))

    def topk(self, k: int) -> "Predictions":
        """The k best of every item, in no particular order."""
        return self._take(np.argpartition(self.score, -k, axis=-1)[..., -k:])

    def sort(self) -> "Predictions":
        """Every item's predictions by descending score."""
        return self._take(np.argsort(self.score, axis=-1)[..., ::-1])


KERNEL_NAMES = ("plan", "hidden_fwd", "gather_operands", "score_fwd", "loss_rows", "score_bwd", "reduce_entity",
                "adam_entity", "reduce_relation", "adam_relation", "proj_grad", "adam_proj")


class Engine:
    """Owns one native engine: tables in HBM, variables, and the step."""

    def __init__(self, settings: Settings, shard_to_entity_count: np.ndarray):
        """shard_to_entity_count: int[n_shard], real entities per shard (padding excluded)."""
        m = settings.model
        if shard_to_entity_count.shape != (m.n_shard,):
            raise ValueError("shard_to_entity_count must have shape (n_shard,)")
        if not np.all(shard_to_entity_count < m.n_entity):
            raise ValueError("shard_to_entity_count must be < model.n_entity (row 0 is padding)")
        self.settings = settings
        self.shard_to_entity_count = shard_to_entity_count
        self.random = np.random.RandomState(m.seed)
        flat = {k: v for k, v in settings.flatten().items()
                if v is not None and k not in ("logging.path", "logging.predict_at", "code_changes")}
        self.engine = libpoplar_kge.Engine(flat, gp_folder=str(Path(libpoplar_kge.__file__).parent))
        self.variable_to_shape = {n: tuple(s) for n, s in self.engine.run("variables", {})["variables"]}
        self.variable_to_dtype = {n: np.dtype("uint32" if n == "step" else "float32")
                                  for n in self.variable_to_shape}
        self.uninitialized_variables = set(self.variable_to_shape)
        self.uninitialized_entity_data = np.full(m.n_entity, True)
        self.entity_data_initialized = False
        self.init_scale = m.init_scale / m.embedding_size
        self.step = 0
        self.current_learning_rate = settings.training.learning_rate
        decay = settings.training.learning_rate_decay
        if isinstance(decay, SteppedLearningRateDecay):
            self.decay_step = float(decay.step)

    # ---- variables ---------------------------------------------------------
    @staticmethod
    def _check_shape(name: str, array: np.ndarray, expected: Shape) -> None:
        if array.shape != tuple(expected):
            raise ValueError(f"'{name}' has incorrect shape, expected {expected}, actual {array.shape}")

    def write_variable(self, name: str,
                       value_or_fn: Union[np.ndarray, Callable[[Shape], np.ndarray]]) -> None:
        shape = self.variable_to_shape[name]
        value = value_or_fn if isinstance(value_or_fn, np.ndarray) else value_or_fn(shape)
        self._check_shape(f"write({name})", value, shape)
        value = np.ascontiguousarray(value, dtype=self.variable_to_dtype[name])
        self.engine.run("write", dict(name=name, value=value))
        self.uninitialized_variables.discard(name)

    def read_variable(self, name: str) -> np.ndarray:
        dtype = self.variable_to_dtype[name]
        value = np.full(self.variable_to_shape[name], np.nan if dtype.kind == "f" else 0, dtype=dtype)
        self.engine.run("read", dict(name=name, value=value))
        return value

    # ---- entity rows ---------------------------------------------------------
    def _rw_indices(self, offset: int) -> np.ndarray:
        m = self.settings.model
        idx = np.arange(offset, offset + self.settings.execution.rw_batch_size, dtype=np.uint32)
        idx[idx >= m.n_entity] = 0  # the overflow of the last chunk goes to the padding row
        return np.ascontiguousarray(np.broadcast_to(idx, (m.n_shard, idx.size)))

    @staticmethod
    def _int16_if_float16(array: np.ndarray) -> np.ndarray:
        return array.view(np.int16) if array.dtype == np.float16 else array

    def write_entity(self, offset: int, data: np.ndarray) -> None:
        """Initialise rows [offset, offset + rw_batch_size): random-normal
        embedding, zero moments, ``data`` as the feature block."""
        self._check_shape("write_entity(data)", data, self.settings.entity_data_w_shape)
        idx = self._rw_indices(offset)
        self.engine.run("write_entity", dict(
            write_indices=idx, write_features=self._int16_if_float16(np.ascontiguousarray(data))))
        self.uninitialized_entity_data[idx[0]] = False

    def write_entity_raw(self, offset: int, rows: np.ndarray) -> None:
        """Additive: write whole [emb | m | sqrt v | feature] rows (float32)."""
        self._check_shape("write_entity_raw(rows)", rows, self.settings.entity_data_r_shape)
        idx = self._rw_indices(offset)
        self.engine.run("write_entity_raw", dict(
            write_indices=idx, write_data=np.ascontiguousarray(rows, np.float32)))
        self.uninitialized_entity_data[idx[0]] = False

    def read_entity(self, offset: int) -> np.ndarray:
        idx = self._rw_indices(offset)
        out = np.zeros(self.settings.entity_data_r_shape, dtype=self.settings.execution.dtype)
        self.engine.run("read_entity", dict(read_indices=idx, read_data=self._int16_if_float16(out)))
        return out[:, :self.settings.model.n_entity - offset, :]

    def read_entity_all(self) -> np.ndarray:
        """The whole table on the host -- only sensible for small models."""
        step = self.settings.execution.rw_batch_size
        return np.concatenate(
            [self.read_entity(o) for o in range(0, self.settings.model.n_entity, step)], axis=1)

    # ---- seeded helpers ------------------------------------------------------
    def random_normal(self, shape: Shape, dtype: Union[str, np.dtype] = "float32") -> np.ndarray:
        return self.random.normal(size=shape).astype(dtype)

    def random_uniform(self, shape: Shape, low: float = 0, high: float = 1,
                       dtype: Union[str, np.dtype] = "float32") -> np.ndarray:
        return self.random.uniform(low=low, high=high, size=shape).astype(dtype)

    def random_integers(self, limit: int, shape: Shape) -> np.ndarray:
        return self.random.randint(limit, size=shape).astype(np.uint32)

    # ---- initialisation ------------------------------------------------------
    def initialise_variables(self) -> None:
        """step = 0, zero moments, scaled-normal parameters (reference :624-688):
        relation_embedding ~ (init_scale / D) N(0, 1) (RotatE: uniform phases; TransH: relation_normal
        drawn the same way after it); feature_projection
        ~ N(0, 1) scaled the same way and divided by sqrt(F)."""
        m = self.settings.model
        self.write_variable("step", np.zeros(m.n_shard, np.uint32))
        for name, shape in self.variable_to_shape.items():
            if name.endswith(("/adam_m", "/adam_v")):
                self.write_variable(name, np.zeros(shape, np.float32))
        relation_shape = (m.n_relation_type, self.settings.relation_embedding_size)
        if m.score_fn == "RotatE":   # phases, uniform in [-pi, pi) (reference :633-635)
            relation = self.random_uniform(relation_shape, low=-np.pi, high=np.pi)
        else:
            relation = self.random_normal(relation_shape)
        self.write_variable("relation_embedding", self.init_scale * relation)
        if m.score_fn == "TransH":   # the hyperplane normals (reference :643-651)
            self.write_variable("relation_normal", self.init_scale * self.random_normal(relation_shape))
        # one feature network, or one for the heads and one for the tails (reference :652-686)
        separate = not m.share_feature_networks and m.entity_feature_size > 0
        for prefix in (("head_", "tail_") if separate else ("",)):
            self.write_variable(
                prefix + "feature_projection",
                (self.init_scale / np.sqrt(max(m.entity_feature_size, 1)))
                * self.random_normal((m.entity_feature_size, m.embedding_size)))
            if m.feature_mlp_size > 0:
                for name, shape in (("mlp_up_projection", (2 * m.embedding_size, m.feature_mlp_size)),
                                    ("mlp_down_projection", (m.feature_mlp_size, m.embedding_size))):
                    self.write_variable(prefix + name,
                                        (self.init_scale / np.sqrt(shape[0])) * self.random_normal(shape))

    def initialise_all(self, entity_features: np.ndarray) -> None:
        """Variables, then every table row in rw_batch_size chunks."""
        self.initialise_variables()
        ex, n_entity = self.settings.execution, self.settings.model.n_entity
        for offset in range(0, n_entity, ex.rw_batch_size):
            chunk = np.asarray(entity_features[:, offset:offset + ex.rw_batch_size, :])
            short = ex.rw_batch_size - chunk.shape[1]
            if short:
                chunk = np.pad(chunk, [(0, 0), (0, short), (0, 0)])
            self.write_entity(offset, chunk.astype(ex.dtype))

    def read_all(self) -> Dict[str, np.ndarray]:
        state = {name: self.read_variable(name) for name in self.variable_to_shape}
        state["entity_data"] = self.read_entity_all()
        return state

    # ---- training ------------------------------------------------------------
    def _next_learning_rate(self) -> float:
        """Host schedule, evaluated once per program run (reference :737-759)."""
        t = self.settings.training
        decay = t.learning_rate_decay
        if isinstance(decay, LinearLearningRateDecay):
            self.current_learning_rate = t.learning_rate * (1 - self.step / t.n_step)
        elif isinstance(decay, SteppedLearningRateDecay):
            if self.step >= self.decay_step:
                self.current_learning_rate *= decay.multiplier
                self.decay_step *= 1.5
        elif isinstance(decay, ExponentialLearningRateDecay):
            self.current_learning_rate = t.learning_rate * 0.5 ** (self.step / decay.half_life_steps)
        return self.current_learning_rate

    def _check_initialised(self) -> None:
        if not self.entity_data_initialized:
            missing = int(np.sum(self.uninitialized_entity_data))
            if missing:
                raise ValueError(f"Calling train_step() with uninitialised entity data ({missing} entities)")
            self.entity_data_initialized = True
        if self.uninitialized_variables:
            raise ValueError("Calling train_step() with uninitialised variables "
                             f"{sorted(self.uninitialized_variables)}")

    def train_step_loop(self, batch: Optional[Batch], step_begin: Optional[int] = None,
                        step_count: Optional[int] = None,
                        profile_kernels: Optional[bool] = None) -> Tuple[float, float]:
        """``train_steps_per_program_run`` steps; returns (loss summed over
        shards and averaged over steps, learning rate used).  ``batch=None``
        (additive) reuses the index arrays left in HBM by ``stage_batch``,
        optionally only its steps [step_begin, step_begin + step_count)."""
        self._check_initialised()
        n_shard = self.settings.model.n_shard
        lr = self._next_learning_rate()
        n_run = self.settings.execution.train_steps_per_program_run
        loss = np.full(n_shard, np.nan, dtype=np.float32)
        data: Dict[str, Any] = dict(learning_rate=np.full(n_shard, lr, dtype=np.float32), loss=loss)
        if batch is None:
            data["staged"] = True
            if step_count is not None:
                data["step_begin"], data["step_count"] = int(step_begin or 0), int(step_count)
                n_run = int(step_count)
        else:
            data.update({k: np.ascontiguousarray(v) for k, v in vars(batch).items()})
        if profile_kernels is not None:  # additive: HIP-event timing of every kernel
            data["profile_kernels"] = bool(profile_kernels)
        self.step += n_run
        self.engine.run("train_step_loop", data)
        return float(np.sum(loss)), lr

    def stage_batch(self, batch: Batch) -> None:
        """Additive: validate and upload a batch's index arrays once."""
        self.engine.run("stage_batch", {k: np.ascontiguousarray(v) for k, v in vars(batch).items()})

    def timing(self) -> Dict[str, Any]:
        """Additive: device timings of the last loop, per-kernel totals since the
        last call (needs execution.profile_kernels) and per-step row counts."""
        n = len(KERNEL_NAMES)
        phase, kms = np.zeros(4, np.float32), np.zeros(n, np.float32)
        calls = np.zeros(n, np.uint32)
        counts = np.zeros((self.settings.execution.train_steps_per_program_run, 4), np.uint32)
        self.engine.run("timing", dict(phase_ms=phase, kernel_ms=kms, kernel_calls=calls,
                                       plan_counts=counts))
        return dict(
            upload_ms=float(phase[0]), plan_ms=float(phase[1]), steps_ms=float(phase[2]),
            total_ms=float(phase[3]),
            kernels={k: dict(ms=float(kms[i]), calls=int(calls[i])) for i, k in enumerate(KERNEL_NAMES)},
            unique_entity_rows=counts[:, 0].copy(), entity_chunks=counts[:, 1].copy())

    # ---- prediction ------------------------------------------------------------
    def _predict_hr_chunk(self, idx_relation: np.ndarray) -> Predictions:
        """One ``predict`` program run (reference :781-817): idx_relation
        uint32[n_shard, predict_hr_batch_size, 2] = (head row, relation) per
        query shard.  The device returns every tail shard's n_best per query;
        they are merged to the overall n_best here, best first."""
        ex, S = self.settings.execution, self.settings.model.n_shard
        Hb, n_best = ex.predict_hr_batch_size, ex.predict_n_best
        scores = np.full((S, S, Hb, n_best), np.nan, np.float32)  # [query shard, tail shard, query, rank]
        rows = np.zeros(scores.shape, np.uint32)
        self.engine.run("predict", dict(
            predict_head=np.ascontiguousarray(idx_relation[:, :, 0], np.uint32),
            predict_relation=np.ascontiguousarray(idx_relation[:, :, 1], np.uint32),
            predict_entity_count=np.ascontiguousarray(self.shard_to_entity_count, np.uint32),
            predict_scores=scores, predict_indices=rows))
        tail_shard = np.broadcast_to(np.arange(S, dtype=np.uint32)[None, :, None, None], rows.shape)
        shard_idx = np.stack([tail_shard, rows], axis=-1)          # [S, S, Hb, n_best, 2]
        pooled = Predictions(shard_idx=shard_idx.transpose(0, 2, 1, 3, 4).reshape(S, Hb, S * n_best, 2),
                             score=scores.transpose(0, 2, 1, 3).reshape(S, Hb, S * n_best))
        return pooled.topk(n_best).sort()

    def predict(self, shard_idx_relation: np.ndarray) -> Predictions:
        """Best tails for queries uint32[n, 3] = (head shard, head row, relation)
        (reference :820-861): queries are dealt to their shards' slots in chunks
        of predict_hr_batch_size, unused slots query row 0."""
        shard_idx_relation = np.asarray(shard_idx_relation)
        if shard_idx_relation.shape[1:] != (3,):
            raise ValueError("shard_idx_relation should be of shape (n, 3)")
        ex, S = self.settings.execution, self.settings.model.n_shard
        Hb, n_best, n = ex.predict_hr_batch_size, ex.predict_n_best, shard_idx_relation.shape[0]
        out = Predictions(shard_idx=np.zeros((n, n_best, 2), np.uint32), score=np.zeros((n, n_best), np.float32))
        of_shard = [np.flatnonzero(shard_idx_relation[:, 0] == s) for s in range(S)]
        for start in range(0, max(len(x) for x in of_shard), Hb):
            slots = np.zeros((S, Hb, 2), np.uint32)
            part = [x[start:start + Hb] for x in of_shard]
            for s, which in enumerate(part):
                slots[s, :len(which)] = shard_idx_relation[which, 1:3]
            found = self._predict_hr_chunk(slots)
            for s, which in enumerate(part):
                out.shard_idx[which] = found.shard_idx[s, :len(which)]
                out.score[which] = found.score[s, :len(which)]
        return out
