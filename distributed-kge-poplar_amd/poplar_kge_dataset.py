"""Synthetic data, entity partitioning and batch sampling for the training step.

Host-side counterpart of the reference's ``src/python/poplar_kge_dataset.py``
(``RawData`` :17-157, ``unique_pad`` :161-164, ``Dataset`` :171-435): the same
classes, attributes and array layouts, so that code written against the
reference's module drives this engine unchanged, ``DatasetWrapper`` (:437-475)
for a torch ``DataLoader`` with worker processes included.  What is not here:
the OGB loader (``ogb`` is not a dependency; ``RawData.load`` raises for that
dataset).

One addition: ``Dataset.sample_batch(deduplicate=False)`` skips the per-shard
``np.unique`` and hands the engine raw ids with identity slot maps -- the engine
sorts and merges duplicates on the device, which takes the most expensive host
step (the reference spreads it over 10 worker processes) off the critical path.
"""

import dataclasses
from typing import Callable, Dict, Iterable, Tuple

import numpy as np

import poplar_kge as kge

EVAL_PARTS = ("valid", "test-dev", "test-challenge")


@dataclasses.dataclass
class RawData:
    """A knowledge graph in plain entity ids (reference :17-25)."""

    n_entity: int
    n_relation_type: int
    entity_features: np.ndarray      # float16[n_entity, feature_size]
    train_hrt: np.ndarray            # uint32[n_train, 3]
    eval_hr_: Dict[str, np.ndarray]  # part -> uint32[n, 2 or 3]

    @classmethod
    def generate(cls, n_entity: int, n_relation_type: int, feature_size: int, n_train: int,
                 n_eval: int, seed: int) -> "RawData":
        """Uniform random triples and N(0,1) features (reference :27-63; the draws
        come in the same order: per part h, r, t; then features; then the
        evaluation subset of the training triples)."""
        rng = np.random.RandomState(seed)

        def triples(n: int) -> np.ndarray:
            h = rng.randint(n_entity, size=n)
            r = rng.randint(n_relation_type, size=n)
            t = rng.randint(n_entity, size=n)
            return np.stack([h, r, t], axis=-1).astype(np.uint32)

        train = triples(n_train)
        parts = {name: triples(n_eval) for name in EVAL_PARTS}
        features = rng.randn(n_entity, feature_size).astype(np.float16)
        parts["train"] = train[rng.choice(n_train, size=n_eval, replace=False)]
        return cls(n_entity=n_entity, n_relation_type=n_relation_type, entity_features=features,
                   train_hrt=train, eval_hr_=parts)

    @classmethod
    def load(cls, settings: kge.Settings) -> "RawData":
        """Reference :131-157.  Only generated data: the shards hold
        ``n_entity - 1`` real rows each, one entity short of full."""
        ds = settings.data.dataset
        if isinstance(ds, kge.GeneratedDataSettings):
            m = settings.model
            return cls.generate(n_entity=(m.n_entity - 1) * m.n_shard - 1,
                                n_relation_type=m.n_relation_type,
                                feature_size=m.entity_feature_size, n_train=ds.n_train,
                                n_eval=ds.n_eval, seed=ds.seed)
        if isinstance(ds, kge.WikiKg90Mv2Settings):
            raise ValueError("Dataset 'wikikg90mv2' needs the ogb package and its files, which this "
                             "build does not load; use GeneratedDataSettings")
        raise ValueError(f"Unknown dataset '{ds}'")


def unique_pad(idx: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Sorted distinct values of ``idx`` zero-padded to ``len(idx)``, and for
    every element its position among them (reference :161-164)."""
    values, position = np.unique(idx, return_inverse=True)
    padded = np.zeros(len(idx), dtype=values.dtype)
    padded[:len(values)] = values
    return padded, position.astype(np.uint32)


class Dataset:
    """Entities dealt to shards, training triples indexed by (head shard, tail
    shard[, relation]) for sampling, and the batch sampler (reference :171-393).

    Attributes kept from the reference: ``entity_to_shard``, ``entity_to_idx``
    (row inside the shard, from 1: row 0 is padding), ``shard_to_count``,
    ``n_entity_per_shard``, ``shard_idx_to_entity``, ``shardpair_to_count``,
    ``shardpair_to_offset``, ``shardpair_to_flat_hrt``, ``pos_tail_idx``.
    """

    def __init__(self, data: RawData, n_shard: int, train_steps_per_program_run: int,
                 settings: "kge.DataSettings"):
        self.data, self.n_shard, self.settings = data, n_shard, settings
        self.train_steps_per_program_run = train_steps_per_program_run
        self.random = np.random.RandomState(settings.seed)
        S, B, A = n_shard, settings.batch_size, settings.a2a_size

        # a random permutation dealt round-robin: entity e sits in shard p[e] % S, row 1 + p[e] // S
        order = self.random.permutation(data.n_entity)
        self.entity_to_shard = order % S
        self.entity_to_idx = order // S + 1
        self.shard_to_count = np.bincount(self.entity_to_shard, minlength=S)
        self.n_entity_per_shard = 1 + int(self.shard_to_count.max())
        self.shard_idx_to_entity = np.full((S, self.n_entity_per_shard), 1 << 31, dtype=np.uint32)
        self.shard_idx_to_entity[self.entity_to_shard, self.entity_to_idx] = np.arange(data.n_entity)

        # training triples grouped by bucket = (head shard, tail shard[, relation])
        h, r, t = (data.train_hrt[:, i] for i in range(3))
        pair = S * self.entity_to_shard[h] + self.entity_to_shard[t]
        self.by_relation = isinstance(settings.sampling_strategy, kge.CubicRootRelationSampling)
        if self.by_relation:
            bucket, shape = pair * data.n_relation_type + r, (S * S, data.n_relation_type)
        else:
            bucket, shape = pair, (S, S)
        order = np.argsort(bucket, kind="stable")
        counts = np.bincount(bucket, minlength=int(np.prod(shape)))
        self.shardpair_to_count = counts.reshape(shape)
        self.shardpair_to_offset = (np.cumsum(counts) - counts).reshape(shape)
        if self.by_relation:
            # relations are drawn with probability ~ count^(1/3) inside each shard pair
            root = np.cbrt(self.shardpair_to_count)
            self.shardpair_sample_prob = root / root.sum(axis=-1, keepdims=True)
        self.shardpair_to_flat_hrt = np.stack(
            [self.entity_to_idx[h[order]], r[order], self.entity_to_idx[t[order]]]).astype(np.uint32)

        self.entity_projection_seed = self.random.randint(1 << 32)
        if B % S != 0:
            raise ValueError(f"Expected batch_size ({B}) to be a multiple of n_shard ({S})")
        self.positives_per_shardpair = B // S
        if A <= self.positives_per_shardpair:
            raise ValueError(f"Expected a2a_size ({A}) to be >= batch_size/n_shard "
                             f"({self.positives_per_shardpair})")
        self.negatives_per_shardpair = A - self.positives_per_shardpair

        # positive b = (tail shard j, k) of any shard sits at position j*A + k of the tails received
        P = self.positives_per_shardpair
        position = (A * np.arange(S)[:, None] + np.arange(P)[None, :]).reshape(B)
        self.pos_tail_idx = np.ascontiguousarray(
            np.broadcast_to(position, (S, train_steps_per_program_run, B))).astype(np.uint32)

    @classmethod
    def load(cls, data: RawData, settings: kge.Settings) -> "Dataset":
        return cls(data, n_shard=settings.model.n_shard,
                   train_steps_per_program_run=settings.execution.train_steps_per_program_run,
                   settings=settings.data)

    # ---- features ------------------------------------------------------------
    def entity_features(self, feature_size: int) -> np.ndarray:
        """float16[n_shard, n_entity_per_shard, feature_size] in shard layout
        (reference :282-306): zeros, the data's features, or a fixed random
        projection of them."""
        mapping = self.settings.entity_feature_mapping
        out = np.zeros((self.n_shard, self.n_entity_per_shard, feature_size), dtype=np.float16)
        if mapping == "zero":
            return out
        if mapping not in ("full", "random_projection"):
            raise ValueError(f"Unknown entity_feature_mapping: {mapping}")
        features = self.data.entity_features
        width = features.shape[-1]
        if mapping == "full":
            if feature_size != width:
                raise ValueError("Entity_feature_mapping 'full' requires dataset feature_size "
                                 f"({width}) == model feature_size ({feature_size})")
        else:
            rng = np.random.RandomState(self.entity_projection_seed)
            projection = rng.randn(width, feature_size).astype(np.float16) / np.sqrt(width)
            features = features @ projection
        out[self.entity_to_shard, self.entity_to_idx] = features
        return out

    # ---- sampling ------------------------------------------------------------
    def _sample_positive_positions(self) -> np.ndarray:
        """Positions into ``shardpair_to_flat_hrt``: [head shard, step, tail shard, P]."""
        S, n, P = self.n_shard, self.train_steps_per_program_run, self.positives_per_shardpair
        if not self.by_relation:
            draw = self.random.randint(1 << 63, size=(S, n, S, P))
            return (self.shardpair_to_offset[:, None, :, None]
                    + draw % self.shardpair_to_count[:, None, :, None])
        relation = np.stack([self.random.choice(self.data.n_relation_type, size=n * P, p=prob)
                             for prob in self.shardpair_sample_prob])
        pair = np.arange(S * S)[:, None]
        offset = self.shardpair_to_offset[pair, relation].reshape(S, S, n * P)
        count = self.shardpair_to_count[pair, relation].reshape(S, S, n * P)
        draw = self.random.randint(1 << 63, size=(S, S, n * P))
        return (offset + draw % count).reshape(S, S, n, P).transpose(0, 2, 1, 3)

    def sample_batch(self, deduplicate: bool = True) -> "kge.Batch":
        """One program run's index arrays (reference :310-393).

        Per (shard, step) the shard gathers its B heads, the B true tails that
        live on it (P from every head shard) and S * (A - P) uniform negatives.
        """
        S, n = self.n_shard, self.train_steps_per_program_run
        B, P, N = self.settings.batch_size, self.positives_per_shardpair, self.negatives_per_shardpair
        h, r, t = self.shardpair_to_flat_hrt[:, self._sample_positive_positions()]  # [S, n, S, P]
        negative = 1 + (self.random.randint(1 << 63, size=(S, n, S, N))
                        % self.shard_to_count[None, None, :, None]).astype(np.uint32)
        # rows to gather, from the owning shard's point of view: axis 0 = owner.
        # t[hs, step, ts, k] lives on shard ts and is sent to shard hs.
        ids = np.concatenate([h.reshape(S, n, B),
                              t.transpose(2, 1, 0, 3).reshape(S, n, B),
                              negative.transpose(2, 1, 0, 3).reshape(S, n, S * N)], axis=2)
        if deduplicate:
            flat = ids.reshape(S * n, -1)
            remote = np.empty_like(flat)
            slot = np.empty(flat.shape, np.uint32)
            for i, row in enumerate(flat):
                remote[i], slot[i] = unique_pad(row)
            remote, slot = remote.reshape(ids.shape), slot.reshape(ids.shape)
        else:
            remote = ids
            slot = np.broadcast_to(np.arange(ids.shape[2], dtype=np.uint32), ids.shape)
        a2a = np.concatenate([slot[:, :, B:2 * B].reshape(S, n, S, P),
                              slot[:, :, 2 * B:].reshape(S, n, S, N)], axis=3)
        return kge.Batch(remote=np.ascontiguousarray(remote, np.uint32),
                         head=np.ascontiguousarray(slot[:, :, :B]),
                         relation=np.ascontiguousarray(r.reshape(S, n, B)),
                         a2a=np.ascontiguousarray(a2a), tail=self.pos_tail_idx)

    def batches(self) -> Iterable["kge.Batch"]:
        while True:
            yield self.sample_batch()

    # ---- evaluation ------------------------------------------------------------
    def predict(self, part: str, predict_fn: Callable[[np.ndarray], "kge.Predictions"]
                ) -> Tuple[np.ndarray, np.ndarray]:
        """Best tails (plain entity ids) and scores for every (h, r, ?) of an
        evaluation part (reference :399-421).  ``predict_fn`` takes
        uint32[n, 3] = (head shard, head row, relation)."""
        head, relation = self.data.eval_hr_[part][:, 0], self.data.eval_hr_[part][:, 1]
        query = np.stack([self.entity_to_shard[head], self.entity_to_idx[head], relation], axis=1)
        found = predict_fn(query)
        return self.shard_idx_to_entity[found.shard_idx[..., 0], found.shard_idx[..., 1]], found.score

    def mrr(self, part: str, predict_fn: Callable[[np.ndarray], "kge.Predictions"]) -> float:
        """Mean reciprocal rank of the true tail among the ten best predictions,
        0 when it is not among them (the OGB WikiKG90Mv2 evaluator's definition,
        reference :423-435)."""
        truth = self.data.eval_hr_[part][:, 2].astype(np.int64)
        best = self.predict(part, predict_fn)[0][:, :10].astype(np.int64)
        hit = best == truth[:, None]
        rank = np.where(hit.any(axis=1), hit.argmax(axis=1) + 1, 0)
        return float(np.mean(np.where(rank > 0, 1.0 / np.maximum(rank, 1), 0.0)))


class DatasetWrapper:
    """A map-style dataset of sampled batches for ``torch.utils.data.DataLoader``
    (reference :437-475): ``DataLoader(DatasetWrapper(ds), batch_size=None, num_workers=10,
    worker_init_fn=ds.worker_init_fn)`` samples batches in worker processes, each from its
    own random stream.  torch is only needed by the loader itself, not to define this class."""

    def __init__(self, dataset: Dataset) -> None:
        self.ds = dataset

    def __len__(self) -> int:
        return (2 ** 31) - 1

    def __getitem__(self, item: int) -> Dict[str, np.ndarray]:
        batch = self.ds.sample_batch()
        return {name: getattr(batch, name).astype(np.int32)
                for name in ("remote", "a2a", "head", "relation", "tail")}

    @staticmethod
    def tensors_to_batch(remote, a2a, head, relation, tail) -> "kge.Batch":
        """What a DataLoader yields (int32 tensors) back as the engine's uint32 arrays."""
        as_u32 = lambda t: np.ascontiguousarray(t.numpy() if hasattr(t, "numpy") else t).astype(np.uint32)  # noqa: E731
        return kge.Batch(remote=as_u32(remote), head=as_u32(head), relation=as_u32(relation),
                         a2a=as_u32(a2a), tail=as_u32(tail))

    @staticmethod
    def worker_init_fn(worker_id: int) -> None:
        import torch.utils.data

        unwrapped = torch.utils.data.get_worker_info().dataset.ds
        unwrapped.random = np.random.RandomState(unwrapped.settings.seed + worker_id)
