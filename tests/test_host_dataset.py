"""Host batch sampler (poplar_kge_dataset): the invariants the reference's own
tests hold for it (tests/python/test_poplar_kge_dataset.py:12-138), plus the
raw-id mode this build adds.  CPU only."""

import itertools

import numpy as np
import pytest

import poplar_kge as kge
import poplar_kge_dataset as kge_data


def _data_settings(**kw):
    base = dict(seed=9842, batch_size=16, a2a_size=10, entity_feature_mapping="full", dataset=None,
                sampling_strategy=None)
    base.update(kw)
    return kge.DataSettings(**base)


def test_unique_pad():
    values, slot = kge_data.unique_pad(np.array([7, 3, 7, 9, 3, 3], np.uint32))
    np.testing.assert_array_equal(values, [3, 7, 9, 0, 0, 0])
    np.testing.assert_array_equal(slot, [1, 0, 1, 2, 0, 0])
    assert slot.dtype == np.uint32 and len(values) == 6


def test_generate_shapes_and_ranges():
    data = kge_data.RawData.generate(n_entity=70, n_relation_type=9, feature_size=8, n_train=100,
                                     n_eval=50, seed=29483)
    assert data.train_hrt.shape == (100, 3) and data.train_hrt.dtype == np.uint32
    assert data.entity_features.shape == (70, 8) and data.entity_features.dtype == np.float16
    assert set(data.eval_hr_) == {"train", "valid", "test-dev", "test-challenge"}
    for part in data.eval_hr_.values():
        assert part.shape == (50, 3)
        assert part[:, [0, 2]].max() < 70 and part[:, 1].max() < 9
    train = set(map(tuple, data.train_hrt))
    assert all(tuple(x) in train for x in data.eval_hr_["train"])
    again = kge_data.RawData.generate(n_entity=70, n_relation_type=9, feature_size=8, n_train=100,
                                      n_eval=50, seed=29483)
    np.testing.assert_array_equal(again.train_hrt, data.train_hrt)


def test_load_generated_fits_the_shards():
    settings = kge.Settings.create_demo()
    settings.seed = 100
    settings.prepare()
    data = kge_data.RawData.load(settings)
    m = settings.model
    assert data.n_entity == (m.n_entity - 1) * m.n_shard - 1
    dataset = kge_data.Dataset.load(data, settings)
    assert dataset.n_entity_per_shard <= m.n_entity
    assert dataset.shard_to_count.sum() == data.n_entity


def test_entity_features():
    data = kge_data.RawData.generate(n_entity=70, n_relation_type=100, feature_size=8, n_train=100,
                                     n_eval=50, seed=29483)

    def features(mapping, feature_size):
        dataset = kge_data.Dataset(data, n_shard=4, train_steps_per_program_run=10,
                                   settings=_data_settings(entity_feature_mapping=mapping))
        out = dataset.entity_features(feature_size=feature_size)
        assert out.shape == (4, 1 + int(np.ceil(70 / 4)), feature_size)
        assert out.dtype == np.float16
        return dataset, out

    _, zero = features("zero", 6)
    assert not zero.any()
    dataset, full = features("full", 8)
    # every entity's features sit at its (shard, row); row 0 stays the padding row
    np.testing.assert_array_equal(full[dataset.entity_to_shard, dataset.entity_to_idx],
                                  data.entity_features)
    assert not full[:, 0].any()
    features("random_projection", 6)
    with pytest.raises(ValueError):
        features("full", 6)
    with pytest.raises(ValueError):
        features("nonsense", 8)


def test_partition_is_a_bijection():
    data = kge_data.RawData.generate(n_entity=71, n_relation_type=5, feature_size=0, n_train=40,
                                     n_eval=10, seed=1)
    ds = kge_data.Dataset(data, n_shard=4, train_steps_per_program_run=2, settings=_data_settings())
    assert ds.entity_to_idx.min() == 1
    np.testing.assert_array_equal(ds.shard_idx_to_entity[ds.entity_to_shard, ds.entity_to_idx],
                                  np.arange(71))
    assert (ds.shard_idx_to_entity == 1 << 31).sum() == 4 * ds.n_entity_per_shard - 71
    assert ds.shard_to_count.max() - ds.shard_to_count.min() <= 1


def test_constructor_guards():
    data = kge_data.RawData.generate(n_entity=70, n_relation_type=5, feature_size=0, n_train=40,
                                     n_eval=10, seed=1)
    with pytest.raises(ValueError, match="multiple of n_shard"):
        kge_data.Dataset(data, 4, 2, _data_settings(batch_size=18))
    with pytest.raises(ValueError, match="a2a_size"):
        kge_data.Dataset(data, 4, 2, _data_settings(batch_size=16, a2a_size=4))


def _entities_of(dataset, batch):
    """(positive (h, r, t) in plain entity ids, negative tail entities) of a batch,
    resolved the way the engine resolves it: remote rows by slot, tails through
    the all-to-all (what shard j sends to shard d lands at position j*A + i)."""
    S, n = dataset.n_shard, dataset.train_steps_per_program_run
    to_entity = np.full((S, dataset.n_entity_per_shard), -1, np.int64)
    to_entity[dataset.entity_to_shard, dataset.entity_to_idx] = np.arange(dataset.data.n_entity)
    positives, negatives = [], []
    for d in range(S):
        for step in range(n):
            rows = lambda s, slots: to_entity[s, batch.remote[s, step][slots]]  # noqa: E731
            heads = rows(d, batch.head[d, step])
            received = np.concatenate([rows(j, batch.a2a[j, step, d]) for j in range(S)])
            assert received.min() >= 0
            label = batch.tail[d, step]
            positives.append(np.stack([heads, batch.relation[d, step], received[label]], axis=-1))
            mask = np.ones(len(received), bool)
            mask[label] = False
            negatives.append(received[mask])
    return np.concatenate(positives), np.concatenate(negatives)


@pytest.mark.parametrize("strategy", ["cubic_root", None])
def test_sample_batch(strategy):
    data = kge_data.RawData.generate(n_entity=70, n_relation_type=1024, feature_size=0, n_train=100,
                                     n_eval=50, seed=2835)
    S, n = 4, 11
    s = _data_settings(seed=12039, batch_size=8, a2a_size=5,
                       sampling_strategy=kge.CubicRootRelationSampling() if strategy else None)
    dataset = kge_data.Dataset(data, n_shard=S, train_steps_per_program_run=n, settings=s)
    batch = dataset.sample_batch()
    assert batch.remote.shape == (S, n, s.batch_size + S * s.a2a_size)
    assert batch.a2a.shape == (S, n, S, s.a2a_size)
    for part in (batch.head, batch.relation, batch.tail):
        assert part.shape == (S, n, s.batch_size)
    for name, value in vars(batch).items():
        assert value.dtype == np.uint32, name
        assert value.flags.c_contiguous, name
    # remote: sorted distinct rows, then zero padding
    for row in batch.remote.reshape(S * n, -1):
        real = row[row > 0]
        assert np.all(np.diff(real) > 0) and not row[len(real):].any()

    all_hrt = set(map(tuple, data.train_hrt.astype(np.int64)))
    missed_hrt, missed_negative = set(all_hrt), set(range(data.n_entity))
    for batch in itertools.islice(dataset.batches(), 100):
        positive, negative = _entities_of(dataset, batch)
        positive = set(map(tuple, positive))
        assert positive <= all_hrt
        missed_hrt -= positive
        assert negative.min() >= 0 and negative.max() < data.n_entity
        missed_negative -= set(negative.tolist())
    assert not missed_hrt, "unlikely to omit any positive (h,r,t)"
    assert not missed_negative, "unlikely to omit any negative tail entity"


def test_raw_ids_resolve_to_the_same_triples():
    data = kge_data.RawData.generate(n_entity=70, n_relation_type=20, feature_size=0, n_train=100,
                                     n_eval=50, seed=7)
    make = lambda: kge_data.Dataset(data, n_shard=4, train_steps_per_program_run=3,  # noqa: E731
                                    settings=_data_settings(seed=5, batch_size=8, a2a_size=5))
    a, b = make(), make()
    dedup, raw = a.sample_batch(), b.sample_batch(deduplicate=False)
    pos_a, neg_a = _entities_of(a, dedup)
    pos_b, neg_b = _entities_of(b, raw)
    np.testing.assert_array_equal(pos_a, pos_b)
    np.testing.assert_array_equal(neg_a, neg_b)
    assert raw.remote.min() >= 1                       # no padding: every slot is a real row
    np.testing.assert_array_equal(raw.head[0, 0], np.arange(8))


def test_mrr_definition():
    data = kge_data.RawData.generate(n_entity=30, n_relation_type=4, feature_size=0, n_train=40,
                                     n_eval=12, seed=3)
    ds = kge_data.Dataset(data, n_shard=2, train_steps_per_program_run=1,
                          settings=_data_settings(batch_size=4, a2a_size=3))
    truth = data.eval_hr_["valid"][:, 2]

    def predict_fn(query):
        # the true tail at rank 1, 2, 3, ... 10, then missing
        n = len(query)
        ent = np.zeros((n, 10), np.int64)
        for i in range(n):
            others = [e for e in range(data.n_entity) if e != truth[i]][:10]
            ent[i] = others
            if i < 10:
                ent[i, i] = truth[i]
        shard_idx = np.stack([ds.entity_to_shard[ent], ds.entity_to_idx[ent]], axis=-1)
        return kge.Predictions(shard_idx=shard_idx.astype(np.uint32), score=-np.arange(10.0)[None].repeat(n, 0))

    expected = np.mean([1.0 / (i + 1) if i < 10 else 0.0 for i in range(len(truth))])
    assert abs(ds.mrr("valid", predict_fn) - expected) < 1e-12


@pytest.mark.parametrize("workers", [0, 2])
def test_dataset_wrapper_with_torch_dataloader(workers):
    """The reference's training script feeds the engine through a torch DataLoader over
    DatasetWrapper (scripts/run_training.py:36-41, 68-71): batches arrive as int32 tensors
    and go back to the engine's uint32 arrays; worker processes sample from their own streams."""
    import torch

    data = kge_data.RawData.generate(n_entity=70, n_relation_type=20, feature_size=0, n_train=100,
                                     n_eval=50, seed=7)
    S, n = 4, 3
    settings = _data_settings(seed=5, batch_size=8, a2a_size=5)
    dataset = kge_data.Dataset(data, n_shard=S, train_steps_per_program_run=n, settings=settings)
    wrapper = kge_data.DatasetWrapper(dataset)
    assert len(wrapper) == 2 ** 31 - 1
    loader = torch.utils.data.DataLoader(wrapper, batch_size=None, num_workers=workers,
                                         worker_init_fn=wrapper.worker_init_fn)
    all_hrt = set(map(tuple, data.train_hrt.astype(np.int64)))
    seen = []
    for tensors in itertools.islice(iter(loader), 4):
        assert all(t.dtype == torch.int32 for t in tensors.values())
        batch = wrapper.tensors_to_batch(**tensors)
        assert batch.remote.shape == (S, n, settings.batch_size + S * settings.a2a_size)
        for part in vars(batch).values():
            assert part.dtype == np.uint32
        positive, negative = _entities_of(dataset, batch)
        assert set(map(tuple, positive)) <= all_hrt
        assert negative.min() >= 0 and negative.max() < data.n_entity
        seen.append(batch.head.tobytes())
    if workers:   # two workers, two streams: their first batches differ
        assert seen[0] != seen[1]
