"""The device's index work, bit for bit.  The plan phase of a training step resolves every
head / tail contribution to its table row, finds the distinct rows and groups the
contributions by row: the device-side counterpart of the host's ``unique_pad``
(/root/reference/src/python/poplar_kge_dataset.py:161-164, ``np.unique`` with inverse
indices) and of the grouping ``multiUpdateAdd`` performs for duplicate indices
(/root/reference/src/pag/pag.cpp:721-743).  With ``execution.merge_tails`` (the default) a
block's tail list is first reduced to its distinct rows, each with its multiplicity.  Every
array has an exact integer answer, which NumPy supplies here."""

import numpy as np
import pytest

import hip_harness as H
import kge_cases as K

pytestmark = pytest.mark.gpu


def _expected_rows(c, batch, i):
    """Table row of every contribution of step i, in the device's item order: heads of every
    block, then the tails block by block in all-to-all order (tail slot j*A + k of block d is
    what shard j sends to d, tests/python/reference_model.py:132-138), then every remote slot."""
    S, B, A, NE = c["n_shard"], c["batch"], c["a2a"], c["n_entity"]
    base = np.zeros(S, np.int64) if c["shared_table"] else np.arange(S, dtype=np.int64) * NE
    remote, a2a, head = batch["remote"][:, i], batch["a2a"][:, i], batch["head"][:, i]
    heads = np.concatenate([base[d] + remote[d][head[d]] for d in range(S)])
    tails = np.concatenate([base[j] + remote[j][a2a[j, d]] for d in range(S) for j in range(S)])
    slots = np.concatenate([base[s] + remote[s] for s in range(S)])
    return np.concatenate([heads, tails]).astype(np.uint32), slots.astype(np.uint32)


def _dump(engine, c, i, n_rel_items):
    S, B, A = c["n_shard"], c["batch"], c["a2a"]
    R, NRR = S * (B + S * A), c["n_relation"]
    out = dict(contribution_row=np.zeros(R, np.uint32), unique_rows=np.zeros(R, np.uint32),
               segment_start=np.zeros(R + 1, np.uint32), segment_contributions=np.zeros(R, np.uint32),
               sorted_items=np.zeros(2 * R, np.uint32), counts=np.zeros(2, np.uint32),
               relation_unique_rows=np.zeros(NRR, np.uint32), relation_segment_start=np.zeros(NRR + 1, np.uint32),
               relation_segment_contributions=np.zeros(NRR, np.uint32),
               relation_sorted_items=np.zeros(n_rel_items, np.uint32), relation_counts=np.zeros(2, np.uint32),
               label_column=np.zeros(S * B, np.uint32))
    engine.run("plan_dump", dict(step=i, **out))
    return out


def _merged_tails(tails, S, T):
    """Per block the distinct tail rows in ascending order: what the device keeps one score column
    for.  Returns the contribution rows of the tail part (columns past a block's distinct count
    repeat its first row), a mask of the columns that carry gradient, the distinct counts, the
    multiplicities and the column of every tail position."""
    rows = np.zeros(S * T, np.uint32)
    live = np.zeros(S * T, bool)
    mult = np.zeros(S * T, np.float32)
    col = np.zeros(S * T, np.uint32)
    count = np.zeros(S, np.uint32)
    for d in range(S):
        uniq, inverse, counts = np.unique(tails[d * T:(d + 1) * T], return_inverse=True, return_counts=True)
        n = uniq.size
        count[d] = n
        rows[d * T:d * T + n] = uniq
        rows[d * T + n:(d + 1) * T] = uniq[0]
        live[d * T:d * T + n] = True
        mult[d * T:d * T + n] = counts
        col[d * T:(d + 1) * T] = inverse
    return rows, live, count, mult, col


def _check_plan(c, batch, n_step, merge=True):
    import libpoplar_kge

    S, B, A = c["n_shard"], c["batch"], c["a2a"]
    T = S * A
    R, SB, NRR = S * (B + S * A), S * B, c["n_relation"]
    engine = libpoplar_kge.Engine(H.engine_settings(c, n_step, **{"execution.merge_tails": merge}), "")
    H.train(engine, c, 0.01, batch)   # zero table: the numbers do not matter, the plan does
    for i in range(n_step):
        got = _dump(engine, c, i, SB + NRR)
        contrib, slots = _expected_rows(c, batch, i)
        label = np.concatenate([batch["tail"][d, i] for d in range(S)]).astype(np.uint32)
        real = np.ones(R, bool)   # which contributions carry gradient
        if merge:
            # one score column per distinct tail row of a block
            extra = dict(tail_count=np.zeros(S, np.uint32), tail_column=np.zeros(S * T, np.uint32),
                         tail_multiplicity=np.zeros(S * T, np.float32))
            engine.run("plan_dump", dict(step=i, **extra))
            rows, live, count, mult, col = _merged_tails(contrib[SB:], S, T)
            np.testing.assert_array_equal(extra["tail_count"], count)
            np.testing.assert_array_equal(extra["tail_column"], col)
            np.testing.assert_array_equal(extra["tail_multiplicity"], mult)
            assert mult.sum() == S * T
            contrib = np.concatenate([contrib[:SB], rows])
            real[SB:] = live
            label = col.reshape(S, T)[np.repeat(np.arange(S), B), label]
        np.testing.assert_array_equal(got["label_column"], label)
        np.testing.assert_array_equal(got["contribution_row"], contrib)
        # entity plan: items = R contributions then the R remote slots
        keys = np.concatenate([contrib, slots])
        other = np.concatenate([~real, np.ones(R, bool)])   # members of the update set without gradient
        uniq, inverse, counts = np.unique(keys, return_inverse=True, return_counts=True)
        U = uniq.size
        assert got["counts"][0] == U
        np.testing.assert_array_equal(got["unique_rows"][:U], uniq)
        starts = np.concatenate([[0], np.cumsum(counts)])
        np.testing.assert_array_equal(got["segment_start"][:U + 1], starts)
        np.testing.assert_array_equal(got["segment_contributions"][:U],
                                      np.bincount(inverse[~other], minlength=U))
        # the sorted items: ordered by (row, contribution or not, item number)
        np.testing.assert_array_equal(got["sorted_items"], np.lexsort((np.arange(2 * R), other, keys)))
        # every distinct row of `remote` is in the update set, as unique_pad's output is
        assert np.array_equal(np.unique(slots), uniq)
        # relation plan: the positives' relations, then every relation id once
        rel = np.concatenate([batch["relation"][d, i] for d in range(S)]).astype(np.uint32)
        rkeys = np.concatenate([rel, np.arange(NRR, dtype=np.uint32)])
        assert got["relation_counts"][0] == NRR
        np.testing.assert_array_equal(got["relation_unique_rows"], np.arange(NRR))
        np.testing.assert_array_equal(got["relation_segment_start"],
                                      np.concatenate([[0], np.cumsum(np.bincount(rkeys, minlength=NRR))]))
        np.testing.assert_array_equal(got["relation_segment_contributions"], np.bincount(rel, minlength=NRR))
        np.testing.assert_array_equal(got["relation_sorted_items"], np.argsort(rkeys, kind="stable"))


@pytest.mark.parametrize("merge", [False, True])
@pytest.mark.parametrize("shape", ["c2", "c3"])
def test_plan_raw_zipf_ids_bit_exact(shape, merge):
    """Raw (not de-duplicated) Zipf ids at the benchmark workloads' per-step shape: 32 blocks x
    (256 + 256) and 64 blocks x (256 + 512) over one shared table, hot rows of thousands of
    contributions."""
    blocks, batch, tails, n_entity, n_rel = ((32, 256, 256, 1_000_000, 1000) if shape == "c2" else
                                             (64, 256, 512, 22_800_000 // 64, 1387))
    # (the c3-shaped case keeps the table small: keys still need 19 bits, three sort passes)
    c = K.cfg_dict(n_shard=blocks, batch=batch, a2a=tails // blocks, n_entity=n_entity, n_relation=n_rel,
                   dim=8, feature=0, shared_table=True, distance_fn="L2")
    rng = np.random.default_rng(12)
    _check_plan(c, K.raw_batch(c, 2, rng), 2, merge)


@pytest.mark.parametrize("merge", [False, True])
@pytest.mark.parametrize("shared", [False, True])
def test_plan_unique_pad_layout_bit_exact(shared, merge):
    """The reference's own batch layout: `remote` = sorted distinct ids zero-padded to B + S*A
    (unique_pad), head / a2a = inverse indices.  Private tables offset every shard's rows."""
    c = K.cfg_dict(n_shard=4, batch=96, a2a=24, n_entity=3000, n_relation=52, dim=8, feature=0,
                   shared_table=shared)
    S, B, A, NE = 4, 96, 24, 3000
    NR = B + S * A
    rng = np.random.default_rng(3)
    n_step = 3
    remote = np.zeros((S, n_step, NR), np.uint32)
    head = np.zeros((S, n_step, B), np.uint32)
    a2a = np.zeros((S, n_step, S, A), np.uint32)
    for s in range(S):
        for i in range(n_step):
            ids = K.zipf_ids(rng, NE, NR)                  # duplicates: the unique list is shorter
            uniq, inv = np.unique(ids, return_inverse=True)
            remote[s, i, :uniq.size] = uniq                # zero padding behind (row 0)
            head[s, i], a2a[s, i] = inv[:B], inv[B:].reshape(S, A)
    batch = dict(remote=remote, a2a=a2a, head=head,
                 relation=rng.integers(0, 52, (S, n_step, B)).astype(np.uint32),
                 tail=rng.integers(0, S * A, (S, n_step, B)).astype(np.uint32))
    _check_plan(c, batch, n_step, merge)


@pytest.mark.parametrize("n_entity,n_relation", [(50, 5000), (3000, 300), (70_000, 3)])
def test_plan_shared_sort_launches_key_widths(n_entity, n_relation):
    """The entity and the relation sort share their launches on the wider key's pass schedule:
    relation keys wider than entity keys (13 bits against 6: the entity sort takes part in the
    first of two passes only), about equal, and much narrower (2 bits against 17)."""
    c = K.cfg_dict(n_shard=2, batch=160, a2a=40, n_entity=n_entity, n_relation=n_relation, dim=8, feature=0,
                   shared_table=True)
    rng = np.random.default_rng(21)
    _check_plan(c, K.raw_batch(c, 3, rng), 3)
