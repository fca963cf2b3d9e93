"""Inspector parity: bit-exact against numpy unique + stable argsort."""
import numpy as np
import pytest
import torch

from cuke_amd import synth

pytestmark = pytest.mark.gpu


def check(oracle, parts, n_rows):
    from cuke_amd.kge import inspect
    dev = torch.device("cuda:0")
    ins = inspect([torch.from_numpy(p).to(dev) for p in parts], n_rows)
    ref = oracle.inspect(np.concatenate(parts))
    U = ins.num_unique
    assert U == ref.unique_ids.shape[0]
    assert np.array_equal(ins.ids().cpu().numpy(), ref.unique_ids)
    assert np.array_equal(ins.offsets().cpu().numpy().astype(np.int64), ref.seg_offsets)
    assert np.array_equal(ins.perm[: ins.n].cpu().numpy().astype(np.int64), ref.perm)
    assert np.array_equal(ins.inverse[: ins.n].cpu().numpy().astype(np.int64), ref.inverse)
    assert np.array_equal(ins.sorted_seg[: ins.n].cpu().numpy().astype(np.int64), ref.inverse[ref.perm])


@pytest.mark.parametrize("n,n_rows", [(0, 10), (1, 10), (37, 1), (64, 64), (2048, 2000), (2049, 5),
                                      (5000, 1 << 11), (5000, (1 << 11) + 1), (12288, 1_000_000),
                                      (49152, 4_000_000), (70000, 1 << 22), (300_000, 40_000),
                                      # block size (1024 keys) and the mid / large path switch (65536 keys)
                                      (1023, 50), (1024, 50), (1025, 50), (65535, 70_000), (65536, 1000),
                                      (65537, 1000), (65537, 1 << 30)])
def test_inspect_uniform(oracle, n, n_rows):
    rng = np.random.default_rng(n + n_rows)
    check(oracle, [rng.integers(0, n_rows, n, dtype=np.int64)], n_rows)


def test_inspect_all_equal_and_all_distinct(oracle):
    check(oracle, [np.full(5000, 123, np.int64)], 1000)
    check(oracle, [np.random.default_rng(0).permutation(6000).astype(np.int64)], 6000)
    check(oracle, [np.arange(4096, dtype=np.int64)[::-1].copy()], 4096)
    check(oracle, [np.array([(1 << 32) - 1, 0, (1 << 32) - 1, 7], np.int64)], 1 << 32)


@pytest.mark.parametrize("name", ["cfg2_distmult", "cfg3_transr", "cfg4_rotate", "cfg5_transh"])
def test_inspect_benchmark_index_sets(oracle, name):
    w = synth.make_workload(name, tables=False)
    a = w.arrays
    parts = [a["h"], a["t"]] + ([a["neg"]] if "neg" in a else [])
    check(oracle, parts, w.n_ent)
    check(oracle, [a["r"]], w.n_rel)


def test_inspect_multi_part_ragged(oracle):
    rng = np.random.default_rng(3)
    parts = [rng.integers(0, 777, k, dtype=np.int64) for k in (5, 0, 2047, 1)]
    check(oracle, parts, 777)
