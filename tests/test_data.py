"""Dataset reader (CPU) and the device negative sampler against its numpy restatement (GPU)."""
import numpy as np
import pytest


def write_dataset(tmp_path):
    (tmp_path / "entities.dict").write_text("0\ta\n1\tb\n2\tc\n3\td\n")
    (tmp_path / "relations.dict").write_text("0\tlikes\n1\tknows\n")
    (tmp_path / "train.txt").write_text("a\tlikes\tb\nb\tknows\tc\nd\tlikes\ta\nc\tknows\td\n")
    (tmp_path / "valid.txt").write_text("a\tknows\tc\n")
    return tmp_path


def test_kgdataset_reads_the_reference_layout(tmp_path):
    # same five-file layout and defaults as apps/kge/data/preprocess.py:26-99
    from cuke_amd.data import KGDataset
    d = write_dataset(tmp_path)
    ds = KGDataset(d / "entities.dict", d / "relations.dict", d / "train.txt", d / "valid.txt")
    assert ds.n_entities == 4 and ds.n_relations == 2
    h, r, t = ds.train
    assert h.tolist() == [0, 1, 3, 2] and r.tolist() == [0, 1, 0, 1] and t.tolist() == [1, 2, 0, 3]
    assert h.dtype == np.int64
    assert [x.tolist() for x in ds.valid] == [[0], [1], [2]]
    assert ds.test is None
    # column order given by `format` (e.g. head, tail, relation files)
    (d / "htr.txt").write_text("a\tb\tlikes\n")
    assert [x.tolist() for x in ds.read_triple(d / "htr.txt", format=(0, 2, 1))] == [[0], [0], [1]]


def test_sampler_oracle_is_uniform_and_deterministic(oracle):
    a = oracle.sample_negatives(20000, 1000, seed=7, step=3)
    b = oracle.sample_negatives(20000, 1000, seed=7, step=3)
    assert np.array_equal(a, b) and a.min() >= 0 and a.max() < 1000
    assert not np.array_equal(a, oracle.sample_negatives(20000, 1000, seed=7, step=4))
    counts = np.bincount(a, minlength=1000)
    assert abs(counts.mean() - 20) < 1e-9 and counts.max() < 50  # ~Poisson(20) per id
    # splitmix64 known answer (first output of the reference implementation seeded with 0)
    assert int(oracle._splitmix64(np.uint64(0))) == 0xE220A8397B1DCDAF


@pytest.mark.gpu
def test_device_sampler_bit_exact_and_feeds_a_step(oracle, tmp_path):
    import torch
    from cuke_amd.data import KGDataset, TrainSampler
    from cuke_amd.kge import KGEModel
    d = write_dataset(tmp_path)
    ds = KGDataset(d / "entities.dict", d / "relations.dict", d / "train.txt")
    s = TrainSampler(ds.train, ds.n_entities, batch_size=4, neg_sample_size=3, neg_chunk_size=2, seed=11)
    h, r, t, neg = next(s)
    assert neg.numel() == 2 * 3
    assert np.array_equal(neg.cpu().numpy(), oracle.sample_negatives(6, 4, seed=11, step=0))
    h2, r2, t2, neg2 = next(s)
    assert np.array_equal(neg2.cpu().numpy(), oracle.sample_negatives(6, 4, seed=11, step=1))
    big = TrainSampler((np.zeros(8, np.int64),) * 3, 4_000_000, 8, 1024, 8, seed=5)
    _, _, _, nb = next(big)
    assert np.array_equal(nb.cpu().numpy(), oracle.sample_negatives(1024, 4_000_000, seed=5, step=0))
    # the batch goes straight into the score path
    E = torch.randn(4, 8, device="cuda:0"); R = torch.randn(2, 8, device="cuda:0")
    fw = KGEModel("DistMult", E, R).score(h, r, t, neg, chunk=2)
    assert fw.neg.shape == (4, 3)


@pytest.mark.gpu
def test_sampler_alternates_head_and_tail_batches(oracle, tmp_path):
    # apps/kge/data/sampler.py:481-487: odd steps tail, even steps head, starting with tail
    import torch
    from cuke_amd.data import KGDataset, TrainSampler
    from cuke_amd.kge import KGEModel
    d = write_dataset(tmp_path)
    ds = KGDataset(d / "entities.dict", d / "relations.dict", d / "train.txt")
    s = TrainSampler(ds.train, ds.n_entities, batch_size=4, neg_sample_size=3, neg_chunk_size=2, seed=3, mode="both")
    E = torch.randn(4, 8, device="cuda:0"); R = torch.randn(2, 8, device="cuda:0")
    m = KGEModel("TransE", E, R)
    modes = []
    for _ in range(4):
        h, r, t, neg = next(s)
        modes.append(s.neg_mode)
        fw = m.score(h, r, t, neg, chunk=2, neg_mode=s.neg_mode)
        _, want = oracle.score("TransE", E.cpu().numpy(), R.cpu().numpy(), None, h.cpu().numpy(), r.cpu().numpy(),
                               t.cpu().numpy(), neg.cpu().numpy(), 2, neg_mode=s.neg_mode)
        np.testing.assert_allclose(fw.neg.cpu().numpy(), want, rtol=1e-5, atol=1e-6)
    assert modes == ["tail", "head", "tail", "head"]
    assert TrainSampler(ds.train, ds.n_entities, 4, 3, 2, mode="head").neg_mode == "head"
    with pytest.raises(ValueError):
        TrainSampler(ds.train, ds.n_entities, 4, 3, 2, mode="sideways")
