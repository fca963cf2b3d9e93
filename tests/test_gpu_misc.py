"""Margin loss and the reference-compatible chunk inspector on the GPU against the oracle."""
import numpy as np
import pytest
import torch

from helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("B,N", [(64, 9), (1024, 256), (5, 1)])
@pytest.mark.parametrize("sign", [1.0, -1.0])
def test_margin_loss(oracle, B, N, sign):
    from cuke_amd.kge import margin_loss
    rng = np.random.default_rng(B + N)
    pos = rng.standard_normal(B).astype(np.float32)
    neg = rng.standard_normal((B, N)).astype(np.float32)
    loss, dpos, dneg = margin_loss(torch.from_numpy(pos).to(DEV), torch.from_numpy(neg).to(DEV), 0.7, sign)
    rl, rdp, rdn = oracle.margin_loss(pos, neg, 0.7, sign)
    assert_close(loss.cpu().numpy(), np.array([rl], np.float32), what="loss")
    assert_close(dpos.cpu().numpy(), rdp, what="dpos")
    assert np.array_equal(dneg.cpu().numpy(), rdn)


def test_build_index_matches_reference_restatement(oracle):
    from cuke_amd.kge import inspector
    rng = np.random.default_rng(5)
    for rel_num, n in ((7, 16 * 64), (1345, 8192), (3, 16 * 10), (40, 16 * 33 + 5)):
        r = np.sort(rng.integers(0, rel_num, n)).astype(np.int64)
        uniq, buf, cnt = inspector(torch.from_numpy(r).to(DEV), rel_num)
        ru, rb, rc, undefined = oracle.build_index(r, rel_num)
        keep = np.ones(ru.shape[0], bool)
        if undefined:  # chunks with 16 distinct ids have no defined result in the reference
            keep = np.array([len(set(c)) < 16 for c in r[: ru.shape[0] * 16].reshape(-1, 16)])
        assert np.array_equal(uniq.cpu().numpy()[keep], ru[keep])
        assert np.array_equal(buf.cpu().numpy()[keep], rb[keep])
        assert np.array_equal(cnt.cpu().numpy()[keep], rc[keep])


def test_build_index_exhaustive_three_values(oracle):
    from cuke_amd.kge import inspector
    rows = [[0] * a + [1] * b + [2] * (16 - a - b) for a in range(17) for b in range(17 - a)]
    r = np.array(rows, np.int64).reshape(-1)
    uniq, buf, cnt = inspector(torch.from_numpy(r).to(DEV), 5)
    ru, rb, rc, _ = oracle.build_index(r, 5)
    assert np.array_equal(uniq.cpu().numpy(), ru)
    assert np.array_equal(buf.cpu().numpy(), rb)
    assert np.array_equal(cnt.cpu().numpy(), rc)


def test_build_index_chunks_of_every_number_of_distinct_values(oracle):
    """1 to 15 distinct values per chunk, sorted and unsorted, ties between run lengths: the HIP kernel against
    the oracle, which the CPU suite pins on the same chunk family against the reference kernel run in lockstep."""
    from cuke_amd.kge import inspector
    rng = np.random.default_rng(21)
    rel_num = 40
    chunks = []
    for distinct in range(1, 16):
        for rep in range(40):
            vals = rng.choice(rel_num, distinct, replace=False)
            row = np.concatenate([vals, rng.choice(vals, 16 - distinct)])
            chunks.append(np.sort(row) if rep % 2 == 0 else rng.permutation(row))
    r = np.concatenate(chunks).astype(np.int64)
    uniq, buf, cnt = inspector(torch.from_numpy(r).to(DEV), rel_num)
    ru, rb, rc, undefined = oracle.build_index(r, rel_num)
    assert not undefined
    assert np.array_equal(uniq.cpu().numpy(), ru)
    assert np.array_equal(buf.cpu().numpy(), rb)
    assert np.array_equal(cnt.cpu().numpy(), rc)


def test_check_indices():
    import ctypes as C
    from cuke_amd import _lib
    idx = torch.tensor([0, 5, 9], dtype=torch.int64, device=DEV)
    flag = torch.zeros(1, dtype=torch.int32, device=DEV)
    L = _lib.lib()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.kge_check_indices(C.c_void_p(idx.data_ptr()), 3, 10, C.c_void_p(flag.data_ptr()), st) == 0
    assert int(flag.item()) == 0
    assert L.kge_check_indices(C.c_void_p(idx.data_ptr()), 3, 9, C.c_void_p(flag.data_ptr()), st) == 0
    assert int(flag.item()) == 1


@pytest.mark.parametrize("dim", [64, 22, 400])
def test_sparse_optimizer_steps(oracle, dim):
    """SGD / row-wise Adagrad on (unique ids, gradient rows) exactly as backward leaves them."""
    from cuke_amd.kge import inspect, sparse_sgd, sparse_adagrad
    rng = np.random.default_rng(dim)
    n_rows = 3000
    table = rng.standard_normal((n_rows, dim)).astype(np.float32)
    state = rng.random(n_rows).astype(np.float32)
    idx = rng.integers(0, n_rows, 1500)
    ins = inspect([torch.from_numpy(idx).to(DEV)], n_rows)
    U = ins.num_unique
    rows_full = rng.standard_normal((1500, dim)).astype(np.float32)  # capacity n, first U rows valid
    rows_dev = torch.from_numpy(rows_full).to(DEV)
    ids = ins.ids().cpu().numpy()
    t_dev = torch.from_numpy(table).to(DEV)
    sparse_sgd(t_dev, ins, rows_dev, 0.05)
    assert_close(t_dev.cpu().numpy(), oracle.sparse_sgd(table, ids, rows_full[:U], 0.05), what="sgd", rows=True)
    t_dev = torch.from_numpy(table).to(DEV); s_dev = torch.from_numpy(state).to(DEV)
    sparse_adagrad(t_dev, s_dev, ins, rows_dev, 0.05)
    want_t, want_s = oracle.sparse_adagrad(table, state, ids, rows_full[:U], 0.05)
    assert_close(t_dev.cpu().numpy(), want_t, what="adagrad table", rows=True)
    assert_close(s_dev.cpu().numpy(), want_s, what="adagrad state")


def test_current_stream_lookup_follows_the_stream_context():
    """The step loop's cached lookup of torch's current stream: the Stream object that belongs to the
    raw handle of the moment, inside and outside a stream context, and the same object on a second call."""
    from cuke_amd import kge
    idx = torch.cuda.current_device()
    default = kge._current_stream(idx)
    assert default.cuda_stream == torch.cuda.current_stream().cuda_stream
    other = torch.cuda.Stream()
    with torch.cuda.stream(other):
        inside = kge._current_stream(idx)
        assert inside.cuda_stream == other.cuda_stream
        assert kge._current_stream(idx) is inside
        assert kge._stream().value == other.cuda_stream
    assert kge._current_stream(idx) is default
    assert (kge._stream().value or 0) == torch.cuda.current_stream().cuda_stream
