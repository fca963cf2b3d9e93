"""Committed golden vectors (tests/golden/kge_small.npz, written by tests/golden/make_golden.py from float64
torch library operations and autograd): the CPU oracle (no GPU needed) and the HIP path (gpu) both have to
reproduce them within the fp32 parity bar, for every score function, both norm orders and both negative modes."""
import os

import numpy as np
import pytest

from helpers import assert_close

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kge_small.npz")
CASES = ["TransE_p1", "TransE_p2", "TransH_p1", "TransH_p2", "TransR_p1", "TransR_p2", "DistMult_p2", "ComplEx_p2",
         "RotatE_p2", "TransF_p2", "RESCAL_p2"]


def load(case):
    z = np.load(GOLD)  # allow_pickle stays False
    get = lambda k: z[f"{case}/{k}"] if f"{case}/{k}" in z.files else None  # noqa: E731
    chunk, n_neg, p = (int(x) for x in z[f"{case}/meta"])
    return get, chunk, n_neg, p, float(z[f"{case}/gamma"][0])


def dense(ids, rows, n):
    out = np.zeros((n,) + rows.shape[1:], np.float64)
    out[np.asarray(ids)] = rows
    return out


def check_grads(get, mode, g_ids_e, g_rows_e, g_ids_r, g_rows_r, g_rows_a, what, rtol):
    gE = get(f"{mode}/gE")
    assert_close(dense(g_ids_e, g_rows_e, gE.shape[0]), gE, rtol=rtol, what=what + " dE")
    gR = get(f"{mode}/gR")
    if gR is not None and g_rows_r is not None and g_rows_r.size:
        assert_close(dense(g_ids_r, g_rows_r, gR.shape[0]), gR, rtol=rtol, what=what + " dR")
    gA = get(f"{mode}/gA")
    if gA is not None:
        assert_close(dense(g_ids_r, g_rows_a, gA.shape[0]), gA, rtol=rtol, what=what + " dA")


@pytest.mark.parametrize("mode", ["tail", "head"])
@pytest.mark.parametrize("case", CASES)
def test_oracle_reproduces_golden_vectors(oracle, case, mode):
    get, chunk, n_neg, p, gamma = load(case)
    model = case.split("_")[0]
    E, R, A = get("E"), get("R"), get("A")
    h, r, t, neg = get("h"), get("r"), get("t"), get("neg")
    pos, negs = oracle.score(model, E, R, A, h, r, t, neg, chunk, p=p, gamma=gamma, neg_mode=mode)
    assert_close(pos, get(f"{mode}/pos"), what=f"{case} {mode} pos")
    assert_close(negs, get(f"{mode}/neg"), what=f"{case} {mode} neg")
    g = oracle.backward(model, E, R, A, h, r, t, neg, chunk, get("dpos"), get("dneg"), p=p, neg_mode=mode)
    check_grads(get, mode, g.ent_ids, g.ent_rows, g.rel_ids, g.rel_rows, g.aux_rows, f"{case} {mode}", 1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["tail", "head"])
@pytest.mark.parametrize("case", CASES)
def test_hip_path_reproduces_golden_vectors(case, mode):
    import torch
    from cuke_amd.kge import KGEModel
    get, chunk, n_neg, p, gamma = load(case)
    model = case.split("_")[0]
    dev = torch.device("cuda:0")
    tt = lambda x: None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(dev)  # noqa: E731
    R = get("R")
    m = KGEModel(model, tt(get("E")), tt(R) if R is not None and R.size else None, tt(get("A")), norm_p=p, gamma=gamma)
    fw = m.score(tt(get("h")), tt(get("r")), tt(get("t")), tt(get("neg")), chunk, neg_mode=mode)
    assert_close(fw.pos.cpu().numpy(), get(f"{mode}/pos"), what=f"{case} {mode} pos")
    assert_close(fw.neg.cpu().numpy(), get(f"{mode}/neg"), what=f"{case} {mode} neg")
    g = m.backward(fw, tt(get("dpos")), tt(get("dneg")))
    cpu = lambda x: None if x is None else x.cpu().numpy()  # noqa: E731
    check_grads(get, mode, cpu(g.ent_ids), cpu(g.ent_rows), cpu(g.rel_ids), cpu(g.rel_rows), cpu(g.aux_rows),
                f"{case} {mode}", 1e-5)
