"""CPU oracle for the KGE score path -- TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this.  It wraps ``kge_oracle.c`` (the
serial restatement of the loops cuke's ``codegen.cpu`` emits, see that file's
header for the reference citations) through ctypes and adds the index
"inspector" oracle, which is numpy's ``unique`` + stable ``argsort``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

MODELS = {
    "TransE": 0,
    "TransH": 1,
    "TransR": 2,
    "DistMult": 3,
    "ComplEx": 4,
    "RotatE": 5,
    "TransF": 6,
    "RESCAL": 7,
}


def build(force: bool = False) -> None:
    """Compile the oracle libraries with gcc (oracle/Makefile)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


_libs: dict[str, ctypes.CDLL] = {}


def _lib(fast=False) -> ctypes.CDLL:
    """fast: False = the checker (-O2); "o3" = -O3 one thread; True / "omp" = -O3 + OpenMP over the batch;
    "o0" = -O0 one thread (the flags the reference's JIT build of its generated C++ gets)."""
    name = {False: "libkge_oracle.so", "o3": "libkge_oracle_o3.so", True: "libkge_oracle_omp.so",
            "omp": "libkge_oracle_omp.so", "o0": "libkge_oracle_o0.so"}[fast]
    if name not in _libs:
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        _libs[name] = lib
    return _libs[name]


def _fp(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int64)


def rel_width(model: str, d: int) -> int:
    return {"RotatE": d // 2, "RESCAL": 0}.get(model, d)


def aux_width(model: str, d: int) -> int:
    return {"TransH": d, "TransR": d * d, "RESCAL": d * d}.get(model, 0)


def residual(model, E, R, A, h, r, t):
    """[B, d] residual vector of TransE / TransH / TransR (the reference's output)."""
    E, R, A = _f32(E), _f32(R), _f32(A)
    h, r, t = _i64(h), _i64(r), _i64(t)
    B, d = h.shape[0], E.shape[1]
    out = np.empty((B, d), np.float32)
    rc = _lib().orc_residual(
        ctypes.c_int(MODELS[model]), ctypes.c_int64(B), ctypes.c_int64(d),
        _fp(E), _fp(R), _fp(A), _fp(h), _fp(r), _fp(t), _fp(out))
    if rc != 0:
        raise ValueError(f"oracle residual: model {model} has no residual form")
    return out


def _neg_head(neg_mode) -> int:
    if neg_mode not in ("tail", "head"):
        raise ValueError("neg_mode is 'tail' or 'head'")
    return 1 if neg_mode == "head" else 0


def score(model, E, R, A, h, r, t, neg=None, chunk=0, p=2, gamma=0.0, fast=False,
          want_pos=True, neg_mode="tail"):
    """pos[B] and (when ``neg`` is given) negs[B, N] scores; the shared negatives replace the
    tail (``neg_mode='tail'``) or the head (``'head'``) of every positive of their chunk."""
    E, R, A = _f32(E), _f32(R), _f32(A)
    h, r, t, neg = _i64(h), _i64(r), _i64(t), _i64(neg)
    B, d = h.shape[0], E.shape[1]
    pos = np.empty((B,), np.float32) if want_pos else None
    negs = None
    C = N = 0
    if neg is not None:
        C = int(chunk)
        assert C > 0 and B % C == 0
        N = neg.shape[0] // (B // C)
        assert N * (B // C) == neg.shape[0]
        negs = np.empty((B, N), np.float32)
    rc = _lib(fast).orc_score(
        ctypes.c_int(MODELS[model]), ctypes.c_int(p), ctypes.c_float(gamma),
        ctypes.c_int64(B), ctypes.c_int64(d), _fp(E), _fp(R), _fp(A),
        _fp(h), _fp(r), _fp(t), _fp(neg), ctypes.c_int64(C), ctypes.c_int64(N),
        ctypes.c_int(_neg_head(neg_mode)), _fp(pos), _fp(negs))
    assert rc == 0
    return pos, negs


@dataclass
class Inspection:
    """What the index inspector must produce for one index array."""
    unique_ids: np.ndarray   # int64 [U], strictly ascending
    seg_offsets: np.ndarray  # int64 [U+1], seg_offsets[0] = 0, seg_offsets[U] = n
    perm: np.ndarray         # int64 [n], stable sort permutation: idx[perm] ascending
    inverse: np.ndarray      # int64 [n], unique_ids[inverse] == idx


def inspect(idx) -> Inspection:
    idx = _i64(idx)
    uniq, inverse, counts = np.unique(idx, return_inverse=True, return_counts=True)
    perm = np.argsort(idx, kind="stable")
    seg = np.zeros(uniq.shape[0] + 1, np.int64)
    np.cumsum(counts, out=seg[1:])
    return Inspection(uniq.astype(np.int64), seg, perm.astype(np.int64),
                      inverse.reshape(-1).astype(np.int64))


@dataclass
class SparseGrads:
    ent_ids: np.ndarray
    ent_rows: np.ndarray
    rel_ids: np.ndarray
    rel_rows: np.ndarray | None
    aux_rows: np.ndarray | None


def backward(model, E, R, A, h, r, t, neg=None, chunk=0, dpos=None, dneg=None, p=2, fast=False,
             neg_mode="tail") -> SparseGrads:
    """Sparse row gradients (unique ids ascending, one row per id) per table."""
    E, R, A = _f32(E), _f32(R), _f32(A)
    h, r, t, neg = _i64(h), _i64(r), _i64(t), _i64(neg)
    dpos, dneg = _f32(dpos), _f32(dneg)
    B, d = h.shape[0], E.shape[1]
    C = N = 0
    occ = [h, t]
    if neg is not None:
        C = int(chunk)
        N = neg.shape[0] // (B // C)
        occ.append(neg)
    ins_e = inspect(np.concatenate(occ))
    ins_r = inspect(r)
    slot_h = np.ascontiguousarray(ins_e.inverse[:B])
    slot_t = np.ascontiguousarray(ins_e.inverse[B:2 * B])
    slot_n = np.ascontiguousarray(ins_e.inverse[2 * B:]) if neg is not None else None
    slot_r = np.ascontiguousarray(ins_r.inverse)
    rw, aw = rel_width(model, d), aux_width(model, d)
    gE = np.zeros((ins_e.unique_ids.shape[0], d), np.float32)
    gR = np.zeros((ins_r.unique_ids.shape[0], rw), np.float32) if rw else None
    gA = np.zeros((ins_r.unique_ids.shape[0], aw), np.float32) if aw else None
    rc = _lib(fast).orc_backward(
        ctypes.c_int(MODELS[model]), ctypes.c_int(p), ctypes.c_int64(B), ctypes.c_int64(d),
        _fp(E), _fp(R), _fp(A), _fp(h), _fp(r), _fp(t), _fp(neg),
        ctypes.c_int64(C), ctypes.c_int64(N), ctypes.c_int(_neg_head(neg_mode)), _fp(dpos), _fp(dneg),
        _fp(slot_h), _fp(slot_t), _fp(slot_n), _fp(slot_r),
        ctypes.c_int64(gE.shape[0]), ctypes.c_int64(ins_r.unique_ids.shape[0]),
        _fp(gE), _fp(gR), _fp(gA))
    assert rc == 0
    return SparseGrads(ins_e.unique_ids, gE, ins_r.unique_ids, gR, gA)


def l1_ambiguous_rows(model, E, R, A, h, r, t, neg=None, chunk=0, eps=6e-8, fast=False, neg_mode="tail"):
    """Rows of the sparse L1 gradient (TransE / TransH) that a sign ambiguity can reach: for every unique
    entity id and every unique relation id (same order as ``backward``) the number of residual elements with
    |u| <= eps in the triples and pairs that touch the row (0 = the row is clear), plus their total."""
    E, R, A = _f32(E), _f32(R), _f32(A)
    h, r, t, neg = _i64(h), _i64(r), _i64(t), _i64(neg)
    B, d = h.shape[0], E.shape[1]
    C = N = 0
    occ = [h, t]
    if neg is not None:
        C = int(chunk)
        N = neg.shape[0] // (B // C)
        occ.append(neg)
    ins_e, ins_r = inspect(np.concatenate(occ)), inspect(r)
    slot_h = np.ascontiguousarray(ins_e.inverse[:B])
    slot_t = np.ascontiguousarray(ins_e.inverse[B:2 * B])
    slot_n = np.ascontiguousarray(ins_e.inverse[2 * B:]) if neg is not None else None
    flag_e = np.zeros(ins_e.unique_ids.shape[0], np.int32)
    flag_r = np.zeros(ins_r.unique_ids.shape[0], np.int32)
    fn = _lib(fast).orc_l1_ambiguous
    fn.restype = ctypes.c_int64
    n = fn(ctypes.c_int(MODELS[model]), ctypes.c_int64(B), ctypes.c_int64(d), _fp(E), _fp(R), _fp(A),
           _fp(h), _fp(r), _fp(t), _fp(neg), ctypes.c_int64(C), ctypes.c_int64(N),
           ctypes.c_int(_neg_head(neg_mode)), ctypes.c_float(eps), _fp(slot_h), _fp(slot_t), _fp(slot_n),
           _fp(np.ascontiguousarray(ins_r.inverse)), _fp(flag_e), _fp(flag_r))
    if n < 0:
        raise ValueError(f"{model} has no L1 form")
    return flag_e, flag_r, int(n)


def margin_loss(pos, neg, margin, sign=1.0):
    pos, neg = _f32(pos), _f32(neg)
    B, N = neg.shape
    loss = ctypes.c_float(0.0)
    dpos = np.empty((B,), np.float32)
    dneg = np.empty((B, N), np.float32)
    _lib().orc_margin_loss(_fp(pos), _fp(neg), ctypes.c_int64(B), ctypes.c_int64(N),
                           ctypes.c_float(margin), ctypes.c_float(sign), ctypes.byref(loss),
                           _fp(dpos), _fp(dneg))
    return float(loss.value), dpos, dneg


def build_index(r, rel_num):
    """uniq[batch/16,16], buf[batch/16,16], cnt[batch/16] of the reference's chunk inspector.

    Returns (uniq, buf, cnt, undefined) where ``undefined`` is True when some chunk has 16
    distinct ids (out-of-bounds write in the reference, no defined result)."""
    r = _i64(r)
    nb = r.shape[0] // 16
    uniq = np.zeros((nb, 16), np.int64)
    buf = np.zeros((nb, 16), np.int64)
    cnt = np.zeros((nb,), np.int64)
    rc = _lib().orc_build_index(_fp(r), ctypes.c_int64(r.shape[0]), ctypes.c_int64(rel_num),
                                _fp(uniq), _fp(buf), _fp(cnt))
    return uniq, buf, cnt, bool(rc)


def sparse_sgd(table, ids, rows, lr):
    """Returns the updated copy of ``table``."""
    table, rows, ids = _f32(table).copy(), _f32(rows), _i64(ids)
    _lib().orc_sparse_sgd(_fp(table), ctypes.c_int64(table.shape[1]), _fp(ids), ctypes.c_int64(ids.shape[0]),
                          _fp(rows), ctypes.c_float(lr))
    return table


def sparse_adagrad(table, state, ids, rows, lr, eps=1e-10):
    """Returns the updated copies of (table, state)."""
    table, state, rows, ids = _f32(table).copy(), _f32(state).copy(), _f32(rows), _i64(ids)
    _lib().orc_sparse_adagrad(_fp(table), _fp(state), ctypes.c_int64(table.shape[1]), _fp(ids),
                              ctypes.c_int64(ids.shape[0]), _fp(rows), ctypes.c_float(lr), ctypes.c_float(eps))
    return table, state


def _splitmix64(z):
    """splitmix64 finaliser on uint64 scalars or arrays (wrap-around arithmetic intended)."""
    with np.errstate(over="ignore"):
        z = np.asarray(z, dtype=np.uint64)
        z = (z + np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def sample_negatives(count, n_ent, seed, step):
    """numpy restatement of the device negative sampler (see kge_sample_negatives in the C header)."""
    with np.errstate(over="ignore"):
        i = np.arange(count, dtype=np.uint64)
        base = np.uint64(seed) ^ _splitmix64(np.uint64(step))
        x = _splitmix64(base ^ (i * np.uint64(0x9E3779B97F4A7C15)))
    # 64 x 64 -> high 64 bits, with Python integers (exact)
    return np.array([(int(v) * int(n_ent)) >> 64 for v in x], dtype=np.int64)


def threads(fast=True) -> int:
    return int(_lib(fast).orc_threads())
