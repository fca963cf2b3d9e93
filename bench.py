#!/usr/bin/env python3
"""Benchmark of the KGE score path on one MI355X.

A step is one pass over one batch of synthetic input with every table and index
array already resident in HBM: index inspection (radix sort + dedup of the entity
and relation ids) -> scores of the positives and of the shared negatives ->
(margin loss) -> sparse row gradients.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|cfg2_distmult|...]

With no --workload every benchmark configuration is timed in the one run: the headline fields
of the line are those of the largest single-GPU configuration (cfg5_transh) and `per_workload`
holds the same fields for the other five.  Per workload:
  * the timed loop rotates over --batches distinct seeded batches (index sets), so the gathered
    rows of a step are not left in the caches by the step before; the same loop over one batch
    is reported beside it (`ms_per_step_same_batch`);
  * before anything is timed the step's own inputs are spot-checked against the CPU oracle
    (sampled pair scores, positive scores and whole gradient rows); a mismatch aborts the run;
  * `roofline` describes the kernel with the largest share of the step, timed live with HIP
    events recorded behind every kernel on the stream the kernels run on.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
WARMUP_MIN_S = 0.02         # least untimed warm-up in front of every timed region
FP32_PEAK_TFLOPS = 157.3    # MI355X fp32 vector / fp32 MFMA, published

ALL_WORKLOADS = ["cfg5_transh", "cfg1_transe", "cfg2_distmult", "cfg2_complex", "cfg3_transr", "cfg4_rotate"]
# which roof binds a workload by arithmetic (flop per algorithmic byte against the ridge of 19.7)
BOUND = {"cfg1_transe": "hbm", "cfg2_distmult": "fp32", "cfg2_complex": "fp32", "cfg3_transr": "hbm",
         "cfg4_rotate": "fp32", "cfg5_transh": "fp32", "ref_transr_8192x512": "hbm"}

# Kernels of the profile summaries (profiles/score_path_kernels_<workload>.txt) behind a timeline label.
PROFILE_KERNELS = {
    "score_pos_kernel": ["score_pos_kernel"],
    "score_neg_kernel": ["score_neg_kernel", "score_neg_mfma_kernel", "score_neg_finish_kernel"],
    "bwd_tile_kernel": ["bwd_tile_kernel"],
    "bwd_pos_kernel": ["bwd_pos_kernel"],
    "seg_reduce_l1": ["seg_reduce_l1"],
    "seg_reduce_l2": ["seg_reduce_l2"],
    "transr_plan_kernel + transr_gemm_kernel<fwd>": ["transr_plan_kernel", "transr_gemm_kernel<0>"],
    "transr_plan_kernel + transr_fwd_back_kernel": ["transr_plan_kernel", "transr_fwd_back_kernel"],
    "transr_gemm_kernel<dX>": ["transr_gemm_kernel<2>"],
    "transr_dm_kernel": ["transr_dm_kernel"],
}


def measured_traffic(workload, label, matrix_core_tiles=False, dense=False):
    """HBM bytes per launch of the kernel(s) behind a timeline label, read from the committed profile
    summary of the workload: rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of this script (KiB
    per dispatch), each scaled by what the same counter reads for the 256 MiB copy kernel of
    --calibrate-copy (the file states the factors).  Returns (bytes or None, the profile's kernel
    names) so that the line shows which compiled kernels the figure belongs to.  matrix_core_tiles: the
    workload's tile kernels are the matrix-core forms (the profile of such a workload also holds the
    vector-ALU forms that the run times beside them).  dense: rows of the profile's second table (the
    TransR step that writes every projection gradient dense) replace those of the first."""
    import re
    path = os.path.join(ROOT, "profiles", f"score_path_kernels_{workload}.txt")
    want = PROFILE_KERNELS.get(label)
    if not want or not os.path.exists(path):
        return None, []
    rows, in_table = {}, False
    for line in open(path):
        if line.startswith("## HBM traffic per dispatch"):
            in_table = dense or "dense" not in line
            continue
        if in_table and line.startswith("## "):
            in_table = False
            continue
        m = re.match(r"^(kge::.*?)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line) if in_table else None
        if m:
            rows[m.group(1)] = (float(m.group(4)) + float(m.group(5))) * 1e6
    total, names = 0.0, []
    for key in want:
        for name, by in rows.items():
            base = name.replace("kge::", "")
            if base == key or base.startswith(key + "<") or (key.endswith(">") and base.replace(" ", "") == key.replace(" ", "")):
                if matrix_core_tiles and ((key == "score_neg_kernel") or (key == "bwd_tile_kernel" and not base.endswith("true>"))):
                    continue  # the vector-ALU form of a tile kernel
                total += by
                names.append(name)
    return (int(total) if names else None), names


# ---- algorithmic bytes and flops ---------------------------------------------------------------
def algorithmic_bytes(w, u_ent, u_rel):
    """Bytes the step has to move by the problem statement alone: every gathered row once per
    gather (h, r, t [, w] per positive; negatives once per chunk), 8 B per index, 4 B per score;
    backward: 4 B per upstream score gradient, the same row reads again, one row write per
    distinct row and 8 B per distinct id.  TransR: every distinct projection once per pass and
    one dense d x d gradient per distinct relation."""
    B, d, rd, N = w.batch, w.dim, w.rel_dim, w.n_neg
    nn = w.n_chunks * N
    aux_row = d if w.model == "TransH" else 0
    rows = 4 * (B * (2 * d + rd + aux_row) + nn * d)
    if w.model in ("TransR", "RESCAL"):
        rows += 4 * u_rel * d * d
    idx = 8 * (3 * B + nn)
    scores = 4 * B * (1 + N)
    fwd = rows + idx + scores
    bwd = scores + rows + idx + 4 * (u_ent * d + u_rel * (rd + aux_row)) + 8 * (u_ent + u_rel)
    if w.model in ("TransR", "RESCAL"):
        # one gradient per distinct relation: dense d x d, or the 2 d floats per triple of a group left factored
        bwd += 4 * (w.dense_rel * d * d + 2 * w.factored_rows * d) if hasattr(w, "dense_rel") else 4 * u_rel * d * d
    return fwd, bwd


# flop per (pair, element of the reduction axis) of the forward pass: multiply-add for the dot
# products; sub, fma with w.t', abs/accumulate and the w.t' multiply-add for TransH (6); the
# complex difference, modulus and accumulate for RotatE (7 per complex element, its square root
# not counted).  Backward does the same pair work in both orientations: twice the forward count.
PAIR_FLOPS = {"DistMult": 2, "ComplEx": 2, "TransE": 3, "TransH": 6, "RotatE": 7, "TransF": 2}


def algorithmic_flops(w):
    klen = w.dim // 2 if w.model == "RotatE" else w.dim
    if w.model in ("TransR", "RESCAL"):
        f = 2 * w.batch * w.dim * w.dim
        return f, 2 * f
    f = PAIR_FLOPS[w.model] * w.batch * (1 + w.n_neg) * klen
    return f, 2 * f


def kernel_model(w, label, u_ent, u_rel):
    """(algorithmic bytes, algorithmic flops, arithmetic unit) of ONE launch of the kernel `label`."""
    B, d, rd, N = w.batch, w.dim, w.rel_dim, w.n_neg
    nn = w.n_chunks * N
    klen = d // 2 if w.model == "RotatE" else d
    aux_row = d if w.model == "TransH" else 0
    dot = w.model in ("DistMult", "ComplEx")
    pair_flops = PAIR_FLOPS.get(w.model, 0) * B * N * klen
    l2 = w.model in ("TransE", "TransH") and w.norm_p == 2
    if label == "score_pos_kernel":
        by = 4 * B * (2 * d + rd + aux_row) + 8 * 3 * B + 4 * B
        by += 4 * B * d if w.model == "RotatE" else 0
        by += 4 * B if w.model == "TransH" else 0
        return by, PAIR_FLOPS.get(w.model, 2) * B * klen, "valu"
    if label == "score_neg_kernel":
        if w.model == "RotatE":  # one rotated-head row per positive, written by the positive kernel of the same call
            by = 4 * (B * d + nn * d) + 8 * nn + 4 * B * N
        else:
            out_planes = 3 if w.model == "TransH" else 1
            by = 4 * (B * (d + rd + aux_row) + nn * d) + 8 * (2 * B + nn) + 4 * out_planes * B * N
        return by, pair_flops, "mfma" if dot else "valu"
    if label == "bwd_tile_kernel":
        planes_in = 1 + (1 if l2 else 0) + (2 if w.model == "TransH" else 0)   # dneg, scores, TransH side planes
        rows_in = B * (d if w.model == "RotatE" else d + rd + aux_row) + nn * d
        rows_out = B * d * (2 if w.model == "TransH" else 1) + nn * d
        by = 4 * (rows_in + rows_out) + 8 * (2 * B + nn) + 4 * planes_in * B * N
        return by, 2 * pair_flops, "mfma" if dot else "valu"
    if label == "bwd_pos_kernel":
        g_rows = (B * d * (2 if w.model == "TransH" else 1)) if N else 0
        by = 4 * (B * (2 * d + rd + aux_row) + g_rows + B * (2 * d + rd + aux_row)) + 8 * 3 * B + 8 * B
        return by, 6 * B * klen, "valu"
    if label == "seg_reduce_l1":
        n_occ = 2 * B + nn
        by = 4 * (n_occ * d + B * (rd + aux_row)) + 8 * (n_occ + B) + 4 * (u_ent * d + u_rel * (rd + aux_row))
        return by, n_occ * d, "valu"
    if label == "seg_reduce_l2":
        return 4 * (u_ent * d) // 8, 0, "valu"
    if label.startswith("transr_plan_kernel") or label == "transr_gemm_kernel<dX>":
        by = 4 * (u_rel * d * d + 3 * B * d + u_rel * d) + 8 * 3 * B
        if "fwd_back" in label:  # the forward kernel also does the backward pass's product with the transposed projections
            return 2 * by, 4 * B * d * d, "mfma"
        return by, 2 * B * d * d, "mfma"
    # dM: the x rows (two entity rows for TransR) and the residual rows in, one gradient per distinct relation out
    # (dense d x d, or 2 d floats per triple for the groups left factored: `dense_rel` / `factored_rows` say how many)
    dm_out = 4 * (w.dense_rel * d * d + 2 * w.factored_rows * d) if hasattr(w, "dense_rel") else 4 * u_rel * d * d
    if label == "transr_dm_kernel":
        return dm_out + 4 * 3 * B * d, 2 * B * d * d, "mfma"
    return 0, 0, "valu"


# ---- timing ------------------------------------------------------------------------------------
def time_events(fn, iters, torch):
    """Average milliseconds per call of fn over `iters` back-to-back calls, by HIP events on the
    stream the kernels are launched on (torch's current stream)."""
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


# ---- parity spot check of the inputs that are timed ----------------------------------------------
class SpotCheckError(RuntimeError):
    pass


def _tol_ok(got, ref, rows, rtol=1e-5):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    rms = np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True)) if rows else float(np.sqrt(np.mean(ref * ref)))
    err = np.abs(got - ref)
    bound = rtol * np.abs(ref) + rtol * rms
    return err, bound


def spot_check(w, model, step, ix, n_pairs=4096, n_pos=512, n_rows=64, n_rel_rows=8, max_triples=40_000, seed=7):
    """Runs one step on the device and compares, against the CPU oracle evaluated on rows copied
    back from the device tables: `n_pairs` sampled (positive, negative) pair scores, `n_pos`
    positive scores and the complete gradient rows of `n_rows` sampled entity ids and `n_rel_rows`
    relation ids.  A gradient row is checked exactly: the oracle differentiates every triple and
    pair of the batch that touches the row, written out as explicit triples.  Bar: |got - ref| <=
    1e-5 |ref| + 1e-5 rms(ref) (rms per gradient row).  L1 gradients are sums of signs of
    residual elements, and an element within an ulp of zero may take either sign: up to 0.5 % of
    the elements of the sampled rows may differ, each by at most two flips of the largest
    upstream gradient.  RotatE unit vectors u/|u| with tiny |u| admit 1e-4 of the elements within
    4x the bound.  Raises SpotCheckError on a mismatch."""
    import torch
    import oracle
    oracle.build()
    rng = np.random.default_rng(seed)
    h, r, t = (ix[k].cpu().numpy() for k in ("h", "r", "t"))
    neg = ix["neg"].cpu().numpy() if "neg" in ix else None
    B, N, C = w.batch, w.n_neg, w.chunk
    do_bwd = w.backward
    step.select(0)
    step.run(do_bwd)
    torch.cuda.synchronize()
    pos_dev = step.pos.cpu().numpy()
    neg_dev = step.neg.cpu().numpy() if step.neg is not None else None
    report = {}

    def gathered(ent_ids, rel_ids):
        """Compact host copies of the device rows for these ids + the id -> compact index maps."""
        ue, ur = np.unique(ent_ids), np.unique(rel_ids)
        dev = model.E.device
        E = model.E[torch.from_numpy(ue).to(dev)].cpu().numpy()
        R = model.R[torch.from_numpy(ur).to(dev)].cpu().numpy() if model.R is not None and model.rel_dim else None
        A = model.A[torch.from_numpy(ur).to(dev)].cpu().numpy() if model.A is not None else None
        return E, R, A, (lambda x: np.searchsorted(ue, x)), (lambda x: np.searchsorted(ur, x))

    # -- scores
    bs = rng.choice(B, size=min(n_pos, B), replace=False)
    fh, fr, ft, want = [h[bs]], [r[bs]], [t[bs]], [pos_dev[bs]]
    if neg is not None:
        pb = rng.integers(0, B, n_pairs)
        pk = rng.integers(0, N, n_pairs)
        fh.append(h[pb]), fr.append(r[pb]), ft.append(neg[(pb // C) * N + pk]), want.append(neg_dev[pb, pk])
    fh, fr, ft, want = (np.concatenate(x) for x in (fh, fr, ft, want))
    E, R, A, me, mr = gathered(np.concatenate([fh, ft]), fr)
    ref, _ = oracle.score(w.model, E, R, A, me(fh), mr(fr), me(ft), p=w.norm_p, gamma=w.gamma)
    err, bound = _tol_ok(want, ref, rows=False)
    if (err > bound).any():
        i = int(np.argmax(err - bound))
        raise SpotCheckError(f"{w.name}: {int((err > bound).sum())}/{ref.size} sampled scores differ from the oracle; "
                             f"worst: device {want[i]!r} oracle {ref[i]!r}")
    report["scores_checked"] = int(ref.size)
    if not do_bwd:
        return report

    # -- upstream gradients as the device step used them
    if w.loss == "margin":
        sign = step.sign
        loss_ref, _, _ = oracle.margin_loss(pos_dev, neg_dev, w.margin, sign)
        loss_dev = float(step.loss.item())
        if abs(loss_dev - loss_ref) > 1e-5 * max(1.0, abs(loss_ref)):
            raise SpotCheckError(f"{w.name}: margin loss {loss_dev!r} differs from the oracle's {loss_ref!r}")
    dpos = step.dpos.cpu().numpy() if step.dpos is not None else np.zeros(B, np.float32)
    dneg = step.dneg.cpu().numpy() if step.dneg is not None else None
    g = step.sparse_grads()
    ent_ids, rel_ids = g.ent_ids.cpu().numpy(), g.rel_ids.cpu().numpy()
    occ = np.concatenate([h, t] + ([neg] if neg is not None else []))
    if not np.array_equal(ent_ids, np.unique(occ)) or not np.array_equal(rel_ids, np.unique(r)):
        raise SpotCheckError(f"{w.name}: unique ids of the sparse gradients differ from numpy.unique")
    l1 = w.model in ("TransE", "TransH") and w.norm_p == 1
    gmax = float(max(np.abs(dpos).max(), np.abs(dneg).max() if dneg is not None else 0.0))

    def explicit_triples(mask_b_full, neg_slots):
        """Every triple / pair of the batch named by: positives whose whole row set is wanted
        (mask over b: the positive and all its pairs) and negative slots (chunk, k): all pairs of
        the chunk with that negative.  Returned as flat (h, r, t, g) without duplicates."""
        items = set()
        for b in np.flatnonzero(mask_b_full):
            items.add((int(b), -1))
            for k in range(N if neg is not None else 0):
                items.add((int(b), k))
        for (c, k) in neg_slots:
            for b in range(c * C, (c + 1) * C):
                items.add((b, int(k)))
        it = np.array(sorted(items), dtype=np.int64).reshape(-1, 2)
        b_, k_ = it[:, 0], it[:, 1]
        is_pos = k_ < 0
        tt = np.where(is_pos, t[b_], neg[(b_ // C) * N + np.maximum(k_, 0)] if neg is not None else t[b_])
        gg = np.where(is_pos, dpos[b_], dneg[b_, np.maximum(k_, 0)] if dneg is not None else 0.0).astype(np.float32)
        return h[b_], r[b_], tt, gg

    def check_rows(kind, ids, dev_rows_of, ref_rows_of):
        bad_total = checked = flips = 0
        for e in ids:
            got, ref = dev_rows_of(e), ref_rows_of(e)
            if ref is None:
                continue
            err, bound = _tol_ok(got, ref, rows=True)
            bad = err > bound
            checked += ref.size
            if bad.any():
                if l1 and (err[bad] <= 4.0 * gmax * (1 + 1e-5)).all():
                    flips += int(bad.sum())
                elif w.model == "RotatE" and (err <= 4 * bound).all():
                    bad_total += int(bad.sum())
                else:
                    i = np.unravel_index(np.argmax(err - bound), err.shape)
                    raise SpotCheckError(f"{w.name}: gradient row of {kind} {int(e)} differs from the oracle at {i}: "
                                         f"device {np.asarray(got)[i]!r} oracle {np.asarray(ref)[i]!r}")
        if checked and flips > 5e-3 * checked:
            raise SpotCheckError(f"{w.name}: {flips}/{checked} L1 gradient elements of {kind} rows differ by sign flips")
        if checked and bad_total > 1e-4 * checked + 1:
            raise SpotCheckError(f"{w.name}: {bad_total}/{checked} RotatE gradient elements of {kind} rows outside the bound")
        return checked, flips

    ent_rows_dev, rel_rows_dev, aux_rows_dev = g.ent_rows, g.rel_rows, g.aux_rows
    seg = g.rel_seg_offsets.cpu().numpy() if g.factor_max else None

    def aux_row_dev(u):
        """Row u of the auxiliary-table gradients; a factored relation group multiplied out on the host."""
        if seg is not None and seg[u + 1] - seg[u] <= g.factor_max:
            x = g.aux_x[seg[u]:seg[u + 1]].cpu().numpy().astype(np.float64)
            q = g.aux_q[seg[u]:seg[u + 1]].cpu().numpy().astype(np.float64)
            return (x.T @ q).reshape(-1)
        return aux_rows_dev[u].cpu().numpy()

    def oracle_rows(fh, fr, ft, fg):
        E, R, A, me, mr = gathered(np.concatenate([fh, ft]), fr)
        ref = oracle.backward(w.model, E, R, A, me(fh), mr(fr), me(ft), None, 0, fg, None, p=w.norm_p)
        return ref, np.unique(np.concatenate([fh, ft])), np.unique(fr)

    # -- entity rows
    def ent_ref(e):
        mb = (h == e) | (t == e)
        slots = [(int(s // N), int(s % N)) for s in np.flatnonzero(neg == e)] if neg is not None else []
        n_tr = int(mb.sum()) * (1 + (N if neg is not None else 0)) + len(slots) * C
        if n_tr > max_triples:
            return None
        fh, fr, ft, fg = explicit_triples(mb, slots)
        ref, ue, _ = oracle_rows(fh, fr, ft, fg)
        return ref.ent_rows[int(np.searchsorted(ue, e))]

    pick = rng.permutation(ent_ids)[: 4 * n_rows]
    done = []

    def ent_ref_capped(e):
        if len(done) >= n_rows:
            return None
        ref = ent_ref(e)
        if ref is not None:
            done.append(e)
        return ref

    pos_of = {int(e): i for i, e in enumerate(ent_ids)}
    n_e, f_e = check_rows("entity", pick, lambda e: ent_rows_dev[pos_of[int(e)]].cpu().numpy(), ent_ref_capped)

    # -- relation (and auxiliary) rows
    rpos_of = {int(e): i for i, e in enumerate(rel_ids)}
    done_r = []

    def rel_ref(rid, aux):
        mb = r == rid
        if int(mb.sum()) * (1 + (N if neg is not None else 0)) > max_triples or len(done_r) >= 2 * n_rel_rows:
            return None
        fh, fr, ft, fg = explicit_triples(mb, [])
        ref, _, ur = oracle_rows(fh, fr, ft, fg)
        done_r.append(rid)
        rows = ref.aux_rows if aux else ref.rel_rows
        return rows[int(np.searchsorted(ur, rid))]

    rpick = rng.permutation(rel_ids)[: 4 * n_rel_rows]
    n_r = f_r = 0
    if rel_rows_dev is not None:
        n_r, f_r = check_rows("relation", rpick, lambda e: rel_rows_dev[rpos_of[int(e)]].cpu().numpy(),
                              lambda e: rel_ref(e, False))
    n_a = f_a = 0
    if aux_rows_dev is not None:
        done_r.clear()
        n_a, f_a = check_rows("relation (aux table)", rpick[: n_rel_rows],
                              lambda e: aux_row_dev(rpos_of[int(e)]), lambda e: rel_ref(e, True))
    report.update({"entity_rows_checked": len(done), "gradient_elements_checked": int(n_e + n_r + n_a),
                   "l1_sign_flips": int(f_e + f_r + f_a)})
    return report


# ---- CPU baseline ------------------------------------------------------------------------------
def cpu_baseline(w, target_s=4.0):
    """The oracle's loops (the restatement of cuke's generated CPU code) timed on this host over a
    bounded sample of the same workload: whole chunks of the batch (same dim, chunk size, negatives
    and index distributions; entity table cut to 200k rows to bound host memory), forward +
    backward, repeated until about `target_s` seconds of CPU work have been spent on one thread
    (gcc -O3), then the same with OpenMP over the batch on all host cores for about half as long."""
    import oracle
    from cuke_amd import synth
    oracle.build()
    n_ent = min(w.n_ent, 200_000)
    unit = w.chunk if w.chunk else min(w.batch, 1024)
    base, over = (w.name, {}) if w.name in synth.CONFIGS else ("cfg3_transr", dict(dim=w.dim))
    s = synth.make_workload(base, seed=w.seed, n_ent=n_ent, **over)
    if s.model in ("TransR", "RESCAL") and s.dim >= 512:
        unit = 256  # bounds the per-thread d x d gradient accumulators of the OpenMP leg
    a = s.arrays

    def run(b0, b1, fast):
        sl = slice(b0, b1)
        neg = a["neg"][(b0 // s.chunk) * s.n_neg:(b1 // s.chunk) * s.n_neg] if s.chunk else None
        t0 = time.perf_counter()
        pos, negs = oracle.score(s.model, a["E"], a["R"], a["A"], a["h"][sl], a["r"][sl], a["t"][sl], neg,
                                 s.chunk, p=s.norm_p, gamma=s.gamma, fast=fast)
        tf = time.perf_counter() - t0
        tb = 0.0
        if s.backward:
            dneg = np.ones_like(negs) if negs is not None else None
            t0 = time.perf_counter()
            oracle.backward(s.model, a["E"], a["R"], a["A"], a["h"][sl], a["r"][sl], a["t"][sl], neg, s.chunk,
                            np.ones_like(pos), dneg, p=s.norm_p, fast=fast)
            tb = time.perf_counter() - t0
        return tf, tb

    def leg(fast, budget):
        t_fwd = t_bwd = 0.0
        scored = done = 0
        while True:
            b0 = (done * unit) % s.batch
            tf, tb = run(b0, b0 + unit, fast)
            t_fwd, t_bwd, done = t_fwd + tf, t_bwd + tb, done + 1
            scored += unit * (1 + s.n_neg)
            spent = t_fwd + t_bwd
            if spent >= budget or spent + spent / done > 2.5 * budget:
                return scored, t_fwd, t_bwd, done

    scored, t_fwd, t_bwd, done = leg("o3", target_s)
    run(0, unit, "omp")  # first call starts the OpenMP thread pool
    scored_m, tf_m, tb_m, done_m = leg("omp", target_s / 2)
    what = "fwd+bwd" if s.backward else "fwd"
    out = {"value": scored / (t_fwd + t_bwd), "unit": "triples scored/s", "cores": 1, "kind": "port",
           "sample": f"{s.model} dim={s.dim} n_ent={s.n_ent}: {done} x (B={unit}, N={s.n_neg}) = {scored} scores {what}, "
                     f"fwd {t_fwd:.2f}s + bwd {t_bwd:.2f}s, gcc -O3 -march=x86-64-v3, 1 thread",
           "fwd_s": t_fwd, "bwd_s": t_bwd,
           "all_cores": {"value": scored_m / (tf_m + tb_m), "unit": "triples scored/s", "cores": oracle.threads("omp"),
                         "sample": f"{done_m} x (B={unit}, N={s.n_neg}) {what}, OpenMP over the batch, "
                                   f"fwd {tf_m:.2f}s + bwd {tb_m:.2f}s"}}
    if not s.chunk and not s.backward:
        # the flags the reference's own JIT build of its generated C++ gets: no optimisation flag, one thread
        sc0, tf0, tb0, d0 = leg("o0", 1.0)
        out["as_the_reference_builds_it"] = {"value": sc0 / (tf0 + tb0), "unit": "triples scored/s", "cores": 1,
                                             "sample": f"{d0} x B={unit} fwd, gcc -O0, 1 thread"}
    return out


# ---- one workload ------------------------------------------------------------------------------
def make_named_workload(name, seed):
    from cuke_amd import synth
    if name == "ref_transr_8192x512":
        # the TransR shape of the reference's own sweep scripts (apps/kge/scripts/test_fig9c_cuke.sh:
        # batch 8192, dim 512); tables and relation distribution as in the TransR benchmark configuration
        w = synth.make_workload("cfg3_transr", seed=seed, tables=False, dim=512)
        w.name = name
        return w
    return synth.make_workload(name, seed=seed, tables=False)


def same_bits(torch, step, ref):
    """The outputs of the step enqueued last against clones taken from another issue of the same batch."""
    g = step.sparse_grads()
    cur = [step.pos, step.neg, g.ent_ids, g.ent_rows, g.rel_ids, g.rel_rows]
    if g.factor_max:
        seg = g.rel_seg_offsets
        dense = (seg[1:] - seg[:-1]) > g.factor_max
        rows = torch.repeat_interleave(~dense, (seg[1:] - seg[:-1]).long())
        cur += [g.aux_rows[dense], g.aux_x[: rows.numel()][rows], g.aux_q[: rows.numel()][rows]]
    else:
        cur.append(g.aux_rows)
    if ref is None:
        return [x.clone() if x is not None else None for x in cur]
    return all((a is None and b is None) or torch.equal(a, b) for a, b in zip(cur, ref))


def run_workload(name, args, torch, factor_max=0):
    from cuke_amd.kge import KGEModel, TrainStep
    dev = torch.device("cuda:0")
    w = make_named_workload(name, args.seed)
    from cuke_amd import synth
    E, R, A = synth.device_tables(w, dev)
    model = KGEModel(w.model, E, R, A, norm_p=w.norm_p, gamma=w.gamma)
    nb = max(1, args.batches)
    sets = [w] + [make_named_workload(name, args.seed + 1 + i) for i in range(nb - 1)]
    ixs = [{k: torch.from_numpy(v).to(dev) for k, v in s.arrays.items() if v is not None} for s in sets]
    sign = 1.0 if w.model in ("DistMult", "ComplEx", "RotatE", "TransF", "RESCAL") else -1.0
    ix = ixs[0]
    step = TrainStep(model, ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, loss=w.loss,
                     margin=w.margin, sign=sign, factor_max=factor_max, back_rows=not args.no_back_rows)
    if w.model in ("TransR", "RESCAL"):  # what the projection gradients of batch 0 cost to write (algorithmic bytes)
        cnt = np.unique(w.arrays["r"], return_counts=True)[1]
        w.dense_rel, w.factored_rows = int((cnt > factor_max).sum()), int(cnt[cnt <= factor_max].sum())
    for o in ixs[1:]:
        step.add_batch(o["h"], o["r"], o["t"], o.get("neg"))
    do_bwd = w.backward

    check = {"parity_spot_check": "skipped (--no-check)"}
    if not args.no_check:
        t0 = time.perf_counter()
        check = {"parity_spot_check": "ok", **spot_check(w, model, step, ix), "seconds": None}
        check["seconds"] = round(time.perf_counter() - t0, 2)

    def timed(one):
        # untimed warm-up: the W steps asked for, and at least WARMUP_MIN_S of device work (a timed region
        # of 20 steps of 60 us is over before the clocks have settled otherwise)
        t0, n = time.perf_counter(), 0
        while n < args.warmup or time.perf_counter() - t0 < WARMUP_MIN_S:
            one()
            n += 1
            if n % 16 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        return time_events(one, args.steps, torch)

    counter = [0]

    def rotating(run_one):
        def f():
            i = counter[0] % nb
            counter[0] += 1
            run_one(i)
        return f

    def direct(i):
        step.select(i)
        step.run(do_bwd)

    step.select(0)
    ms_same = timed(lambda: step.run(do_bwd))
    ms_rot = timed(rotating(direct))
    ms_graph = None
    issue, ms = "direct", ms_rot
    if not args.no_graph:
        graphs = []
        for i in range(nb):
            step.select(i)
            graphs.append(step.capture(do_bwd))
        ms_graph = timed(rotating(lambda i: graphs[i].replay()))
        if ms_graph < ms:
            issue, ms = "graph", ms_graph
        del graphs
        step.graph = None

    # Staged issue: batch i + 1 is inspected on a side stream (TransR: its relation groups planned too)
    # while batch i's step runs; every timed step still inspects one batch and runs one forward / loss /
    # backward.  The riding (fused) inspection of `direct` is not used in this form.
    ms_staged = None
    ref_bits0 = None
    if do_bwd and not args.no_staged:
        state = {"next": 0}

        def staged_step():
            nxt = state["next"]
            state["next"] = (nxt + 1) % nb
            step.stage(batch=nxt)
            step.run(pipeline=True)

        # the staged issue takes other launch forms than the direct one (no riding inspection, merged
        # launches): before it is timed, its outputs for batch 0 must be the direct issue's, bit for bit
        step.select(0)
        step.run(do_bwd)
        torch.cuda.synchronize()
        ref_bits = same_bits(torch, step, None)
        step.stage(batch=0)
        step.run(pipeline=True)
        torch.cuda.synchronize()
        if not same_bits(torch, step, ref_bits):
            raise SpotCheckError(f"{w.name}: the staged issue's outputs differ from the direct issue's for batch 0")
        check["staged_equals_direct_bits"] = True
        ref_bits0 = ref_bits
        step.stage(batch=state["next"])          # one batch ahead from here on
        state["next"] = (state["next"] + 1) % nb
        if nb >= 3:
            ms_staged = timed(staged_step)
            step.run(pipeline=True)              # drain the batch still staged
            torch.cuda.synchronize()
            if ms_staged < ms:
                issue, ms = "staged", ms_staged
        else:
            step.run(pipeline=True)
            torch.cuda.synchronize()

    # The staged issue from native code: the same launches, one library call per step (kge_train_step_staged).
    ms_native = None
    if do_bwd and not args.no_staged and nb >= 3:
        step.run_native(None, 0)
        step.run_native(0, 1)
        torch.cuda.synchronize()
        if ref_bits0 is not None and not same_bits(torch, step, ref_bits0):
            raise SpotCheckError(f"{w.name}: the native staged issue differs from the direct issue for batch 0")
        check["native_equals_direct_bits"] = True
        state = {"cur": 1}

        def native_step():
            cur = state["cur"]
            state["cur"] = (cur + 1) % nb
            step.run_native(cur, (cur + 1) % nb)

        ms_native = timed(native_step)
        torch.cuda.synchronize()
        if ms_native < ms:
            issue, ms = "staged_native", ms_native

    # DistMult / ComplEx: the same rotating loop with the pair sums of the tile kernels on the vector ALUs
    ms_forms = None
    if w.model in ("DistMult", "ComplEx") and w.chunk and do_bwd:
        model.pair_sums = "vector_alus"
        ms_valu = timed(rotating(direct))
        model.pair_sums = "matrix_cores"
        ms_forms = {"matrix_cores": ms_rot, "vector_alus": ms_valu}

    step.select(0)
    u_ent, u_rel = step.ent_insp.num_unique, step.rel_insp.num_unique
    if not do_bwd:
        occ = torch.cat([ix["h"], ix["t"]] + ([ix["neg"]] if "neg" in ix else []))
        u_ent, u_rel = int(torch.unique(occ).numel()), int(torch.unique(ix["r"]).numel())
    fwd_b, bwd_b = algorithmic_bytes(w, u_ent, u_rel)
    fwd_f, bwd_f = algorithmic_flops(w)
    total_b = fwd_b + (bwd_b if do_bwd else 0)
    total_f = fwd_f + (bwd_f if do_bwd else 0)
    scores = w.scores_per_step

    # per-kernel durations, live: an event behind every kernel, rotating batches; a spin kernel of
    # about 0.2 ms in front of each step lets the host enqueue the whole step before the device starts
    # it (no memory traffic: the caches hold what the timed loop's previous step left, as there)
    # The timeline follows the issue that is reported: the staged issue launches other kernel forms than the
    # direct one (no inspection riding along); its inspection runs on the side stream a batch
    # ahead, so those entries (taken here in front of the step on one stream) are not part of the step.
    kt_fused = False if issue.startswith("staged") else None
    if hasattr(torch.cuda, "_sleep"):
        kt = step.kernel_times(steps=max(8, min(32, args.steps)), backward=do_bwd, batches=list(range(nb)),
                               lead=lambda: torch.cuda._sleep(400_000), fused=kt_fused)
    else:
        lead = torch.empty(1024 * 1024, dtype=torch.float32, device=dev)
        kt = step.kernel_times(steps=max(8, min(32, args.steps)), backward=do_bwd, batches=list(range(nb)), lead=lead,
                               fused=kt_fused)
        del lead
    on_step = [(n_, m_) for n_, m_ in kt if not (issue.startswith("staged") and n_.startswith("inspect"))]
    kt_sum = sum(ms_k for _, ms_k in on_step)
    kname, k_ms = max(on_step, key=lambda x: x[1])
    k_bytes, k_flops, k_unit = kernel_model(w, kname, u_ent, u_rel)
    bound = BOUND.get(name, "hbm")
    gbs = k_bytes / (k_ms * 1e-3) / 1e9
    tfs = k_flops / (k_ms * 1e-3) / 1e12
    hbm_roof = {"achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}
    fp32_roof = {"achieved": tfs, "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tfs / FP32_PEAK_TFLOPS,
                 "arithmetic_unit": "fp32 MFMA" if k_unit == "mfma" else "fp32 vector ALUs"}
    main_roof, other = (hbm_roof, fp32_roof) if bound == "hbm" else (fp32_roof, hbm_roof)
    step_gbs = total_b / (ms * 1e-3) / 1e9
    step_tfs = total_f / (ms * 1e-3) / 1e12
    traffic, profile_kernels = measured_traffic(name, kname, w.model in ("DistMult", "ComplEx") and bool(w.chunk),
                                                dense=w.model in ("TransR", "RESCAL") and factor_max == 0)
    roofline = {"kernel": kname, "bound": "hbm" if bound == "hbm" else "mfma" if k_unit == "mfma" else "fp32_valu",
                "achieved": main_roof["achieved"], "peak": main_roof["peak"], "unit": main_roof["unit"],
                "frac": main_roof["frac"], "traffic": traffic, "traffic_profile_kernels": profile_kernels,
                "kernel_ms": k_ms, "kernel_share_of_step": k_ms / kt_sum if kt_sum else None,
                "algorithmic_bytes_per_launch": k_bytes, "algorithmic_flops_per_launch": k_flops,
                "other_roof": {"bound": "fp32" if bound == "hbm" else "hbm", **other},
                "step": {"bound": bound, "frac": (step_gbs / HBM_PEAK_GBS) if bound == "hbm" else (step_tfs / FP32_PEAK_TFLOPS),
                         "hbm_gbs": step_gbs, "hbm_frac": step_gbs / HBM_PEAK_GBS, "fp32_tflops": step_tfs,
                         "fp32_frac": step_tfs / FP32_PEAK_TFLOPS, "algorithmic_bytes": total_b,
                         "algorithmic_flops": total_f}}

    out = {
        "metric": "triples scored/sec fwd+bwd per KGE model; % of HBM (or MFMA) roofline",
        "value": scores / (ms * 1e-3),
        "unit": "triples scored/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded N(0,sigma) tables, Zipf/uniform indices, shared negatives per chunk)",
        "config": {"workload": w.name, "score_function": w.model, "n_ent": w.n_ent, "n_rel": w.n_rel, "dim": w.dim,
                   "batch": w.batch, "chunk": w.chunk, "n_neg": w.n_neg, "norm_p": w.norm_p,
                   "backward": do_bwd, "loss": w.loss, "issue": issue, "rotating_batches": nb, "warmup_min_ms": WARMUP_MIN_S * 1e3,
                   "pair_sums": "matrix cores, fp32" if w.model in ("DistMult", "ComplEx") and w.chunk else "vector ALUs",
                   "ms_per_step_rotating_direct": ms_rot, "ms_per_step_rotating_graph": ms_graph,
                   "ms_per_step_rotating_staged": ms_staged, "ms_per_step_rotating_staged_native": ms_native,
                   "ms_per_step_same_batch": ms_same, "ms_per_step_by_pair_sum_unit": ms_forms,
                   "scores_per_step": scores, "positives_per_s": w.batch / (ms * 1e-3),
                   "unique_entity_rows": u_ent, "unique_relation_rows": u_rel,
                   "projection_gradients": (None if w.model not in ("TransR", "RESCAL") else
                                            {"factor_max": factor_max, "dense_groups": w.dense_rel,
                                             "factored_rows": w.factored_rows,
                                             "back_rows_from_forward": step.back_rows is not None})},
        "kernels_ms": [[n_ + (" (side stream, a batch ahead)" if (n_, m_) not in on_step else ""), round(m_, 6)]
                       for n_, m_ in kt],
        "roofline": roofline,
        **check,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(w, args.cpu_seconds)
    del step, model, E, R, A, ixs
    torch.cuda.empty_cache()
    return out


def run_neg_transr(args, torch, model_name="TransR"):
    """TransR (or RESCAL) with shared negatives at B=4096, N=64, dim=200 (relations Zipf 1.2 over 1345, as the
    TransR benchmark configuration), forward + backward, beside the flattened B * (1 + N) explicit triples (the
    reference's neg_transR, apps/examples/examples.py:1447-1480).  TransR: every negative projected once per
    (relation, chunk) group; rows through the grouped matrix-core kernels are counted on the host from the
    index arrays, 2 B + G N against B (1 + N), G = distinct (relation, chunk) pairs.  RESCAL: the pair score
    (E[h] Proj[r]) . E[t'] needs the B projected rows only (a dot-product tile over them)."""
    from cuke_amd import synth
    from cuke_amd.kge import KGEModel, inspect
    dev = torch.device("cuda:0")
    out = {"workload": f"neg_{model_name.lower()}_4096x64x200", "batch": 4096, "n_neg": 64, "dim": 200, "by_chunk": []}
    for chunk in (64, 512, 4096):
        w = synth.custom_workload(model_name, seed=args.seed, n_ent=40000, n_rel=1345, dim=200, batch=4096, chunk=chunk,
                                  n_neg=64, norm_p=2, sigma=0.05, rel_zipf=1.2)
        a = w.arrays
        m = KGEModel(model_name, torch.from_numpy(a["E"]).to(dev), torch.from_numpy(a["R"]).to(dev) if model_name == "TransR" else None,
                     torch.from_numpy(a["A"]).to(dev), norm_p=2)
        ix = {k: torch.from_numpy(a[k]).to(dev) for k in ("h", "r", "t", "neg")}
        g_pairs = len(np.unique(a["r"] * w.n_chunks + np.arange(w.batch) // chunk))
        rows_grouped = 2 * w.batch + g_pairs * w.n_neg if model_name == "TransR" else w.batch
        rows_flat = w.batch * (1 + w.n_neg)
        dpos = torch.ones(w.batch, device=dev)
        dneg = torch.ones((w.batch, w.n_neg), device=dev)
        ent_insp, rel_insp = m.inspect_batch(ix["h"], ix["r"], ix["t"], ix["neg"])

        def grouped():
            fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], chunk, ent_insp=ent_insp, rel_insp=rel_insp)
            return fw, m.backward(fw, dpos, dneg)

        def flattened():
            fw = m._score_projected_negatives(ix["h"], ix["r"], ix["t"], ix["neg"], chunk)
            return fw, m.backward(fw, dpos, dneg)

        fg, gg = grouped()
        ff, gf = flattened()
        torch.cuda.synchronize()
        err = float((fg.neg - ff.neg).abs().max() / ff.neg.abs().max())
        gerr = float((gg.aux_rows - gf.aux_rows).abs().max() / gf.aux_rows.abs().max())
        if not (err < 1e-5 and gerr < 1e-4):
            raise SpotCheckError(f"neg_transr chunk {chunk}: grouped and flattened paths differ ({err:.2e}, {gerr:.2e})")
        del fg, gg, ff, gf
        res = {}
        for label, fn in (("grouped", grouped), ("flattened", flattened)):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            res[label] = time_events(fn, max(5, min(20, args.steps)), torch)
        out["by_chunk"].append({"chunk": chunk, "groups": g_pairs, "rows_projected_grouped": rows_grouped,
                                "rows_projected_flattened": rows_flat, "row_ratio": rows_flat / rows_grouped,
                                "ms_grouped": res["grouped"], "ms_flattened": res["flattened"],
                                "max_rel_diff_scores": err, "max_rel_diff_projection_gradients": gerr})
        del m
        torch.cuda.empty_cache()
    return out


def stream_calibration(torch, dev):
    """What a plain streaming kernel reaches on this GPU: read + written bytes over time of torch's
    256 MiB elementwise copy kernel, sources rotating over 1 GiB so that no cache holds a pass."""
    n = 64 * 1024 * 1024
    srcs = [torch.empty(n, dtype=torch.float32, device=dev).normal_() for _ in range(4)]
    dst = torch.empty_like(srcs[0])
    it = [0]

    def copy():
        dst.copy_(srcs[it[0] % 4])
        it[0] += 1

    for _ in range(4):
        copy()
    ms = time_events(copy, 12, torch)
    del srcs, dst
    torch.cuda.empty_cache()
    return {"stream_copy_gbs": 2 * 4 * n / (ms * 1e-3) / 1e9, "peak_gbs": HBM_PEAK_GBS,
            "sample": "256 MiB device-to-device copy kernel, (bytes read + bytes written) / time, 4 rotating sources"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    help="all (default), one of " + ", ".join(ALL_WORKLOADS) + ", ref_transr_8192x512, or neg_transr / "
                         "neg_rescal (shared negatives of the projection models: grouped form against flattened triples)")
    ap.add_argument("--batches", type=int, default=8, help="distinct seeded batches the timed loop rotates over")
    ap.add_argument("--no-graph", action="store_true", help="do not also time HIP-graph replays of the step")
    ap.add_argument("--no-staged", action="store_true",
                    help="do not also time the staged issue (next batch inspected on a side stream)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-check", action="store_true", help="skip the parity spot check (profiling runs)")
    ap.add_argument("--dense-only", action="store_true",
                    help="TransR: time only the step that writes every projection gradient dense (profiling runs)")
    ap.add_argument("--no-back-rows", action="store_true",
                    help="TransR: the forward pass does not also form phi(residual) Proj^T; the backward pass reads the "
                         "projections a second time in a dX kernel of its own (the form before back rows)")
    ap.add_argument("--factored-only", action="store_true",
                    help="TransR: time only the headline step (small groups' projection gradients factored), not "
                         "the dense one beside it (profiling runs)")
    ap.add_argument("--cpu-seconds", type=float, default=4.0, help="one-thread CPU work per workload")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy kernel (a known-traffic reference "
                         "for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (nothing here shards across GPUs)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    if args.workload in ("neg_transr", "neg_rescal"):
        try:
            print(json.dumps(run_neg_transr(args, torch, "TransR" if args.workload == "neg_transr" else "RESCAL")))
        except SpotCheckError as e:
            print(f"bench.py: {e}", file=sys.stderr)
            sys.exit(1)
        return
    names = ALL_WORKLOADS if args.workload == "all" else [args.workload]
    machine = stream_calibration(torch, dev)
    results = []
    for n in names:
        t0 = time.perf_counter()
        try:
            if n in ("cfg3_transr", "ref_transr_8192x512") and not args.dense_only:
                # The projection gradients of relation groups of at most four triples (most relations of a
                # long-tailed batch) are left factored, the form the optimizer entry points consume; the same
                # step with every gradient written dense is timed in the same run and reported beside it.
                res = run_workload(n, args, torch, factor_max=4)
                if not args.factored_only:
                    saved_no_cpu, args.no_cpu = args.no_cpu, True
                    dense = run_workload(n, args, torch, factor_max=0)
                    args.no_cpu = saved_no_cpu
                    res["config"]["dense_projection_gradients"] = {
                        k: dense[k] for k in ("ms_per_step", "value", "kernels_ms", "roofline")}
                    res["config"]["dense_projection_gradients"]["issue"] = dense["config"]["issue"]
            else:
                res = run_workload(n, args, torch)
        except SpotCheckError as e:
            print(f"bench.py: parity spot check failed, nothing is reported: {e}", file=sys.stderr)
            sys.exit(1)
        res["bench_seconds"] = round(time.perf_counter() - t0, 1)
        results.append(res)
        dn = res["config"].get("dense_projection_gradients")
        print(f"[bench] {n}: {res['ms_per_step']:.4f} ms/step, {res['value']:.3e} scores/s, dominant "
              f"{res['roofline']['kernel']} {res['roofline']['frac']:.3f} of {res['roofline']['bound']}, step "
              f"{res['roofline']['step']['frac']:.3f} of {res['roofline']['step']['bound']}"
              + (f"; every projection gradient dense: {dn['ms_per_step']:.4f} ms/step, step "
                 f"{dn['roofline']['step']['frac']:.3f}" if dn else ""),
              file=sys.stderr, flush=True)
    out = results[0]
    out["machine"] = machine
    if len(results) > 1:
        out["per_workload"] = results[1:]
    # one compact row per workload inside `roofline` (the full records are in per_workload)
    table = []
    for r in results:
        rf, cb = r["roofline"], r.get("cpu_baseline") or {}
        row = {"workload": r["config"]["workload"], "ms_per_step": round(r["ms_per_step"], 5), "issue": r["config"]["issue"],
               "scores_per_s": float(f"{r['value']:.4g}"), "kernel": rf["kernel"], "kernel_ms": round(rf["kernel_ms"], 5),
               "bound": rf["bound"], "frac": round(rf["frac"], 4), "step_bound": rf["step"]["bound"],
               "step_frac": round(rf["step"]["frac"], 4), "traffic": rf["traffic"],
               "cpu_1_thread": float(f"{cb['value']:.4g}") if cb else None,
               "cpu_all_cores": float(f"{cb['all_cores']['value']:.4g}") if cb else None,
               "cpu_cores": cb["all_cores"]["cores"] if cb else None}
        dn = r["config"].get("dense_projection_gradients")
        if dn:
            row["dense_ms_per_step"] = round(dn["ms_per_step"], 5)
            row["dense_step_frac"] = round(dn["roofline"]["step"]["frac"], 4)
        table.append(row)
    out["roofline"]["per_workload"] = table
    print(json.dumps(out))


if __name__ == "__main__":
    main()
