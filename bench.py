#!/usr/bin/env python3
"""Benchmark of the KGE score path on one MI355X.

A step is one pass over one batch of synthetic input with every table and index
array already resident in HBM: index inspection (radix sort + dedup of the entity
and relation ids) -> scores of the positives and of the shared negatives ->
(margin loss) -> sparse row gradients.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2_distmult]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3    # MI355X fp32 vector / fp32 MFMA, published

# HBM bytes per launch of each workload's roofline kernel, from rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE runs of this script (KiB per dispatch), each scaled by what the same counter
# reads for the 256 MiB copy kernel of --calibrate-copy (fetch x2.000, write x1.000).  The
# summaries the numbers come from are profiles/score_path_kernels_<workload>.txt.
MEASURED_TRAFFIC_BYTES = {
    "cfg1_transe": 1_687_370,      # score_pos_kernel
    "cfg2_distmult": 13_060_992,   # score_neg_mfma_kernel
    "cfg2_complex": 13_093_719,    # score_neg_mfma_kernel
    "cfg3_transr": 164_398_014,    # transr_plan_kernel + transr_gemm_kernel<0>
    "cfg4_rotate": 12_060_695,     # score_neg_kernel
    "cfg5_transh": 531_454_520,    # score_neg_kernel
}


def device_tables(w, dev):
    """Tables drawn on the GPU (seeded); benchmark-size tables are too large to push through numpy."""
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(1000 + w.seed)
    E = torch.randn((w.n_ent, w.dim), generator=g, device=dev, dtype=torch.float32) * w.sigma
    if w.model == "RotatE":
        R = (torch.rand((w.n_rel, w.rel_dim), generator=g, device=dev, dtype=torch.float32) * 2 - 1) * np.pi
    else:
        R = torch.randn((w.n_rel, w.rel_dim), generator=g, device=dev, dtype=torch.float32) * w.sigma
    A = None
    if w.model == "TransH":
        A = torch.randn((w.n_rel, w.dim), generator=g, device=dev, dtype=torch.float32)
        A = A / A.norm(dim=1, keepdim=True)
    elif w.model in ("TransR", "RESCAL"):
        A = torch.randn((w.n_rel, w.dim, w.dim), generator=g, device=dev, dtype=torch.float32) * w.sigma
    return E, R, A


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
        bwd += 4 * u_rel * d * d
    return fwd, bwd


def neg_kernel_bytes(w):
    """Algorithmic bytes of ONE launch of the shared-negative forward kernel: the h and r (and w)
    rows of every positive (RotatE: its one rotated-head row), every negative row once per chunk,
    the indices, the scores out."""
    B, d, rd, N = w.batch, w.dim, w.rel_dim, w.n_neg
    nn = w.n_chunks * N
    if w.model == "RotatE":
        # one rotated-head row per positive (written by the positive kernel of the same call), no h / r gathers
        return 4 * (B * d + nn * d) + 8 * nn + 4 * B * N
    aux_row = d if w.model == "TransH" else 0
    out_planes = 3 if w.model == "TransH" else 1
    return 4 * (B * (d + rd + aux_row) + nn * d) + 8 * (2 * B + nn) + 4 * out_planes * B * N


def neg_kernel_flops(w):
    per_elem = {"DistMult": 2, "ComplEx": 2, "TransE": 2, "TransH": 9, "RotatE": 8}[w.model]
    klen = w.dim // 2 if w.model == "RotatE" else w.dim
    return per_elem * w.batch * w.n_neg * klen


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


def cpu_baseline(w, target_s=12.0, cap_s=40.0):
    """The oracle's loops (the restatement of cuke's generated CPU code; gcc -O3, ONE thread)
    timed on this host over a bounded sample of the same workload: whole chunks of the batch
    (same dim, chunk size, negatives and index distributions; entity table cut to 200k rows to
    bound host memory), forward + backward, repeated until about `target_s` seconds of CPU
    work have been spent.  Beside it: the forward pass alone with OpenMP over all host cores."""
    import oracle
    from cuke_amd import synth
    oracle.build()
    n_ent = min(w.n_ent, 200_000)
    unit = w.chunk if w.chunk else min(w.batch, 1024)
    s = synth.make_workload(w.name, seed=w.seed, n_ent=n_ent)
    a = s.arrays

    def run(b0, b1, fast):
        sl = slice(b0, b1)
        neg = a["neg"][(b0 // s.chunk) * s.n_neg:(b1 // s.chunk) * s.n_neg] if s.chunk else None
        t0 = time.perf_counter()
        pos, negs = oracle.score(s.model, a["E"], a["R"], a["A"], a["h"][sl], a["r"][sl], a["t"][sl], neg,
                                 s.chunk, p=s.norm_p, gamma=s.gamma, fast=fast)
        tf = time.perf_counter() - t0
        tb = 0.0
        if s.backward and fast == "o3":
            dneg = np.ones_like(negs) if negs is not None else None
            t0 = time.perf_counter()
            oracle.backward(s.model, a["E"], a["R"], a["A"], a["h"][sl], a["r"][sl], a["t"][sl], neg, s.chunk,
                            np.ones_like(pos), dneg, p=s.norm_p, fast="o3")
            tb = time.perf_counter() - t0
        return tf, tb

    t_fwd = t_bwd = 0.0
    scored = 0
    done = 0
    while True:
        b0 = (done * unit) % s.batch
        tf, tb = run(b0, b0 + unit, "o3")
        t_fwd, t_bwd, done = t_fwd + tf, t_bwd + tb, done + 1
        scored += unit * (1 + s.n_neg)
        spent = t_fwd + t_bwd
        if spent >= target_s or spent + spent / done > cap_s:
            break
    run(0, unit, "omp")  # first call starts the OpenMP thread pool
    tf_omp, _ = run(0, unit, "omp")
    return {"value": scored / (t_fwd + t_bwd), "unit": "triples scored/s", "cores": 1, "kind": "port",
            "sample": f"{s.model} dim={s.dim} n_ent={s.n_ent}: {done} x (B={unit}, N={s.n_neg}) = {scored} scores, "
                      f"fwd {t_fwd:.2f}s + bwd {t_bwd:.2f}s, gcc -O3 -march=x86-64-v3, 1 thread",
            "fwd_s": t_fwd, "bwd_s": t_bwd,
            "forward_only_openmp": {"value": unit * (1 + s.n_neg) / tf_omp, "unit": "triples scored/s",
                                    "cores": oracle.threads("omp")}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2_distmult")
    ap.add_argument("--no-graph", action="store_true", help="launch kernels one by one instead of a HIP graph")
    ap.add_argument("--no-pipeline", action="store_true", help="do not try the double-buffered inspector")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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
    from cuke_amd import synth
    from cuke_amd.kge import KGEModel, TrainStep

    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    w = synth.make_workload(args.workload, seed=args.seed, tables=False)
    E, R, A = device_tables(w, dev)
    model = KGEModel(w.model, E, R, A, norm_p=w.norm_p, gamma=w.gamma)
    ix = {k: torch.from_numpy(v).to(dev) for k, v in w.arrays.items() if v is not None}
    sign = 1.0 if w.model in ("DistMult", "ComplEx", "RotatE", "TransF", "RESCAL") else -1.0
    step = TrainStep(model, ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, loss=w.loss,
                     margin=w.margin, sign=sign)
    do_bwd = w.backward

    # Three ways to issue the same step: kernel by kernel from the host; kernel by kernel with the
    # index tensors and inspections in a ring of sets, so the inspector of batch i+1 (side stream)
    # is enqueued before step i and neither stream waits for the other on the critical path (every
    # timed step still enqueues exactly one inspection and one forward / loss / backward); or as
    # one HIP graph replay.  All are warmed up and timed
    # over exactly --steps steps, every step doing its own inspection, forward, loss and backward;
    # the fastest is the reported configuration (a graph replay has a fixed host cost that only
    # pays off when the step has many kernels).
    def timed(one):
        for _ in range(args.warmup):
            one()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ms_ = time_events(one, args.steps, torch)
        return ms_, time.perf_counter() - t0

    ms_direct, wall = timed(lambda: step.run(do_bwd))
    ms_graph = ms_pipe = None
    issue = "direct"
    ms = ms_direct
    if do_bwd and not args.no_pipeline:
        def one_pipelined():
            step.stage()  # inspector of the batch after the one that runs now (side stream)
            step.run(do_bwd, pipeline=True)
        step.stage()  # primes the ring: from here on one batch is always inspected ahead
        ms_pipe, wall_p = timed(one_pipelined)
        step.run(do_bwd, pipeline=True)  # drains the batch staged last
        if ms_pipe < ms:
            ms, wall, issue = ms_pipe, wall_p, "pipelined"
    if not args.no_graph:
        step.capture(do_bwd)
        ms_graph, wall_g = timed(step.replay)
        if ms_graph < ms:
            ms, wall, issue = ms_graph, wall_g, "graph"
    use_graph = issue == "graph"

    # DistMult / ComplEx: the same step with the pair sums of the tile kernels on the other unit
    # (matrix cores <-> vector ALUs), direct launches, for comparison; the setting is restored
    ms_forms = None
    if w.model in ("DistMult", "ComplEx") and w.chunk and do_bwd:
        from cuke_amd import _lib as _l
        was = _l.lib().kge_set_pair_sum_unit(0)
        _l.lib().kge_set_pair_sum_unit(1 - was)
        ms_other, _ = timed(lambda: step.run(do_bwd))
        _l.lib().kge_set_pair_sum_unit(was)
        ms_forms = {"matrix_cores": ms_other if was else ms_direct, "vector_alus": ms_direct if was else ms_other}

    u_ent, u_rel = step.ent_insp.num_unique, step.rel_insp.num_unique
    fwd_b, bwd_b = algorithmic_bytes(w, u_ent, u_rel)
    total_b = fwd_b + (bwd_b if do_bwd else 0)
    scores = w.scores_per_step

    # per-stage times, un-graphed, each stage launched back to back
    st = torch.cuda.current_stream().cuda_stream
    import ctypes
    stc = ctypes.c_void_p(st)
    stages = {"inspect_ms": time_events(lambda: step.inspect(stc), 50, torch),
              "forward_ms": time_events(lambda: step.forward(stc), 50, torch)}
    if do_bwd:
        stages["loss_ms"] = time_events(lambda: step.loss_grad(stc), 50, torch)
        stages["backward_ms"] = time_events(lambda: step.backward(stc), 50, torch)

    # dominant kernel in isolation: the shared-negative forward tile kernel (or, for
    # positive-only workloads, the per-triple kernel), K launches between two events
    from cuke_amd import _lib
    L = _lib.lib()
    if w.chunk:
        P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
        kname = "score_neg_mfma_kernel" if w.model in ("DistMult", "ComplEx") else "score_neg_kernel"
        if w.model in ("TransH", "RotatE"):
            # the tile kernel reads what the positive kernel of the same call leaves behind (w.h, the
            # rotated heads): time the forward call and the positive kernel alone, report the
            # difference
            t_pair = time_events(lambda: step.forward(stc), 100, torch)
            t_pos = time_events(lambda: L.kge_score_fwd(ctypes.byref(model._tab), ctypes.byref(step.bat), P(step.pos),
                                                        None, P(step.side_pos), None, P(step.residual), None, 0, stc),
                                100, torch)
            k_ms = t_pair - t_pos
        else:
            k_ms = time_events(lambda: L.kge_score_fwd(ctypes.byref(model._tab), ctypes.byref(step.bat), None,
                                                       P(step.neg), None, None, None, None, 0, stc), 100, torch)
        k_bytes, k_flops = neg_kernel_bytes(w), neg_kernel_flops(w)
        # the two memory-bound pieces of a shared-negative step, on their own: the per-positive
        # gather kernel and the inspection of concat(h, t, neg) and r
        if w.model not in ("TransH", "RotatE"):
            t_pos = time_events(lambda: L.kge_score_fwd(ctypes.byref(model._tab), ctypes.byref(step.bat), P(step.pos),
                                                        None, P(step.side_pos), None, P(step.residual), None, 0, stc),
                                100, torch)
        aux_row = w.dim if w.model == "TransH" else 0
        pos_bytes = 4 * w.batch * (2 * w.dim + w.rel_dim + aux_row) + 8 * 3 * w.batch + 4 * w.batch \
            + (4 * w.batch * w.dim if w.model == "RotatE" else 0) + (4 * w.batch if w.model == "TransH" else 0)
        n_ids = step.n_occ + w.batch
        insp_bytes = n_ids * (8 + 3 * 4) + (u_ent + u_rel) * (8 + 4)  # ids in; perm, inverse, segment per id; unique ids, offsets
        extra = {"positive_gather": {"kernel": "score_pos_kernel", "ms": t_pos, "algorithmic_bytes": pos_bytes,
                                     "gbs": pos_bytes / (t_pos * 1e-3) / 1e9,
                                     "hbm_frac": pos_bytes / (t_pos * 1e-3) / 1e9 / HBM_PEAK_GBS},
                 "inspection": {"ids": n_ids, "ms": stages["inspect_ms"], "algorithmic_bytes": insp_bytes,
                                "ids_per_s": n_ids / (stages["inspect_ms"] * 1e-3),
                                "note": "stand-alone inspector launches; in the timed step its workgroups ride with the "
                                        "score kernels where the batch qualifies"}}
    else:
        # positive-only workloads: the forward call is one kernel (TransR: the tile-plan kernel,
        # a few microseconds, plus the grouped MFMA kernel)
        kname = "score_pos_kernel" if w.model != "TransR" else "transr_plan_kernel + transr_gemm_kernel<0>"
        k_ms = time_events(lambda: step.forward(stc), 100, torch)
        k_bytes = fwd_b
        k_flops = 2 * w.batch * w.dim * w.dim if w.model == "TransR" else 3 * w.batch * w.dim
        extra = {}
    achieved = k_bytes / (k_ms * 1e-3) / 1e9

    out = {
        "metric": "triples scored/sec fwd+bwd per KGE model; % of HBM (or MFMA) roofline",
        "value": scores / (ms * 1e-3),
        "unit": "triples scored/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded N(0,sigma) tables, Zipf/uniform indices, shared negatives per chunk)",
        "config": {"workload": w.name, "score_function": w.model, "n_ent": w.n_ent, "n_rel": w.n_rel, "dim": w.dim,
                   "batch": w.batch, "chunk": w.chunk, "n_neg": w.n_neg, "norm_p": w.norm_p,
                   "backward": do_bwd, "loss": w.loss, "hip_graph": use_graph, "issue": issue,
                   "pair_sums": ("vector ALUs (KGE_DOT_VALU=1)" if os.environ.get("KGE_DOT_VALU", "0") not in ("", "0")
                                 else "matrix cores, fp32 (default)") if w.model in ("DistMult", "ComplEx") and w.chunk
                   else "vector ALUs",
                   "ms_per_step_direct": ms_direct, "ms_per_step_pipelined": ms_pipe,
                   "ms_per_step_graph": ms_graph, "ms_per_step_direct_by_pair_sum_unit": ms_forms,
                   "scores_per_step": scores, "positives_per_s": w.batch / (ms * 1e-3),
                   "unique_entity_rows": u_ent, "unique_relation_rows": u_rel},
        "step": {"algorithmic_bytes": total_b, "hbm_gbs": total_b / (ms * 1e-3) / 1e9,
                 "hbm_frac": total_b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "wall_s": wall, **stages, **extra},
        "roofline": {"kernel": kname, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES.get(w.name),
                     "kernel_ms": k_ms,
                     "algorithmic_bytes_per_launch": k_bytes,
                     ("fp32_mfma" if w.model in ("TransR", "DistMult", "ComplEx") else "fp32_valu"): {"flops_per_launch": k_flops,
                                   "achieved_tflops": k_flops / (k_ms * 1e-3) / 1e12,
                                   "frac_of_157.3": k_flops / (k_ms * 1e-3) / 1e12 / FP32_PEAK_TFLOPS}},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
