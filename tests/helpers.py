"""Shared helpers for the parity tests."""
import numpy as np
import torch

# fp32 parity bar: |got - ref| <= RTOL * |ref| + RTOL * rms(ref).  The second term is the
# absolute floor for entries that cancel to (nearly) zero: the oracle sums serially with
# separate multiply and add, the GPU sums as a tree with fused multiply-add, and both are
# fp32, so entries much smaller than the array's scale cannot agree to a pure relative bound.
# For gradient rows (rows=True) the floor is taken per row: each row is its own sum over the
# row's occurrences, and a hot row's scale is orders of magnitude above a cold row's.
RTOL = 1e-5


# RotatE gradients contain unit vectors u/|u| of complex differences u = h e^{i theta} - t.
# Where |u| is ~10^-3 of the operands, the fp32 rounding of the rotated head (the oracle's
# libm sin/cos and the GPU's differ in the last bit) is magnified by 1/|u| in BOTH
# implementations, so a few elements per million legitimately differ by more than the bar.
# `outliers=(fraction, factor)` admits at most that fraction of elements, each within
# factor x the bound; it is only used by the RotatE gradient tests.
#
# `global_floor=f` adds f x rtol x rms(whole array) to the bound.  Rows of 2-6 elements have no
# usable scale of their own when the row is the nearly cancelling sum of many unit-size terms
# (the rounding error follows the size of the terms, not of what is left), so the tests over
# such narrow tables take a tenth of the array's scale as the floor.
def assert_close(got, ref, rtol=RTOL, what="", rows=False, outliers=None, global_floor=0.0):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    if ref.size == 0:
        return
    if rows:
        rms = np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True))
    else:
        rms = float(np.sqrt(np.mean(ref * ref)))
    err = np.abs(got - ref)
    bound = rtol * np.abs(ref) + rtol * rms
    if global_floor:
        bound = bound + global_floor * rtol * float(np.sqrt(np.mean(ref * ref)))
    bad = err > bound
    _log_tolerance(what, err, bound, rtol, rows, outliers, global_floor)
    if outliers is not None and bad.any():
        frac, factor = outliers
        if bad.mean() <= frac and not (err > factor * bound).any():
            return
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())}/{ref.size} outside tolerance; worst at {i}: "
                             f"got {got[i]!r} ref {ref[i]!r} err {err[i]:.3e} bound {bound[i]:.3e}")


def _log_tolerance(what, err, bound, rtol, rows, outliers, global_floor):
    """With KGE_TOL_LOG=<file> every comparison appends its worst error relative to its bound (one JSON line):
    the measured margins behind the tolerance table of the design notes."""
    import json
    import os
    path = os.environ.get("KGE_TOL_LOG")
    if not path:
        return
    ratio = float(np.max(err / np.maximum(bound, 1e-300)))
    test = os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0]
    with open(path, "a") as f:
        f.write(json.dumps({"test": test, "what": what, "n": int(err.size), "worst_over_bound": ratio,
                            "rtol": rtol, "rows": bool(rows), "outliers": outliers, "global_floor": global_floor}) + "\n")


def gpu_model(w, device="cuda:0"):
    """KGEModel + index tensors on the GPU for a synth.Workload."""
    from cuke_amd.kge import KGEModel
    a = w.arrays
    dev = torch.device(device)
    E = torch.from_numpy(a["E"]).to(dev)
    R = torch.from_numpy(a["R"]).to(dev) if a["R"] is not None and a["R"].size else None
    A = torch.from_numpy(a["A"]).to(dev) if a["A"] is not None else None
    m = KGEModel(w.model, E, R, A, norm_p=w.norm_p, gamma=w.gamma)
    idx = {k: torch.from_numpy(a[k]).to(dev) for k in ("h", "r", "t", "neg") if k in a}
    return m, idx


def compare_l1_generic(oracle, w, a, g, ref, dmax, what, fast=False):
    """L1 gradients on generic floats.  A residual element within rounding of zero may take either sign in
    two correct fp32 evaluations, and one flipped sign moves every column of the rows of that pair (through
    q.w).  The oracle counts, per row, the such elements that can reach it (|u| <= 6e-8, a few ulps of the
    operands); a row with none must meet the ordinary bar, and a reachable row may be off by at most ITS OWN
    flips (each changes a pair's q_j by 2|g| and, through (q.w) w and (q.w) d0, the other columns by less)."""
    cnt_e, cnt_r, n_amb = oracle.l1_ambiguous_rows(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"],
                                                   a.get("neg"), w.chunk, eps=6e-8, fast=fast)
    amb_e, amb_r = cnt_e > 0, cnt_r > 0
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids) and np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
    assert amb_e.mean() < 0.5, f"{what}: the mask must leave most rows to the ordinary bar ({amb_e.mean():.2f} masked)"
    for name, amb, cnt in (("ent_rows", amb_e, cnt_e), ("rel_rows", amb_r, cnt_r), ("aux_rows", amb_r, cnt_r)):
        got, want = getattr(g, name).cpu().numpy(), getattr(ref, name)
        assert_close(got[~amb], want[~amb], what=f"{what} {name} clear of sign ambiguity", rows=True)
        # a masked row: the flips that can reach THIS row bound it, on top of the ordinary bar
        err = np.abs(got[amb].astype(np.float64) - want[amb])
        rms = np.sqrt(np.mean(want[amb].astype(np.float64) ** 2, axis=-1, keepdims=True))
        bound = 2.0 * dmax * cnt[amb][:, None] * (1 + 1e-3) + RTOL * np.abs(want[amb]) + RTOL * rms
        assert (err <= bound).all() if err.size else True, f"{what} {name}: a masked row is off by more than its own flips"
    return int(amb_e.sum()), n_amb
