"""Shared helpers for the parity tests."""
import numpy as np
import torch

# fp32 parity bar: |got - ref| <= RTOL * |ref| + RTOL * rms(ref).  The second term is the
# absolute floor for entries that cancel to (nearly) zero: the oracle sums serially with
# separate multiply and add, the GPU sums as a tree with fused multiply-add, and both are
# fp32, so entries much smaller than the array's scale cannot agree to a pure relative bound.
RTOL = 1e-5


def assert_close(got, ref, rtol=RTOL, what=""):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    if ref.size == 0:
        return
    rms = float(np.sqrt(np.mean(ref * ref)))
    err = np.abs(got - ref)
    bound = rtol * np.abs(ref) + rtol * rms
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())}/{ref.size} outside tolerance; worst at {i}: "
                             f"got {got[i]!r} ref {ref[i]!r} err {err[i]:.3e} bound {bound[i]:.3e}")


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
