"""The benchmark configurations at their full sizes.

Every configuration is small enough for the CPU oracle to finish in seconds to a minute, so the
forward scores and the sparse gradients are compared directly at full size, and on top of that
through properties that do not need the oracle at all: a shared-negative score must equal the
per-triple score of the explicit triple (h, r, neg), the backward pass is linear in the upstream
gradients, and gradient rows are invariant under a permutation of the chunks."""
import numpy as np
import pytest
import torch

from cuke_amd import synth
from helpers import assert_close, compare_l1_generic, gpu_model

pytestmark = pytest.mark.gpu

FULL = ["cfg1_transe", "cfg2_distmult", "cfg2_complex", "cfg3_transr", "cfg4_rotate", "cfg5_transh"]


@pytest.fixture(scope="module", params=FULL)
def full(request):
    # cfg5 is scored with the L1 norm: lattice-valued tables keep every residual away from the
    # sign discontinuity of the L1 gradient
    w = synth.make_workload(request.param, lattice=(request.param == "cfg5_transh"))
    m, ix = gpu_model(w)
    rel = None
    if w.model == "TransR":
        from cuke_amd.kge import inspect
        rel = inspect([ix["r"]], m.n_rel)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, rel_insp=rel)
    yield w, m, ix, fw
    del m, ix, fw
    torch.cuda.empty_cache()


def upstream(w, seed):
    rng = np.random.default_rng(seed)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32) if w.chunk else None
    return dpos, dneg


def dev(x):
    return None if x is None else torch.from_numpy(x).cuda()


def test_forward_against_oracle(oracle, full):
    w, m, ix, fw = full
    a = w.arrays
    pos, negs = oracle.score(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a.get("neg"), w.chunk,
                             p=w.norm_p, gamma=w.gamma)
    assert_close(fw.pos.cpu().numpy(), pos, what=f"{w.name} pos")
    if w.chunk:
        assert_close(fw.neg.cpu().numpy(), negs, what=f"{w.name} neg")


def test_backward_against_oracle(oracle, full):
    w, m, ix, fw = full
    if not w.backward:
        pytest.skip("forward-only configuration")
    a = w.arrays
    dpos, dneg = upstream(w, 11)
    g = m.backward(fw, dev(dpos), dev(dneg))
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a.get("neg"), w.chunk,
                          dpos, dneg, p=w.norm_p)
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids)
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
    out = (1e-5, 4.0) if w.model == "RotatE" else None
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{w.name} entity rows", rows=True, outliers=out)
    if ref.rel_rows is not None and ref.rel_rows.size:
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=f"{w.name} relation rows", rows=True,
                     outliers=out)
    if ref.aux_rows is not None:
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{w.name} aux rows", rows=True)


def test_shared_negative_equals_explicit_triple(full):
    """neg[b, k] from the tile kernels == the positive-path score of (h[b], r[b], neg[(b / C) * N + k])."""
    w, m, ix, fw = full
    if not w.chunk:
        pytest.skip("no negatives")
    g = torch.Generator(device="cpu").manual_seed(5)
    n = 200_000
    b = torch.randint(0, w.batch, (n,), generator=g).cuda()
    k = torch.randint(0, w.n_neg, (n,), generator=g).cuda()
    tails = ix["neg"][(b // w.chunk) * w.n_neg + k]
    explicit = m.score(ix["h"][b], ix["r"][b], tails).pos
    assert_close(fw.neg[b, k].cpu().numpy(), explicit.cpu().numpy(), what=f"{w.name} sampled negatives")


def test_backward_is_linear_in_upstream_gradients(full):
    w, m, ix, fw = full
    if not w.backward:
        pytest.skip("forward-only configuration")
    x = upstream(w, 21)
    y = upstream(w, 22)
    ca, cb = np.float32(0.75), np.float32(-1.5)
    mix = tuple(None if u is None else ca * u + cb * v for u, v in zip(x, y))
    gx = m.backward(fw, dev(x[0]), dev(x[1]))
    gy = m.backward(fw, dev(y[0]), dev(y[1]))
    gm = m.backward(fw, dev(mix[0]), dev(mix[1]))
    assert torch.equal(gx.ent_ids, gm.ent_ids) and torch.equal(gx.rel_ids, gm.rel_ids)
    for name in ("ent_rows", "rel_rows", "aux_rows"):
        rx, ry, rm = getattr(gx, name), getattr(gy, name), getattr(gm, name)
        if rm is None or rm.numel() == 0:
            continue
        want = float(ca) * rx.double() + float(cb) * ry.double()
        # Three fp32 evaluations are compared with each other, and the combination may cancel, so
        # the error scale is that of the two terms (element and row rms), at 3 x the parity bar.
        size = abs(float(ca)) * rx.double().abs() + abs(float(cb)) * ry.double().abs()
        bound = 3e-5 * (size + size.pow(2).mean(dim=-1, keepdim=True).sqrt())
        bad = (rm.double() - want).abs() > bound
        assert not bool(bad.any()), f"{w.name} linearity of {name}: {int(bad.sum())}/{bad.numel()} outside tolerance"


def test_gradients_invariant_under_chunk_permutation(full):
    """Reordering whole chunks (with their negatives and upstream gradients) permutes the triples
    but not the set of contributions to any table row; only the fp32 summation order changes."""
    w, m, ix, fw = full
    if not w.backward or not w.chunk:
        pytest.skip("needs shared negatives and a backward pass")
    C, N, nc = w.chunk, w.n_neg, w.n_chunks
    perm = torch.randperm(nc, generator=torch.Generator().manual_seed(9)).cuda()
    rows = (perm[:, None] * C + torch.arange(C, device="cuda")[None, :]).reshape(-1)
    nrows = (perm[:, None] * N + torch.arange(N, device="cuda")[None, :]).reshape(-1)
    dpos, dneg = (dev(u) for u in upstream(w, 31))
    g0 = m.backward(fw, dpos, dneg)
    fw2 = m.score(ix["h"][rows], ix["r"][rows], ix["t"][rows], ix["neg"][nrows], C)
    assert torch.equal(fw2.pos, fw.pos[rows]) and torch.equal(fw2.neg, fw.neg[rows])
    g1 = m.backward(fw2, dpos[rows].contiguous(), dneg[rows].contiguous())
    assert torch.equal(g0.ent_ids, g1.ent_ids) and torch.equal(g0.rel_ids, g1.rel_ids)
    out = (1e-5, 4.0) if w.model == "RotatE" else None
    for name in ("ent_rows", "rel_rows", "aux_rows"):
        r0, r1 = getattr(g0, name), getattr(g1, name)
        if r0 is None or r0.numel() == 0:
            continue
        assert_close(r1.cpu().numpy(), r0.cpu().numpy(), what=f"{w.name} {name} after permutation",
                     rows=True, outliers=out)


def test_cfg5_on_its_stated_inputs_at_full_size(oracle):
    """Config 5 as it is stated: a 4,000,000 x 400 entity table N(0, 0.05), 10,000 relations with unit
    normals, 16,384 positives x 1,024 shared negatives, L1 norm.  The tables are drawn on the GPU (as the
    benchmark draws them); the oracle gets the rows the batch names, copied back from the device, under
    compact ids.  Scores: ordinary bar (|u| is continuous, no sign ambiguity in the forward pass).
    Gradients: ordinary bar on every row no sign ambiguity can reach (see compare_l1_generic).  The oracle
    runs its OpenMP build here (same source and loops; threads split the batch)."""
    from cuke_amd.kge import KGEModel
    w = synth.make_workload("cfg5_transh", tables=False)
    a = w.arrays
    E, R, A = synth.device_tables(w, torch.device("cuda:0"))
    assert torch.allclose(A.norm(dim=1), torch.ones(w.n_rel, device=A.device), atol=1e-5)
    m = KGEModel(w.model, E, R, A, norm_p=1)
    ix = {k: torch.from_numpy(a[k]).cuda() for k in ("h", "r", "t", "neg")}
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    ue, ur = np.unique(np.concatenate([a["h"], a["t"], a["neg"]])), np.unique(a["r"])
    c = dict(E=E[torch.from_numpy(ue).cuda()].cpu().numpy(), R=R[torch.from_numpy(ur).cuda()].cpu().numpy(),
             A=A[torch.from_numpy(ur).cuda()].cpu().numpy(), h=np.searchsorted(ue, a["h"]), t=np.searchsorted(ue, a["t"]),
             r=np.searchsorted(ur, a["r"]), neg=np.searchsorted(ue, a["neg"]))
    pos, negs = oracle.score("TransH", c["E"], c["R"], c["A"], c["h"], c["r"], c["t"], c["neg"], w.chunk, p=1,
                             fast="omp")
    assert_close(fw.pos.cpu().numpy(), pos, what="cfg5 (stated inputs) pos")
    assert_close(fw.neg.cpu().numpy(), negs, what="cfg5 (stated inputs) neg")
    dpos, dneg = upstream(w, 13)
    g = m.backward(fw, dev(dpos), dev(dneg))
    ref = oracle.backward("TransH", c["E"], c["R"], c["A"], c["h"], c["r"], c["t"], c["neg"], w.chunk, dpos, dneg,
                          p=1, fast="omp")
    ref.ent_ids, ref.rel_ids = ue[ref.ent_ids], ur[ref.rel_ids]  # compact ids back to table ids
    dmax = float(max(np.abs(dpos).max(), np.abs(dneg).max()))
    compare_l1_generic(oracle, w, c, g, ref, dmax, "cfg5 (stated inputs)", fast="omp")


@pytest.mark.parametrize("model,p", [("DistMult", 2), ("TransE", 2)])
def test_more_than_2_to_31_scores(model, p):
    """262144 x 8192 negatives = 2^31 scores per call: element offsets into the score and upstream
    gradient arrays pass the 32-bit range.  Forward: sampled (b, k) against the per-triple path.
    Backward: the whole batch against the sum of its two halves run as separate calls."""
    C, N, nc, d = 1024, 8192, 256, 32
    w = synth.custom_workload(model, n_ent=100_000, n_rel=100, dim=d, batch=C * nc, chunk=C, n_neg=N, norm_p=p,
                              sigma=0.3, seed=77)
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], C)
    assert fw.neg.numel() == 1 << 31
    gen = torch.Generator(device="cpu").manual_seed(6)
    b = torch.randint(0, w.batch, (300_000,), generator=gen).cuda()
    k = torch.randint(0, N, (300_000,), generator=gen).cuda()
    b[:4] = w.batch - 1  # the last rows sit at the top of the offset range
    k[:4] = torch.tensor([N - 1, N - 2, 0, 1])
    explicit = m.score(ix["h"][b], ix["r"][b], ix["neg"][(b // C) * N + k]).pos
    assert_close(fw.neg[b, k].cpu().numpy(), explicit.cpu().numpy(), what=f"{model} sampled negatives")

    dpos = torch.randn(w.batch, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    dneg = torch.randn(w.batch, N, device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    g = m.backward(fw, dpos, dneg)
    want_e = torch.zeros(w.n_ent, d, dtype=torch.float64, device="cuda")
    want_r = torch.zeros(w.n_rel, d, dtype=torch.float64, device="cuda")
    half = w.batch // 2
    for lo in (0, half):
        rows = slice(lo, lo + half)
        nrows = slice(lo // C * N, (lo + half) // C * N)
        fh = m.score(ix["h"][rows], ix["r"][rows], ix["t"][rows], ix["neg"][nrows], C)
        assert torch.equal(fh.neg, fw.neg[rows])
        gh = m.backward(fh, dpos[rows], dneg[rows])
        want_e.index_add_(0, gh.ent_ids, gh.ent_rows.double())
        want_r.index_add_(0, gh.rel_ids, gh.rel_rows.double())
        del fh, gh
    assert_close(g.ent_rows.cpu().numpy(), want_e[g.ent_ids].cpu().numpy(), what=f"{model} entity rows",
                 rows=True)
    assert_close(g.rel_rows.cpu().numpy(), want_r[g.rel_ids].cpu().numpy(), what=f"{model} relation rows",
                 rows=True)
    touched = torch.zeros(w.n_ent, dtype=torch.bool, device="cuda")
    touched[g.ent_ids] = True
    assert not bool(want_e[~touched].any())


def test_preallocated_step_with_riding_inspection_equals_the_eager_path_bit_for_bit(full):
    """TrainStep.run() at full size (inspection riding inside the score kernels' launches, tile plans
    reused by backward) must give exactly the bits of KGEModel.score + backward with the stand-alone
    inspector: the same kernels do the arithmetic, only where the inspector's workgroups run differs."""
    from cuke_amd.kge import TrainStep
    w, m, ix, fw = full
    if not w.backward:
        pytest.skip("forward-only configuration")
    dpos, dneg = upstream(w, 5)
    g = m.backward(fw, dev(dpos), dev(dneg))
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, dpos=dev(dpos), dneg=dev(dneg),
                     back_rows=fw.back_rows is not None)  # (TransR: the same form of the entity gradients as the eager call)
    assert step.fusable
    step.run()
    torch.cuda.synchronize()
    s = step.sparse_grads()
    assert torch.equal(step.pos, fw.pos) and (fw.neg is None or torch.equal(step.neg, fw.neg))
    assert torch.equal(s.ent_ids, g.ent_ids) and torch.equal(s.rel_ids, g.rel_ids)
    assert torch.equal(s.ent_rows, g.ent_rows)
    for a_, b_ in ((s.rel_rows, g.rel_rows), (s.aux_rows, g.aux_rows)):
        assert (a_ is None) == (b_ is None)
        if a_ is not None:
            assert torch.equal(a_, b_)
