"""TransR / RESCAL: grouped per-relation MFMA path (forward and backward) against the oracle."""
import numpy as np
import pytest
import torch

from cuke_amd import synth
from helpers import assert_close, gpu_model

pytestmark = pytest.mark.gpu


def grouped_forward(m, ix, for_backward=False):
    from cuke_amd.kge import inspect
    rel = inspect([ix["r"]], m.n_rel)
    return m.score(ix["h"], ix["r"], ix["t"], rel_insp=rel, for_backward=for_backward), rel


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
@pytest.mark.parametrize("shape", [
    dict(dim=16, batch=5, n_rel=3),          # one tile, fewer rows than an MFMA block
    dict(dim=200, batch=300, n_rel=7),       # groups larger than a tile, ragged column split
    dict(dim=256, batch=1000, n_rel=400),    # mostly singletons
    dict(dim=64, batch=257, n_rel=1),        # one group, many tiles
    dict(dim=36, batch=130, n_rel=9),        # K tail (36 = 2 * 16 + 4)
    dict(dim=400, batch=60, n_rel=40),       # wide rows: two column sweeps, thin tails in two k-chunks
    dict(dim=496, batch=24, n_rel=20),
    dict(dim=512, batch=4096, n_rel=30),     # the reference's own sweep shapes (apps/kge/scripts/test_fig9c_cuke.sh):
    dict(dim=1024, batch=1024, n_rel=12),    # left-operand tiles of 66.5 KB and 129 KB in LDS
    dict(dim=50, batch=300, n_rel=40),       # row widths that are not multiples of four: the batch is copied into a
    dict(dim=101, batch=64, n_rel=5),        # padded compact problem (dim is a free variable of the reference's
    dict(dim=202, batch=700, n_rel=90),      # transR, apps/kge/kge.py:321-343)
    dict(dim=7, batch=9, n_rel=2),
])
@pytest.mark.parametrize("p", [1, 2])
def test_grouped_forward(oracle, model, shape, p):
    if model == "RESCAL" and p == 1:
        pytest.skip("no norm in RESCAL")
    w = synth.custom_workload(model, n_ent=500, norm_p=p, sigma=0.2, rel_zipf=1.2, seed=shape["dim"], **shape)
    a = w.arrays
    m, ix = gpu_model(w)
    fw, rel = grouped_forward(m, ix)
    pos, _ = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], p=p)
    assert_close(fw.pos.cpu().numpy(), pos, what=f"{model} {shape} grouped score")
    if model == "TransR":
        want = oracle.residual("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"])
        assert_close(fw.residual.cpu().numpy(), want, what="grouped residual")
        assert_close(m.residual(ix["h"], ix["r"], ix["t"], rel_insp=rel).cpu().numpy(), want,
                     what="grouped residual entry point")
    # the ungrouped per-triple path must agree as well
    assert_close(m.score(ix["h"], ix["r"], ix["t"]).pos.cpu().numpy(), pos, what="ungrouped score")


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
@pytest.mark.parametrize("shape", [
    dict(dim=16, batch=5, n_rel=3),
    dict(dim=200, batch=300, n_rel=7),
    dict(dim=36, batch=130, n_rel=9),
    dict(dim=64, batch=257, n_rel=1),
    dict(dim=400, batch=60, n_rel=40),
    dict(dim=496, batch=24, n_rel=20),
    dict(dim=512, batch=4096, n_rel=30),
    dict(dim=1024, batch=1024, n_rel=12),
    dict(dim=50, batch=300, n_rel=40),
    dict(dim=101, batch=64, n_rel=5),
    dict(dim=202, batch=700, n_rel=90),
    dict(dim=7, batch=9, n_rel=2),
    dict(dim=100, batch=200, n_rel=120),   # thin groups of the back-row kernel: two quads per lane
    dict(dim=160, batch=200, n_rel=120),   # three
    dict(dim=208, batch=300, n_rel=200),   # four, the widest row it keeps in registers
    dict(dim=212, batch=300, n_rel=200),   # the first that takes two sweeps again
])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("back", [False, True])
def test_grouped_backward(oracle, model, shape, p, back):
    """back: the forward pass also writes the rows phi(residual) Proj^T (Forward.back_rows) and the backward
    pass reads no projection again; without them it forms the entity gradients with its own pass."""
    if model == "RESCAL" and p == 1:
        pytest.skip("no norm in RESCAL")
    if back and (model == "RESCAL" or shape["dim"] % 4 != 0):
        pytest.skip("back rows: TransR with row widths that are multiples of four")
    w = synth.custom_workload(model, n_ent=120, norm_p=p, sigma=0.2, rel_zipf=1.2, ent_zipf=1.1,
                              seed=shape["dim"] + p, lattice=(p == 1 and model == "TransR"), **shape)
    a = w.arrays
    if w.lattice:  # keep the projected residual exact too: projections on a coarse grid
        a["A"] = (np.rint(a["A"] / 0.2 * 2) / 8).astype(np.float32)
    m, ix = gpu_model(w)
    fw, rel = grouped_forward(m, ix, for_backward=back)
    assert (fw.back_rows is not None) == back
    dpos = np.random.default_rng(1).standard_normal(w.batch).astype(np.float32)
    g = m.backward(fw, torch.from_numpy(dpos).to(fw.pos.device))
    ref = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], dpos=dpos, p=p)
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids)
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
    # dX = Q M^T sums `dim` products per element.  With the L1 norm every q_j is +-g, so a row of dX is
    # g times an alternating sum of projection entries: the partial sums are an order of magnitude above
    # the result, and fp32 accumulation (GPU) differs from the oracle's double accumulation by
    # eps * sqrt(dim) * sum|terms|, not by eps * |result|.  For the wide rows the floor is therefore the
    # scale of the whole array rather than of the (cancelled) row.
    floor = 2.0 if (p == 1 and shape["dim"] >= 400) else 0.0
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what="entity rows", rows=True, global_floor=floor)
    if model == "TransR":
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what="relation rows", rows=True)
    assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what="projection gradients", rows=True)


def dense_projection_gradients(g):
    """Dense [U, dim * dim] projection gradients from partly factored ones: a factored group's matrix is the sum
    of the outer products of its rows (float64 on the host; what the device left in aux_rows for such a group
    is ignored)."""
    off = g.rel_seg_offsets.cpu().numpy()
    x, q = g.aux_x.cpu().numpy().astype(np.float64), g.aux_q.cpu().numpy().astype(np.float64)
    out = g.aux_rows.cpu().numpy().astype(np.float64).copy()
    d = x.shape[1]
    factored = 0
    for u in range(len(off) - 1):
        if off[u + 1] - off[u] <= g.factor_max:
            out[u] = (x[off[u]:off[u + 1]].T @ q[off[u]:off[u + 1]]).reshape(d * d)
            factored += 1
    return out, factored


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("fmax", [1, 3, 4])
@pytest.mark.parametrize("shape", [dict(dim=200, batch=300, n_rel=150), dict(dim=36, batch=130, n_rel=60),
                                   dict(dim=512, batch=64, n_rel=40)])
def test_factored_projection_gradients_equal_the_dense_ones(oracle, model, p, fmax, shape):
    """kge_grads.aux_x / aux_q: groups of at most fmax triples leave x_p, q_p instead of the dense matrix;
    sum_p x_p^T q_p must be the oracle's dense gradient, larger groups stay dense, and the poisoned dense rows
    of the factored groups must not have been written."""
    if model == "RESCAL" and p == 1:
        pytest.skip("no norm in RESCAL")
    w = synth.custom_workload(model, n_ent=120, norm_p=p, sigma=0.2, rel_zipf=1.2, ent_zipf=1.1,
                              seed=shape["dim"] + p, lattice=(p == 1 and model == "TransR"), **shape)
    a = w.arrays
    if w.lattice:
        a["A"] = (np.rint(a["A"] / 0.2 * 2) / 8).astype(np.float32)
    m, ix = gpu_model(w)
    fw, rel = grouped_forward(m, ix)
    dpos = np.random.default_rng(1).standard_normal(w.batch).astype(np.float32)
    dense = m.backward(fw, torch.from_numpy(dpos).cuda())
    g = m.backward(fw, torch.from_numpy(dpos).cuda(), factor_max=fmax)
    ref = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], dpos=dpos, p=p)
    got, n_fact = dense_projection_gradients(g)
    counts = np.diff(g.rel_seg_offsets.cpu().numpy())
    assert n_fact == int((counts <= fmax).sum()) and 0 < n_fact < len(counts), "the shape must mix both kinds of group"
    assert_close(got, ref.aux_rows, what=f"{model} fmax={fmax} projection gradients (factored groups multiplied out)", rows=True)
    # the other outputs do not depend on the form, bit for bit
    assert torch.equal(g.ent_rows, dense.ent_rows)
    if model == "TransR":
        assert torch.equal(g.rel_rows, dense.rel_rows)
    big = torch.from_numpy(counts > fmax).cuda()
    assert torch.equal(g.aux_rows[big], dense.aux_rows[big]), "dense groups are the same bits in both forms"


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
@pytest.mark.parametrize("rule", ["sgd", "adagrad"])
def test_factored_optimizer_step_equals_the_dense_one(oracle, model, rule):
    """kge_sparse_sgd_factored / kge_sparse_adagrad_factored on partly factored gradients against
    kge_sparse_sgd / kge_sparse_adagrad on the dense gradients of the same batch (the oracle-pinned rules)."""
    from cuke_amd import kge
    w = synth.custom_workload(model, n_ent=200, n_rel=80, dim=64, batch=256, norm_p=2, sigma=0.2, rel_zipf=1.2, seed=11)
    m, ix = gpu_model(w)
    fw, rel = grouped_forward(m, ix)
    dpos = torch.from_numpy(np.random.default_rng(2).standard_normal(w.batch).astype(np.float32)).cuda()
    dense = m.backward(fw, dpos)
    fact = m.backward(fw, dpos, factor_max=4)
    n_rel, d = m.A.shape[0], m.dim
    ref_tab, got_tab = m.A.clone().view(n_rel, d * d), m.A.clone()
    if rule == "sgd":
        kge.sparse_sgd(ref_tab, rel, dense.aux_rows, 0.1)
        kge.sparse_sgd_factored(got_tab, fact, 0.1)
    else:
        st0 = torch.rand(n_rel, device="cuda") * 1e-3
        ref_state, got_state = st0.clone(), st0.clone()
        kge.sparse_adagrad(ref_tab, ref_state, rel, dense.aux_rows, 0.1)
        kge.sparse_adagrad_factored(got_tab, got_state, fact, 0.1)
        assert_close(got_state.cpu().numpy(), ref_state.cpu().numpy(), what="Adagrad state")
    assert_close(got_tab.view(n_rel, d * d).cpu().numpy(), ref_tab.cpu().numpy(), what=f"{model} {rule} projection table", rows=True)
    touched = torch.zeros(n_rel, dtype=torch.bool, device="cuda")
    touched[fact.rel_ids] = True
    assert torch.equal(got_tab[~touched], m.A[~touched]), "rows of relations outside the batch must not move"


def test_train_step_factored_all_issue_forms(oracle):
    """TrainStep(factor_max=4) through the one-stream, fused, side-stream and staged issues: every form leaves
    the same factored rows, and multiplied out they are the oracle's dense gradients."""
    from cuke_amd.kge import TrainStep
    ws = [synth.make_workload("cfg3_transr", batch=1024, seed=s) for s in range(3)]
    m, ix0 = gpu_model(ws[0])
    step = TrainStep(m, ix0["h"], ix0["r"], ix0["t"], factor_max=4)
    for w in ws[1:]:
        ix = {k: torch.from_numpy(w.arrays[k]).cuda() for k in ("h", "r", "t")}
        step.add_batch(ix["h"], ix["r"], ix["t"])
    a0 = ws[0].arrays

    def check(w, tag):
        torch.cuda.synchronize()
        a = w.arrays
        ref = oracle.backward("TransR", a0["E"], a0["R"], a0["A"], a["h"], a["r"], a["t"], dpos=step.dpos.cpu().numpy(), p=2)
        g = step.sparse_grads()
        assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), tag
        got, n_fact = dense_projection_gradients(g)
        assert n_fact > 0
        assert_close(got, ref.aux_rows, what=f"{tag} projection gradients", rows=True)
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{tag} entity rows", rows=True)
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=f"{tag} relation rows", rows=True)

    step.run(overlap=False, fused=False)
    check(ws[0], "one stream")
    if step.fusable:
        step.aux_x.zero_(), step.aux_q.zero_()
        step.run(fused=True)
        check(ws[0], "fused inspection")
    step.run(fused=False)
    check(ws[0], "side-stream inspection")
    step.stage(batch=1)
    for i in (1, 2, 0):
        step.stage(batch=(i + 1) % 3)
        step.run(pipeline=True)
        check(ws[i], f"staged batch {i}")
    step.run(pipeline=True)
    check(ws[1], "drained")


def test_train_step_with_an_odd_row_width(oracle):
    """TransR at dim 50 through TrainStep: one stream, side-stream inspection and the staged issue (tile plans a
    batch ahead, kge_transr_plan on the padded problem), against the oracle."""
    from cuke_amd.kge import TrainStep
    ws = [synth.custom_workload("TransR", n_ent=300, n_rel=25, dim=50, batch=256, norm_p=2, sigma=0.2, rel_zipf=1.2, seed=s)
          for s in range(3)]
    m, ix0 = gpu_model(ws[0])
    step = TrainStep(m, ix0["h"], ix0["r"], ix0["t"])
    assert not step.fusable
    for w in ws[1:]:
        ix = {k: torch.from_numpy(w.arrays[k]).cuda() for k in ("h", "r", "t")}
        step.add_batch(ix["h"], ix["r"], ix["t"])
    a0 = ws[0].arrays

    def check(w, tag):
        torch.cuda.synchronize()
        a = w.arrays
        pos, _ = oracle.score("TransR", a0["E"], a0["R"], a0["A"], a["h"], a["r"], a["t"], p=2)
        assert_close(step.pos.cpu().numpy(), pos, what=f"{tag} scores")
        ref = oracle.backward("TransR", a0["E"], a0["R"], a0["A"], a["h"], a["r"], a["t"], dpos=step.dpos.cpu().numpy(), p=2)
        g = step.sparse_grads()
        assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), tag
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{tag} entity rows", rows=True)
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=f"{tag} relation rows", rows=True)
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{tag} projection gradients", rows=True)

    step.run(overlap=False)
    check(ws[0], "one stream")
    step.run()
    check(ws[0], "side-stream inspection")
    step.stage(batch=1)
    for i in (1, 2, 0):
        step.stage(batch=(i + 1) % 3)
        step.run(pipeline=True)
        check(ws[i], f"staged batch {i}")
    step.run(pipeline=True)
    check(ws[1], "drained")


def test_cfg3_scaled(oracle):
    w = synth.make_workload("cfg3_transr", batch=2048)
    a = w.arrays
    m, ix = gpu_model(w)
    fw, rel = grouped_forward(m, ix)
    pos, _ = oracle.score("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], p=2)
    assert_close(fw.pos.cpu().numpy(), pos, what="cfg3 scores")
    dpos = np.random.default_rng(2).standard_normal(w.batch).astype(np.float32)
    g = m.backward(fw, torch.from_numpy(dpos).to(fw.pos.device))
    ref = oracle.backward("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], dpos=dpos, p=2)
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what="cfg3 entity rows", rows=True)
    assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what="cfg3 relation rows", rows=True)
    assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what="cfg3 projection gradients", rows=True)


def test_proj_identity_reduces_to_transe(oracle):
    w = synth.custom_workload("TransR", n_ent=300, n_rel=5, dim=64, batch=200, sigma=0.2, seed=3)
    a = w.arrays
    a["A"] = np.broadcast_to(np.eye(64, dtype=np.float32), (5, 64, 64)).copy()
    m, ix = gpu_model(w)
    fw, _ = grouped_forward(m, ix)
    te, _ = oracle.score("TransE", a["E"], a["R"], None, a["h"], a["r"], a["t"], p=2)
    assert_close(fw.pos.cpu().numpy(), te, what="Proj = I")


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
def test_shared_negatives_through_flattened_triples(oracle, model):
    # neg_transR (examples.py:1447-1480): out[b * bs + k] = (E[h[b]] - E[t'[k]]) Proj[r[b]] + R[r[b]]
    w = synth.custom_workload(model, n_ent=200, n_rel=6, dim=40, batch=48, chunk=16, n_neg=12, sigma=0.2,
                              rel_zipf=1.1, ent_zipf=1.1, seed=5)
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m._score_projected_negatives(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    pos, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, p=2)
    assert_close(fw.pos.cpu().numpy(), pos, what="pos")
    assert_close(fw.neg.cpu().numpy(), negs, what="neg")
    if model == "TransR":  # the reference's output: one residual row per (b, k), b-major
        fh = np.repeat(a["h"], w.n_neg); fr = np.repeat(a["r"], w.n_neg)
        ft = np.array([a["neg"][(b // w.chunk) * w.n_neg + k] for b in range(w.batch) for k in range(w.n_neg)])
        want = oracle.residual("TransR", a["E"], a["R"], a["A"], fh, fr, ft)
        assert_close(fw.residual[w.batch:].cpu().numpy(), want, what="neg_transR residual rows")
    rng = np.random.default_rng(3)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
    g = m.backward(fw, torch.from_numpy(dpos).cuda(), torch.from_numpy(dneg).cuda())
    ref = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, dpos, dneg, p=2)
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids)
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what="entity rows", rows=True)
    if model == "TransR":
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what="relation rows", rows=True)
    assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what="projection gradients", rows=True)


@pytest.mark.parametrize("shape", [
    dict(dim=40, batch=48, chunk=16, n_neg=12, n_rel=6),
    dict(dim=200, batch=512, chunk=64, n_neg=64, n_rel=50),    # Zipf relations, many thin groups
    dict(dim=64, batch=300, chunk=300, n_neg=33, n_rel=1),     # one relation, odd N, ragged tiles
    dict(dim=128, batch=512, chunk=128, n_neg=128, n_rel=100),  # several 64-row tiles per chunk on both sides
    dict(dim=16, batch=7, chunk=7, n_neg=1, n_rel=3),
])
@pytest.mark.parametrize("mode", ["tail", "head"])
def test_rescal_shared_negatives_as_a_dot_product_tile(oracle, shape, mode):
    """RESCAL with shared negatives: (E[h] Proj[r]) . E[t'] for replaced tails, E[h'] . (Proj[r] E[t]) for replaced
    heads, from B projected rows and the dot-product tile kernel (no projection of the negatives, no flattened
    triples), forward and backward against the oracle's explicit pairs; with missing upstream gradients; and
    through TrainStep."""
    from cuke_amd.kge import TrainStep
    w = synth.custom_workload("RESCAL", n_ent=400, norm_p=2, sigma=0.2, rel_zipf=1.1, ent_zipf=1.1, seed=13, **shape)
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=mode)
    assert fw.flat_pos is None, "the flattened triples ran instead of the tile path"
    pos, negs = oracle.score("RESCAL", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, neg_mode=mode)
    assert_close(fw.pos.cpu().numpy(), pos, what="pos")
    assert_close(fw.neg.cpu().numpy(), negs, what="neg")
    rng = np.random.default_rng(5)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
    for gp, gn, tag in ((dpos, dneg, "both"), (None, dneg, "pairs only"), (dpos, None, "positives only")):
        g = m.backward(fw, None if gp is None else torch.from_numpy(gp).cuda(), None if gn is None else torch.from_numpy(gn).cuda())
        ref = oracle.backward("RESCAL", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                              gp if gp is not None else np.zeros_like(dpos), gn if gn is not None else np.zeros_like(dneg),
                              neg_mode=mode)
        assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids) and np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{tag}: entity rows", rows=True)
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{tag}: projection gradients", rows=True)
    # the flattened formulation of the reference must agree
    flat = m._score_projected_negatives(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, mode)
    assert_close(fw.neg.cpu().numpy(), flat.neg.cpu().numpy(), what="tile path vs flattened triples")
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, dpos=torch.from_numpy(dpos).cuda(),
                     dneg=torch.from_numpy(dneg).cuda(), neg_mode=mode)
    ref = oracle.backward("RESCAL", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, dpos, dneg,
                          neg_mode=mode)
    for tag, kw in (("side stream", {}), ("one stream", dict(overlap=False))):
        step.run(**kw)
        torch.cuda.synchronize()
        g = step.sparse_grads()
        assert_close(step.neg.cpu().numpy(), negs, what=f"TrainStep {tag} neg")
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"TrainStep {tag} entity rows", rows=True)
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"TrainStep {tag} projection gradients", rows=True)


def _neg_case(oracle, w, mode, what):
    a = w.arrays
    if w.lattice:  # keep the projected rows exact too: projections on a coarse grid (L1 gradients are sums of signs)
        a["A"] = (np.rint(a["A"] / 0.2 * 2) / 8).astype(np.float32)
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=mode)
    assert fw.fwd_ws is not None and fw.flat_pos is None, "the grouped shared-negative path did not run"
    pos, negs = oracle.score("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, p=w.norm_p,
                             neg_mode=mode)
    assert_close(fw.pos.cpu().numpy(), pos, what=f"{what} pos")
    assert_close(fw.neg.cpu().numpy(), negs, what=f"{what} neg")
    want = oracle.residual("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"])
    assert_close(fw.residual.cpu().numpy(), want, what=f"{what} residual rows of the positives", rows=True)
    rng = np.random.default_rng(w.seed + 11)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
    g = m.backward(fw, torch.from_numpy(dpos).cuda(), torch.from_numpy(dneg).cuda())
    ref = oracle.backward("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, dpos, dneg,
                          p=w.norm_p, neg_mode=mode)
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids)
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{what} entity rows", rows=True)
    assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=f"{what} relation rows", rows=True)
    assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{what} projection gradients", rows=True)
    return m, ix, fw


# Shared negatives with every negative projected once per (relation, chunk) group: the scores and
# gradients of the reference's neg_transR (examples.py:1447-1480) without its batch * blocksize
# vector x matrix products.
@pytest.mark.parametrize("shape", [
    dict(dim=40, batch=48, chunk=16, n_neg=12, n_rel=6),       # a few groups per chunk
    dict(dim=200, batch=512, chunk=64, n_neg=64, n_rel=50),    # benchmark-like: Zipf relations, many singleton groups
    dict(dim=300, batch=96, chunk=96, n_neg=5, n_rel=4),       # one chunk, rows wider than 256 floats, odd N
    dict(dim=16, batch=64, chunk=8, n_neg=2, n_rel=40),        # more relations than positives per chunk; thin dM groups
    dict(dim=64, batch=300, chunk=300, n_neg=33, n_rel=1),     # one relation: a single group
    dict(dim=528, batch=64, chunk=32, n_neg=16, n_rel=3),      # three quads of a row per lane
    dict(dim=8, batch=7, chunk=7, n_neg=1, n_rel=3),           # fewer positives than one reduction block, one negative
    dict(dim=12, batch=45, chunk=5, n_neg=3, n_rel=2),         # nine chunks of five: groups straddle the reduction blocks
])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("mode", ["tail", "head"])
def test_shared_negatives_projected_once_per_group(oracle, shape, p, mode):
    w = synth.custom_workload("TransR", n_ent=500, norm_p=p, sigma=0.2, rel_zipf=1.1, ent_zipf=1.1, seed=7,
                              lattice=(p == 1), **shape)
    _neg_case(oracle, w, mode, f"{shape} p={p} {mode}")


def test_shared_negatives_grouped_path_equals_the_flattened_one(oracle):
    w = synth.custom_workload("TransR", n_ent=400, n_rel=20, dim=128, batch=256, chunk=64, n_neg=32, sigma=0.2,
                              rel_zipf=1.2, seed=3)
    m, ix, fw = _neg_case(oracle, w, "tail", "grouped")
    flat = m._score_projected_negatives(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    assert_close(fw.neg.cpu().numpy(), flat.neg.cpu().numpy(), what="grouped vs flattened negative scores")
    assert_close(fw.pos.cpu().numpy(), flat.pos.cpu().numpy(), what="grouped vs flattened positive scores")


@pytest.mark.parametrize("mode", ["tail", "head"])
def test_train_step_with_shared_negatives_and_margin_loss(oracle, mode):
    """The preallocated training step drives the grouped shared-negative path: relation inspection on the
    step's stream, entity inspection beside it, forward workspace handed to backward, HIP-graph replay."""
    from cuke_amd.kge import TrainStep
    w = synth.custom_workload("TransR", n_ent=600, n_rel=30, dim=64, batch=384, chunk=64, n_neg=48, norm_p=2, sigma=0.2,
                              rel_zipf=1.1, ent_zipf=1.1, seed=9)
    a = w.arrays
    m, ix = gpu_model(w)
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, loss="margin", margin=2.0, sign=-1.0, neg_mode=mode)
    assert not step.fusable
    pos, negs = oracle.score("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk, p=2, neg_mode=mode)

    def check(tag):
        torch.cuda.synchronize()
        assert_close(step.pos.cpu().numpy(), pos, what=f"{tag} pos")
        assert_close(step.neg.cpu().numpy(), negs, what=f"{tag} neg")
        ref = oracle.backward("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                              step.dpos.cpu().numpy(), step.dneg.cpu().numpy(), p=2, neg_mode=mode)
        g = step.sparse_grads()
        assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids) and np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids)
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{tag} entity rows", rows=True)
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=f"{tag} relation rows", rows=True)
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{tag} projection gradients", rows=True)

    step.run()
    check("side-stream inspection")
    step.run(overlap=False)
    check("one stream")
    graph = step.capture()
    for i in range(3):  # replays with eager work and synchronisation between them
        step.neg.zero_()
        graph.replay()
        check(f"graph replay {i}")


def test_staged_batches_are_planned_a_step_ahead(oracle):
    """stage(batch=i) inspects the relations of an added batch and builds its tile plans on the side stream
    (kge_transr_plan); run(pipeline=True) then starts with the projection kernel (kge_batch.plans_ready).
    Every step must match the oracle on its own batch, and a plain run() afterwards still plans for itself."""
    from cuke_amd.kge import TrainStep
    ws = [synth.make_workload("cfg3_transr", batch=1024, seed=s) for s in range(4)]
    m, ix0 = gpu_model(ws[0])
    step = TrainStep(m, ix0["h"], ix0["r"], ix0["t"])
    for w in ws[1:]:
        ix = {k: torch.from_numpy(w.arrays[k]).cuda() for k in ("h", "r", "t")}
        step.add_batch(ix["h"], ix["r"], ix["t"])
    a0 = ws[0].arrays

    def check(w, tag):
        torch.cuda.synchronize()
        a = w.arrays
        ref = oracle.backward("TransR", a0["E"], a0["R"], a0["A"], a["h"], a["r"], a["t"], dpos=step.dpos.cpu().numpy(), p=2)
        g = step.sparse_grads()
        assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), tag
        assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{tag} entity rows", rows=True)
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{tag} projection gradients", rows=True)

    step.stage(batch=0)
    for i in range(6):
        step.stage(batch=(i + 1) % 4)     # one batch ahead
        step.run(pipeline=True)           # consumes batch i % 4
        check(ws[i % 4], f"staged step {i}")
    step.run(pipeline=True)               # the batch still staged
    check(ws[6 % 4], "drained")
    step.select(1)
    step.run()
    check(ws[1], "plain run afterwards")


@pytest.mark.parametrize("p", [1, 2])
def test_train_step_with_and_without_back_rows(oracle, p):
    """TrainStep(back_rows=True), the default where the batch qualifies, against back_rows=False: the two forms
    round differently (another summation order in the thin groups' forward products; the coefficient applied
    after instead of before the product with the transposed projection) and both meet the oracle."""
    from cuke_amd.kge import TrainStep
    w = synth.make_workload("cfg3_transr", batch=2048, seed=5, norm_p=p)
    m, ix = gpu_model(w)
    a = w.arrays
    dpos = torch.from_numpy(np.random.default_rng(3).standard_normal(w.batch).astype(np.float32)).cuda()
    steps = [TrainStep(m, ix["h"], ix["r"], ix["t"], dpos=dpos, back_rows=b) for b in (True, False)]
    assert steps[0].back_rows is not None and steps[1].back_rows is None
    ref = oracle.backward("TransR", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], dpos=dpos.cpu().numpy(), p=p)
    outs = []
    for st in steps:
        st.run(overlap=False, fused=False)
        torch.cuda.synchronize()
        g = st.sparse_grads()
        if p == 2:
            assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what="entity rows", rows=True)
        outs.append((st.pos.clone(), g.ent_ids.clone(), g.ent_rows.clone(), g.rel_rows.clone(), g.aux_rows.clone()))
    # (the forward kernel that also writes the back rows sums a thin group's products in another order)
    assert torch.equal(outs[0][1], outs[1][1])
    assert_close(outs[0][0].cpu().numpy(), outs[1][0].cpu().numpy(), what="scores")
    if p == 2:
        assert_close(outs[0][3].cpu().numpy(), outs[1][3].cpu().numpy(), what="relation rows", rows=True)
        assert_close(outs[0][4].cpu().numpy(), outs[1][4].cpu().numpy(), what="projection gradients", rows=True)
    assert_close(outs[0][2].cpu().numpy(), outs[1][2].cpu().numpy(), what="entity rows, back rows against the dX pass",
                 rows=True, global_floor=0.5 if p == 1 else 0.0)
    # a forward-only step leaves the rows alone
    steps[0].back_rows.fill_(7.0)
    steps[0].run(backward=False)
    torch.cuda.synchronize()
    assert bool((steps[0].back_rows == 7.0).all())
