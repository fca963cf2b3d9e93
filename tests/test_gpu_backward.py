"""Backward parity: sparse row gradients from the HIP path against the CPU oracle."""
import numpy as np
import pytest
import torch

from cuke_amd import synth
from helpers import assert_close, compare_l1_generic, gpu_model

pytestmark = pytest.mark.gpu

NEG_MODELS = ["TransE", "TransH", "DistMult", "ComplEx", "RotatE", "TransF"]


def run_both(oracle, w, seed=0, use_pos=True, use_neg=True, pair_sums="matrix_cores", fast=False, neg_mode="tail"):
    a = w.arrays
    rng = np.random.default_rng(seed)
    dpos = rng.standard_normal(w.batch).astype(np.float32) if use_pos else None
    has_neg = "neg" in a
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32) if (has_neg and use_neg) else None
    m, ix = gpu_model(w)
    m.pair_sums = pair_sums
    fw = m.score(ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, neg_mode=neg_mode)
    dev = fw.pos.device
    g = m.backward(fw, None if dpos is None else torch.from_numpy(dpos).to(dev),
                   None if dneg is None else torch.from_numpy(dneg).to(dev))
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a.get("neg"), w.chunk,
                          dpos, dneg, p=w.norm_p, fast=fast, neg_mode=neg_mode)
    return g, ref


def compare(g, ref, what, outliers=None):
    assert np.array_equal(g.ent_ids.cpu().numpy(), ref.ent_ids), what
    assert np.array_equal(g.rel_ids.cpu().numpy(), ref.rel_ids), what
    assert_close(g.ent_rows.cpu().numpy(), ref.ent_rows, what=f"{what} entity rows", rows=True,
                 outliers=outliers)
    if ref.rel_rows is not None and ref.rel_rows.size:
        assert_close(g.rel_rows.cpu().numpy(), ref.rel_rows, what=f"{what} relation rows", rows=True)
    if ref.aux_rows is not None:
        assert_close(g.aux_rows.cpu().numpy(), ref.aux_rows, what=f"{what} aux rows", rows=True)


@pytest.mark.parametrize("model", NEG_MODELS)
@pytest.mark.parametrize("shape", [
    dict(dim=24, batch=96, chunk=24, n_neg=40),
    dict(dim=22, batch=64, chunk=64, n_neg=7),
    dict(dim=200, batch=256, chunk=128, n_neg=130),
])
@pytest.mark.parametrize("p", [1, 2])
def test_shared_negative_gradients(oracle, model, shape, p):
    if p == 1 and model not in ("TransE", "TransH"):
        pytest.skip("norm order only matters for the translation models")
    # L1 gradients are sums of signs: on generic floats a residual element within an ulp of zero
    # may take either sign depending on summation order, so the L1 cases run on lattice-valued
    # tables where every residual is exact (synth.make_tables) and no sign is ambiguous.
    w = synth.custom_workload(model, n_ent=150, n_rel=11, norm_p=p, sigma=0.2, gamma=4.0, ent_zipf=1.1,
                              seed=shape["dim"] + p, lattice=(p == 1), **shape)
    g, ref = run_both(oracle, w, seed=1)
    compare(g, ref, f"{model} {shape} p={p}")


@pytest.mark.parametrize("model", NEG_MODELS)
def test_positive_only_gradients(oracle, model):
    w = synth.custom_workload(model, n_ent=300, n_rel=9, dim=64, batch=333, sigma=0.2, gamma=4.0,
                              ent_zipf=1.2, seed=3)
    g, ref = run_both(oracle, w, seed=2)
    compare(g, ref, f"{model} positives only")


@pytest.mark.parametrize("model,p,dim", [("TransE", 1, 72), ("TransH", 2, 80), ("TransH", 1, 76), ("RotatE", 2, 152)])
def test_row_widths_that_end_in_a_narrow_column_tile(oracle, model, p, dim):
    """Batches large enough for the 64-owner gradient tiles whose row width leaves 1..16 columns over the
    64-column tiles (72 = 64 + 8, 80 = 64 + 16, 76 = 64 + 12, RotatE 76 complex elements): those columns are
    computed by the narrow tiles, every other column by the wide ones."""
    w = synth.custom_workload(model, n_ent=3000, n_rel=11, dim=dim, batch=128 * 256, chunk=128, n_neg=128, norm_p=p,
                              sigma=0.2, gamma=4.0, ent_zipf=1.1, seed=dim + p, lattice=(p == 1))
    g, ref = run_both(oracle, w, seed=5, fast="omp")
    compare(g, ref, f"{model} p={p} dim={dim}", outliers=(1e-5, 4.0) if model == "RotatE" else None)


@pytest.mark.parametrize("model,p,pair_sums", [
    ("TransE", 1, None), ("TransE", 2, None), ("TransH", 1, None), ("TransH", 2, None), ("RotatE", 2, None),
    ("DistMult", 2, "vector_alus"), ("ComplEx", 2, "vector_alus"), ("TransF", 2, "vector_alus")])
@pytest.mark.parametrize("shape", [
    dict(dim=520, batch=96 * 8, chunk=96, n_neg=72),    # three looper steps either way
    dict(dim=132, batch=40 * 24, chunk=40, n_neg=200),  # seven steps over the negatives, two over the positives
    dict(dim=130, batch=64 * 32, chunk=64, n_neg=33),   # rows that are not 16-byte multiples
])
@pytest.mark.parametrize("mode", ["tail", "head"])
def test_batches_of_a_few_hundred_tiles_in_both_negative_modes(oracle, model, p, pair_sums, shape, mode):
    """Batches between 128 and 511 64-owner tiles (the vector-ALU gradient tiles then own 16 rows each and a CU holds a
    few of them), looper counts that are no multiples of the 32-row step, corrupted tails and corrupted heads."""
    klen = shape["dim"] // 2 if model == "RotatE" else shape["dim"]
    big = -(-klen // 64) * (-(-shape["chunk"] // 64) + -(-shape["n_neg"] // 64)) * (shape["batch"] // shape["chunk"])
    assert 128 <= big < 512, "this shape is meant for the 16-owner tiles"
    w = synth.custom_workload(model, n_ent=500, n_rel=11, norm_p=p, sigma=0.2, gamma=4.0, ent_zipf=1.1,
                              seed=shape["dim"] + p, lattice=(p == 1), **shape)
    g, ref = run_both(oracle, w, seed=9, pair_sums=pair_sums or "matrix_cores", neg_mode=mode, fast="omp")
    compare(g, ref, f"{model} {shape} p={p} {mode}", outliers=(1e-5, 4.0) if model == "RotatE" else None)


def test_missing_upstream_gradients_mean_zero(oracle):
    w = synth.custom_workload("DistMult", n_ent=200, n_rel=7, dim=32, batch=64, chunk=32, n_neg=16,
                              sigma=0.2, seed=5)
    g, ref = run_both(oracle, w, use_pos=False)
    compare(g, ref, "dpos omitted")
    g, ref = run_both(oracle, w, use_neg=False)
    compare(g, ref, "dneg omitted")


def test_hot_rows_long_segments(oracle):
    # a handful of entities: every segment spans many 32-position blocks of the reduction
    w = synth.custom_workload("TransE", n_ent=5, n_rel=3, dim=64, batch=512, chunk=128, n_neg=128,
                              sigma=0.3, seed=6, norm_p=1, lattice=True)
    g, ref = run_both(oracle, w, seed=4)
    compare(g, ref, "hot rows")


@pytest.mark.parametrize("name,over", [
    ("cfg2_distmult", dict(n_ent=100_000, batch=1024)),
    ("cfg2_complex", dict(n_ent=100_000, batch=1024)),
    ("cfg4_rotate", dict(batch=512)),
    ("cfg5_transh", dict(n_ent=200_000, batch=2048, lattice=True)),
])
def test_scaled_configs_gradients(oracle, name, over):
    w = synth.make_workload(name, **over)
    g, ref = run_both(oracle, w, seed=7)
    compare(g, ref, name, outliers=(1e-5, 4.0) if w.model == "RotatE" else None)


def test_margin_loss_step_rotate(oracle):
    # forward -> margin-ranking loss -> backward, the cfg 4 pipeline at reduced batch
    from cuke_amd.kge import margin_loss
    w = synth.make_workload("cfg4_rotate", batch=512)
    a = w.arrays
    m, ix = gpu_model(w)
    fw = m.score(ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    loss, dpos, dneg = margin_loss(fw.pos, fw.neg, w.margin, 1.0)
    g = m.backward(fw, dpos, dneg)
    pos, negs = oracle.score(w.model, a["E"], a["R"], None, a["h"], a["r"], a["t"], a["neg"], w.chunk,
                             gamma=w.gamma)
    rl, rdp, rdn = oracle.margin_loss(pos, negs, w.margin, 1.0)
    assert_close(loss.cpu().numpy(), np.array([rl], np.float32), what="loss")
    # use the GPU's own activity mask for the reference gradient: a pair whose hinge argument
    # is within rounding of zero may legitimately flip between the two implementations
    ref = oracle.backward(w.model, a["E"], a["R"], None, a["h"], a["r"], a["t"], a["neg"], w.chunk,
                          dpos.cpu().numpy(), dneg.cpu().numpy())
    compare(g, ref, "rotate margin step", outliers=(1e-5, 4.0))
    flips = int((dneg.cpu().numpy() != rdn).sum())
    assert flips <= 1e-4 * rdn.size


def test_transh_l1_generic_floats_differ_only_by_sign_flips(oracle):
    w = synth.make_workload("cfg5_transh", n_ent=200_000, batch=1024)
    g, ref = run_both(oracle, w, seed=9)
    rng = np.random.default_rng(9)  # the upstream gradients run_both drew
    dmax = max(np.abs(rng.standard_normal(w.batch)).max(), np.abs(rng.standard_normal((w.batch, w.n_neg))).max())
    masked, n_amb = compare_l1_generic(oracle, w, w.arrays, g, ref, float(dmax), "cfg5 scaled, generic floats")
    assert n_amb > 0, "at this size some residual element is expected within 6e-8 of zero"


@pytest.mark.parametrize("name,over", [
    ("cfg2_distmult", dict(n_ent=50_000, batch=512)),
    ("cfg4_rotate", dict(batch=256)),
    ("cfg3_transr", dict(batch=1024)),
])
def test_train_step_eager_overlapped_and_graph_replays(oracle, name, over):
    """The preallocated step: plain order, inspector overlapped on a side stream, inspector fused into
    the score kernels' launches, and HIP-graph replays (several, with eager work and synchronisation in
    between) all give the oracle's gradients."""
    from cuke_amd.kge import TrainStep
    w = synth.make_workload(name, **over)
    a = w.arrays
    m, ix = gpu_model(w)
    sign = -1.0 if w.model == "TransR" else 1.0
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, loss=w.loss,
                     margin=w.margin, sign=sign)

    def reference():
        dpos, dneg = step.dpos.cpu().numpy(), (step.dneg.cpu().numpy() if step.dneg is not None else None)
        return oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a.get("neg"), w.chunk,
                               dpos, dneg, p=w.norm_p)

    def check(tag):
        torch.cuda.synchronize()
        ref = reference()
        compare(step.sparse_grads(), ref, f"{name} {tag}", outliers=(1e-5, 4.0) if w.model == "RotatE" else None)
        step.ent_rows.zero_()  # eager work between runs; also proves the next run rewrites everything

    step.run(overlap=False, fused=False)
    check("in order")
    step.run(overlap=True, fused=False)
    check("overlapped")
    assert step.fusable
    step.run()  # inspection fused into the score kernels' launches where the batch qualifies
    check("fused" if step.fusable else "default")
    other = torch.cuda.Stream()  # a caller's own stream: the step follows torch's current stream
    other.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(other):
        step.run(overlap=True, fused=False)
        step.run()
    check("on a second stream")
    step.capture()
    for i in range(3):
        step.replay()
        check(f"graph replay {i}")


@pytest.mark.parametrize("name,over", [
    ("cfg2_distmult", dict(n_ent=50_000, batch=512)),
    ("cfg4_rotate", dict(batch=256)),
    ("cfg3_transr", dict(batch=1024)),
    # L1 norm: lattice-valued tables keep every residual element away from the sign ambiguity at zero
    ("cfg5_transh", dict(n_ent=20_000, batch=512, n_neg=64, chunk=64, lattice=True)),
])
@pytest.mark.parametrize("ahead", [0, 1])
def test_train_step_pipelined_inspections(oracle, name, over, ahead):
    """run(pipeline=True): index tensors and inspections live in a ring of sets, so the inspector of a
    batch overlaps the steps before it.  Six steps are enqueued without any synchronisation, each on new
    indices that a loader stream writes into next_inputs() and hands over with stage() -- `ahead` batches
    before the step that consumes them -- and each step's gradients are copied out on the main stream.
    After one synchronisation at the end every step must match the oracle on its own batch."""
    from cuke_amd.kge import SparseGrads, TrainStep
    w = synth.make_workload(name, **over)
    a = w.arrays
    m, ix = gpu_model(w)
    sign = -1.0 if w.model in ("TransR", "TransH") else 1.0
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix.get("neg"), w.chunk or None, loss=w.loss,
                     margin=w.margin, sign=sign)
    rng = np.random.default_rng(11)
    loader = torch.cuda.Stream()
    n_steps = 6
    batches, staged_host, kept = [], [], []

    def hand_over(i):
        new = {k: rng.integers(0, w.n_rel if k == "r" else w.n_ent, size=a[k].shape).astype(np.int64)
               for k in ("h", "r", "t", "neg") if a.get(k) is not None}
        if i == 3:  # a batch with heavy repetition: few distinct rows
            new = {k: v % 7 for k, v in new.items()}
        host = {k: torch.from_numpy(v).pin_memory() for k, v in new.items()}
        with torch.cuda.stream(loader):
            bufs = dict(zip(("h", "r", "t", "neg"), step.next_inputs(loader)))
            for k, v in host.items():
                bufs[k].copy_(v, non_blocking=True)
            ready = torch.cuda.Event()
            ready.record(loader)
        step.stage(ready)
        batches.append(new)
        staged_host.append(host)  # pinned buffers stay alive until the copies have run

    for i in range(ahead):
        hand_over(i)
    for i in range(n_steps):
        if i + ahead < n_steps:
            hand_over(i + ahead)
        step.run(pipeline=True)
        ins_e, ins_r = step.ent_insp, step.rel_insp
        kept.append(dict(ne=ins_e.num_unique_dev.clone(), nr=ins_r.num_unique_dev.clone(),
                         eid=ins_e.unique_ids.clone(), rid=ins_r.unique_ids.clone(), erows=step.ent_rows.clone(),
                         rrows=step.rel_rows.clone() if step.rel_rows is not None else None,
                         arows=step.aux_rows.clone() if step.aux_rows is not None else None,
                         dpos=step.dpos.clone(), dneg=step.dneg.clone() if step.dneg is not None else None))
    torch.cuda.synchronize()
    for i, (new, k) in enumerate(zip(batches, kept)):
        ref = oracle.backward(w.model, a["E"], a["R"], a["A"], new["h"], new["r"], new["t"], new.get("neg"), w.chunk,
                              k["dpos"].cpu().numpy(), k["dneg"].cpu().numpy() if k["dneg"] is not None else None,
                              p=w.norm_p)
        ue, ur = int(k["ne"]), int(k["nr"])
        got = SparseGrads(k["eid"][:ue], k["erows"][:ue], k["rid"][:ur],
                          k["rrows"][:ur] if k["rrows"] is not None else None,
                          k["arows"][:ur] if k["arows"] is not None else None)
        compare(got, ref, f"{name} pipelined step {i}", outliers=(1e-5, 4.0) if w.model == "RotatE" else None)
    # the plain mode still works afterwards, on the set of the step run last
    step.run(fused=False)
    torch.cuda.synchronize()
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], batches[-1]["h"], batches[-1]["r"], batches[-1]["t"],
                          batches[-1].get("neg"), w.chunk, step.dpos.cpu().numpy(),
                          step.dneg.cpu().numpy() if step.dneg is not None else None, p=w.norm_p)
    compare(step.sparse_grads(), ref, f"{name} plain run after the pipelined ones",
            outliers=(1e-5, 4.0) if w.model == "RotatE" else None)


@pytest.mark.parametrize("model,p", [("DistMult", 2), ("ComplEx", 2), ("TransE", 1), ("TransH", 2), ("RotatE", 2)])
@pytest.mark.parametrize("shape", [
    dict(n_ent=50, n_rel=3, dim=24, batch=96, chunk=24, n_neg=40),              # one digit pass for both tables
    dict(n_ent=70_000, n_rel=300, dim=32, batch=1100, chunk=100, n_neg=37),     # ragged block edges, two passes
    dict(n_ent=3_000_000, n_rel=5000, dim=16, batch=4096, chunk=512, n_neg=512),  # 22-bit ids, several workgroups
])
@pytest.mark.parametrize("neg_mode", ["tail", "head"])
def test_fused_inspection_matches_the_separate_inspector(oracle, model, p, shape, neg_mode):
    """run(fused=True): the inspector's workgroups ride in the score kernels' launches.  Its outputs must
    be bit-identical to the stand-alone inspector's, and the gradients must match the oracle."""
    from cuke_amd.kge import TrainStep, inspect
    w = synth.custom_workload(model, norm_p=p, sigma=0.2, gamma=4.0, ent_zipf=1.1, seed=7, lattice=(p == 1), **shape)
    a = w.arrays
    m, ix = gpu_model(w)
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk, neg_mode=neg_mode)
    assert step.fusable
    step.run(fused=True)
    torch.cuda.synchronize()
    want_e = inspect([ix["h"], ix["t"], ix["neg"]], w.n_ent)
    want_r = inspect([ix["r"]], w.n_rel)
    for got, want, what in ((step.ent_insp, want_e, "entities"), (step.rel_insp, want_r, "relations")):
        u = want.num_unique
        assert got.num_unique == u, what
        for f in ("unique_ids", "seg_offsets"):
            assert torch.equal(getattr(got, f)[:u + (f == "seg_offsets")], getattr(want, f)[:u + (f == "seg_offsets")]), (what, f)
        for f in ("perm", "inverse", "sorted_seg"):
            assert torch.equal(getattr(got, f), getattr(want, f)), (what, f)
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                          step.dpos.cpu().numpy(), step.dneg.cpu().numpy(), p=p, neg_mode=neg_mode)
    compare(step.sparse_grads(), ref, f"{model} fused {neg_mode}", outliers=(1e-5, 4.0) if model == "RotatE" else None)


def test_train_step_falls_back_to_the_stream_inspector_for_large_index_sets(oracle):
    """More than 65536 ids in concat(h, t, neg): the batch does not qualify for the fused inspection, the
    default run() uses the multi-block inspector on the side stream, and asking for fused=True is an error."""
    from cuke_amd import KgeError
    from cuke_amd.kge import TrainStep
    w = synth.custom_workload("DistMult", n_ent=5000, n_rel=40, dim=8, batch=32768, chunk=4096, n_neg=512,
                              sigma=0.2, ent_zipf=1.1, seed=2)
    a = w.arrays
    m, ix = gpu_model(w)
    step = TrainStep(m, ix["h"], ix["r"], ix["t"], ix["neg"], w.chunk)
    assert step.n_occ > 65536 and not step.fusable
    with pytest.raises(KgeError):
        step.run(fused=True)
    step.run()
    torch.cuda.synchronize()
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                          step.dpos.cpu().numpy(), step.dneg.cpu().numpy())
    compare(step.sparse_grads(), ref, "large index set, stream inspector")


@pytest.mark.parametrize("model", ["TransR", "RESCAL"])
@pytest.mark.parametrize("shape", [
    dict(n_ent=900, n_rel=37, dim=32, batch=3001),        # ragged last workgroup, two digit passes
    dict(n_ent=60, n_rel=5, dim=16, batch=700),           # one digit pass: finished by the scatter step
    dict(n_ent=2_000_000, n_rel=700, dim=8, batch=20000),  # 21-bit ids, 40 inspector workgroups
])
def test_fused_entity_inspection_with_the_grouped_projection_kernels(oracle, model, shape):
    """TransR / RESCAL: the relation inspection runs first, the entity inspection rides with the forward GEMM,
    prep, dX GEMM and dM kernels.  Bit-identical to the stand-alone inspector; gradients vs the oracle."""
    from cuke_amd.kge import TrainStep, inspect
    w = synth.custom_workload(model, norm_p=2, sigma=0.2, rel_zipf=1.1, seed=5, **shape)
    a = w.arrays
    m, ix = gpu_model(w)
    step = TrainStep(m, ix["h"], ix["r"], ix["t"])
    assert step.fusable
    step.run(fused=True)
    torch.cuda.synchronize()
    want = inspect([ix["h"], ix["t"]], w.n_ent)
    got, u = step.ent_insp, want.num_unique
    assert got.num_unique == u
    assert torch.equal(got.unique_ids[:u], want.unique_ids[:u]) and torch.equal(got.seg_offsets[:u + 1], want.seg_offsets[:u + 1])
    for f in ("perm", "inverse", "sorted_seg"):
        assert torch.equal(getattr(got, f), getattr(want, f)), f
    ref = oracle.backward(w.model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], None, 0,
                          step.dpos.cpu().numpy(), None, p=2)
    compare(step.sparse_grads(), ref, f"{model} fused entity inspection")


@pytest.mark.parametrize("model", ["DistMult", "ComplEx"])
def test_pair_sums_on_matrix_cores_and_on_vector_alus_agree(oracle, model):
    """kge_tables.flags (KGEModel.pair_sums) switches the DistMult / ComplEx tile kernels between the fp32
    matrix-core form (default) and the vector-ALU form per call: both must meet the oracle's tolerance."""
    w = synth.custom_workload(model, n_ent=400, n_rel=9, dim=72, batch=320, chunk=160, n_neg=130, sigma=0.2,
                              ent_zipf=1.1, seed=4)
    for unit in ("matrix_cores", "vector_alus"):
        g, ref = run_both(oracle, w, seed=3, pair_sums=unit)
        compare(g, ref, f"{model} pair sums on the {unit}")


@pytest.mark.parametrize("name,over", [("cfg2_distmult", dict(n_ent=50_000, batch=512)), ("cfg3_transr", dict(batch=1024)),
                                       ("cfg4_rotate", dict(batch=256))])
def test_staged_issue_as_two_branch_graphs(oracle, name, over):
    """capture_staged(i, i + 1): the step of batch i and, on a second branch of the same HIP graph, the inspection
    of batch i + 1.  The graphs are replayed in a ring several times with eager work and synchronisation between
    the replays; every replay must reproduce the oracle's gradients of its own batch."""
    from cuke_amd.kge import TrainStep
    ws = [synth.make_workload(name, seed=s, **over) for s in range(3)]
    m, ix0 = gpu_model(ws[0])
    w = ws[0]
    sign = -1.0 if w.model in ("TransR", "TransH") else 1.0
    step = TrainStep(m, ix0["h"], ix0["r"], ix0["t"], ix0.get("neg"), w.chunk or None, loss=w.loss, margin=w.margin, sign=sign)
    for o in ws[1:]:
        ix = {k: torch.from_numpy(o.arrays[k]).cuda() for k in ("h", "r", "t", "neg") if o.arrays.get(k) is not None}
        step.add_batch(ix["h"], ix["r"], ix["t"], ix.get("neg"))
    graphs = [step.capture_staged(i, (i + 1) % 3) for i in range(3)]
    a0 = ws[0].arrays
    for rep in range(7):
        i = rep % 3
        step.ent_rows.zero_()                      # eager work between the replays
        graphs[i].replay()
        step.use_batch(i)
        torch.cuda.synchronize()
        a = ws[i].arrays
        ref = oracle.backward(w.model, a0["E"], a0["R"], a0["A"], a["h"], a["r"], a["t"], a.get("neg"), w.chunk,
                              step.dpos.cpu().numpy(), step.dneg.cpu().numpy() if step.dneg is not None else None, p=w.norm_p)
        compare(step.sparse_grads(), ref, f"{name} staged graph replay {rep}",
                outliers=(1e-5, 4.0) if w.model == "RotatE" else None)
