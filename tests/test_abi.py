"""The C-ABI library loads and exports every symbol include/kge_mi355.h declares (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kge_mi355.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kge_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("kge_residual_fwd", "kge_score_fwd", "kge_inspect", "kge_score_bwd", "kge_build_index"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from cuke_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m cuke_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(handle, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_table_matches_header():
    from cuke_amd import _lib
    assert sorted(_lib.EXPORTS) == declared_symbols()


def test_strerror_and_version_without_gpu():
    from cuke_amd import _lib
    L = _lib.lib()
    assert L.kge_abi_version() == _lib.ABI_VERSION == 7
    assert L.kge_strerror(0) == b"ok"
    assert b"workspace" in L.kge_strerror(-4)


def test_host_side_rejects_cpu_tensors():
    import pytest
    import torch
    from cuke_amd.kge import KGEModel, KgeError
    with pytest.raises(KgeError):
        KGEModel("TransE", torch.zeros(4, 8), torch.zeros(2, 8))
    with pytest.raises(ValueError):
        KGEModel("NoSuchModel", torch.zeros(4, 8), torch.zeros(2, 8))


def test_argument_validation_returns_status_codes_without_touching_the_gpu():
    """Every entry point validates before it launches: wrong arguments come back as status codes
    (the reference raises c10::Error from tensor accessors instead, pycuke1/codegen/cpu.py:9-13).
    The pointers below are never dereferenced on the host and no kernel is launched."""
    import ctypes as C
    from cuke_amd import _lib
    L = _lib.lib()
    EINVAL, ESHAPE, EWORKSPACE = -1, -2, -4
    fake = C.c_void_p(0x1000)  # stands for a device pointer; validation must reject before any use

    def tables(model=0, dim=16, rel_dim=16, n_ent=10, n_rel=3, p=2, ent=fake, rel=fake, aux=None):
        return _lib.Tables(model, p, 0.0, 0, dim, rel_dim, n_ent, n_rel, ent, rel, aux)

    def batch(B=8, h=fake, r=fake, t=fake, neg=None, chunk=0, n_neg=0, mode=0):
        return _lib.Batch(B, h, r, t, neg, chunk, n_neg, None, None, None, mode, 0)

    out = fake
    # null descriptors / tables
    assert L.kge_residual_fwd(None, C.byref(batch()), out, None, 0, None) == EINVAL
    assert L.kge_score_fwd(C.byref(tables(ent=None)), C.byref(batch()), out, None, None, None, None, None, 0,
                           None) == EINVAL
    # unknown model, bad norm order, odd complex dimension, wrong relation width
    assert L.kge_score_fwd(C.byref(tables(model=99)), C.byref(batch()), out, None, None, None, None, None, 0,
                           None) == EINVAL
    assert L.kge_score_fwd(C.byref(tables(p=3)), C.byref(batch()), out, None, None, None, None, None, 0,
                           None) == EINVAL
    assert L.kge_score_fwd(C.byref(tables(model=_lib.MODELS["ComplEx"], dim=15, rel_dim=15)), C.byref(batch()), out,
                           None, None, None, None, None, 0, None) == ESHAPE
    assert L.kge_score_fwd(C.byref(tables(rel_dim=8)), C.byref(batch()), out, None, None, None, None, None, 0,
                           None) == ESHAPE
    # TransH without its normals
    assert L.kge_score_fwd(C.byref(tables(model=_lib.MODELS["TransH"])), C.byref(batch()), out, None, None, None,
                           None, None, 0, None) == EINVAL
    # batch: missing index arrays, batch not a whole number of chunks, unknown negative mode
    assert L.kge_score_fwd(C.byref(tables()), C.byref(batch(h=None)), out, None, None, None, None, None, 0,
                           None) == EINVAL
    assert L.kge_score_fwd(C.byref(tables()), C.byref(batch(B=10, neg=fake, chunk=4, n_neg=2)), out, fake, None,
                           None, None, None, 0, None) == ESHAPE
    assert L.kge_score_fwd(C.byref(tables()), C.byref(batch(neg=fake, chunk=4, n_neg=2, mode=7)), out, fake, None,
                           None, None, None, 0, None) == EINVAL
    # backward: inspections are mandatory
    saved, grads = _lib.Saved(fake, None, None, None, None), _lib.Grads(fake, fake, None)
    assert L.kge_score_bwd(C.byref(tables()), C.byref(batch()), C.byref(saved), fake, None, C.byref(grads), fake,
                           1 << 20, None) == EINVAL
    # inspector: part count, row range, workspace
    assert L.kge_inspect(None, None, 1, 10, None, None, 0, None) == EINVAL
    assert L.kge_inspect_batch(None, 1, None) == EINVAL
    assert L.kge_inspect_workspace(-1, 10) == 0 and L.kge_inspect_workspace(100, 0) == 0
    # loss: workspace too small
    assert L.kge_margin_loss(fake, fake, 8, 4, 1.0, 1.0, fake, None, None, fake, 8, None) == EWORKSPACE
    # build_index / sampler / index check
    assert L.kge_sample_negatives(fake, 10, 0, 1, 0, None) == ESHAPE
    assert L.kge_sample_negatives(None, 10, 5, 1, 0, None) == EINVAL
    assert L.kge_check_indices(fake, 10, 5, None, None) == EINVAL
    # empty work is not an error and launches nothing
    assert L.kge_score_fwd(C.byref(tables()), C.byref(batch(B=0, h=None, r=None, t=None)), None, None, None, None,
                           None, None, 0, None) == 0
    assert L.kge_sample_negatives(None, 0, 5, 1, 0, None) == 0


def test_transr_negatives_backward_requires_the_positive_scores_for_l2():
    """TransR with shared negatives, L2: the per-positive gradient kernel divides by the saved positive scores
    whether or not dpos is given (dpos == NULL means zeros), so a missing kge_saved.pos is an argument error on
    the host, before anything is launched (the pointers below are never dereferenced)."""
    import ctypes as C
    from cuke_amd import _lib
    L = _lib.lib()
    fake = 0x10000
    B, N, d, n_rel = 64, 8, 16, 5
    tab = _lib.Tables(_lib.MODELS["TransR"], 2, 0.0, 0, d, d, 100, n_rel, fake, fake, fake)
    rel = _lib.Inspection(B, n_rel, fake, fake, fake, fake, fake, fake)
    ent = _lib.Inspection(2 * B + (B // 16) * N, 100, fake, fake, fake, fake, fake, fake)
    bat = _lib.Batch(B, fake, fake, fake, fake, 16, N, C.pointer(ent), C.pointer(rel), None, 0, 0)
    fwd_bytes = int(L.kge_score_fwd_workspace(C.byref(tab), C.byref(bat)))
    bwd_bytes = int(L.kge_score_bwd_workspace(C.byref(tab), C.byref(bat)))
    assert fwd_bytes > 0 and bwd_bytes > 0
    grads = _lib.Grads(fake, fake, fake)
    for dpos in (None, fake):
        saved = _lib.Saved(None, fake, None, None, fake, fake, fwd_bytes)   # pos missing, everything else there
        assert L.kge_score_bwd(C.byref(tab), C.byref(bat), C.byref(saved), dpos, fake, C.byref(grads), fake, bwd_bytes,
                               None) == -1


def test_transr_negatives_grouped_path_declines_shapes_whose_worst_case_workspace_is_huge():
    """The grouped shared-negative TransR path sizes its workspaces for min(B, n_rel * n_chunks) groups; above
    its byte cap both size queries answer 0 (and the host scores the pairs as explicit triples) instead of
    asking the caller for tens of gigabytes."""
    import ctypes as C
    from cuke_amd import _lib
    L = _lib.lib()
    fake = 0x10000

    def sizes(B, N, chunk, d, n_rel):
        tab = _lib.Tables(_lib.MODELS["TransR"], 2, 0.0, 0, d, d, 1000, n_rel, fake, fake, fake)
        rel = _lib.Inspection(B, n_rel, fake, fake, fake, fake, fake, fake)
        bat = _lib.Batch(B, fake, fake, fake, fake, chunk, N, None, C.pointer(rel), None, 0, 0)
        return (int(L.kge_score_fwd_workspace(C.byref(tab), C.byref(bat))),
                int(L.kge_score_bwd_workspace(C.byref(tab), C.byref(bat))))

    f, b = sizes(4096, 64, 512, 200, 1345)
    assert 0 < f + b <= 24 << 30
    f_big, b_big = sizes(16384, 1024, 1024, 400, 10000)   # (2 B + B N) * dim floats, four times over: ~100 GB
    assert b_big == 0


def test_fused_inspection_eligibility_is_decided_on_the_host():
    """kge_fused_inspection_ok only reads the descriptors: shared negatives, index sets of at most 65536 ids and
    tables of at most 2^22 rows qualify; larger sets and larger tables do not,
    and asking the score calls for a fused inspection without the jobs is an argument error."""
    import ctypes as C
    from cuke_amd import _lib
    L = _lib.lib()
    fake = 0x10000  # stands for a 16-byte aligned device pointer; nothing is dereferenced or launched

    def jobs(n_ent_ids, n_rel_ids, n_ent_rows, n_rel_rows=100):
        js = (_lib.InspectJob * 2)()
        for j, n, rows in ((js[0], n_ent_ids, n_ent_rows), (js[1], n_rel_ids, n_rel_rows)):
            j.parts[0], j.part_len[0], j.n_parts, j.n_rows = fake, n, 1, rows
            j.out = _lib.Inspection(n, rows, fake, fake, fake, fake, fake, fake)
            j.workspace, j.workspace_bytes = fake, int(L.kge_inspect_workspace(n, rows))
        return js

    def tables(model, dim=16):
        rel_dim = {"RotatE": dim // 2, "RESCAL": 0}.get(model, dim)
        aux = fake if model in ("TransH", "TransR", "RESCAL") else None
        return _lib.Tables(_lib.MODELS[model], 2, 0.0, 0, dim, rel_dim, 1000, 100, fake, fake if rel_dim else None, aux)

    def batch(B=1024, neg=True):
        return _lib.Batch(B, fake, fake, fake, fake if neg else None, 256 if neg else 0, 256 if neg else 0,
                          None, None, None, 0, 0, None)

    ok = lambda model, bat, js: L.kge_fused_inspection_ok(C.byref(tables(model)), C.byref(bat), js)
    assert ok("DistMult", batch(), jobs(3072, 1024, 1000)) == 1
    assert ok("RotatE", batch(), jobs(3072, 1024, 1 << 22)) == 1
    assert ok("TransE", batch(), jobs(3072, 1024, (1 << 22) + 1)) == 0      # needs a third digit pass
    assert ok("TransH", batch(), jobs(65537, 1024, 1000)) == 0              # multi-block sort territory
    assert ok("TransF", batch(), jobs(3072, 1024, 1000)) == 1
    assert ok("DistMult", batch(neg=False), jobs(2048, 1024, 1000)) == 0
    assert ok("TransR", batch(neg=False), jobs(2048, 1024, 1000)) == 0      # no relation groups given
    # the flag without the jobs
    bat = batch()
    bat.fuse_inspection = 1
    assert L.kge_score_fwd(C.byref(tables("DistMult")), C.byref(bat), fake, fake, None, None, None, None, 0, None) == -1


def test_back_rows_are_offered_only_where_the_forward_pass_writes_them():
    """kge_batch.back_rows (the rows phi(residual) Proj^T that spare the backward pass its second read of the
    projections): kge_back_rows_ok says which batches qualify, and the forward call refuses the others before
    it launches anything."""
    import ctypes as C
    from cuke_amd import _lib
    L = _lib.lib()
    EUNSUPPORTED = -5
    fake = C.c_void_p(0x1000)

    def tables(model, dim=200, p=2):
        rel_dim = 0 if model == "RESCAL" else dim
        aux = fake if model in ("TransH", "TransR", "RESCAL") else None
        return _lib.Tables(_lib.MODELS[model], p, 0.0, 0, dim, rel_dim, 1000, 100, fake, fake if rel_dim else None, aux)

    rel = _lib.Inspection(64, 100, fake, fake, fake, fake, fake, fake)

    def batch(neg=False, with_rel=True):
        return _lib.Batch(64, fake, fake, fake, fake if neg else None, 64 if neg else 0, 8 if neg else 0, None,
                          C.pointer(rel) if with_rel else None, None, 0, 0, None)

    ok = lambda model, bat, **kw: L.kge_back_rows_ok(C.byref(tables(model, **kw)), C.byref(bat))
    assert ok("TransR", batch()) == 1
    assert ok("TransR", batch(), p=1) == 1
    assert ok("TransR", batch(), dim=1024) == 1
    assert ok("TransR", batch(), dim=202) == 0          # padded problem: no rows
    assert ok("TransR", batch(), dim=2048) == 0         # outside the grouped kernels
    assert ok("TransR", batch(neg=True)) == 0
    assert ok("TransR", batch(with_rel=False)) == 0
    assert ok("RESCAL", batch()) == 0
    assert ok("TransE", batch()) == 0
    # the forward call refuses a batch that asks for the rows and does not qualify
    bat = batch()
    bat.back_rows = fake
    assert L.kge_score_fwd(C.byref(tables("TransE")), C.byref(bat), fake, None, None, None, None, None, 0, None) == EUNSUPPORTED
    assert L.kge_score_fwd(C.byref(tables("RESCAL")), C.byref(bat), fake, None, None, None, fake, fake, 1 << 20, None) == EUNSUPPORTED
    # and a backward call that is handed rows for such a batch is an error of the caller
    saved = _lib.Saved(fake, None, None, None, fake, None, 0, fake)
    grads = _lib.Grads(fake, fake, fake, None, None, 0, 0)
    ent = _lib.Inspection(128, 1000, fake, fake, fake, fake, fake, fake)
    b2 = batch()
    b2.ent_insp = C.pointer(ent)
    assert L.kge_score_bwd(C.byref(tables("TransR", dim=202)), C.byref(b2), C.byref(saved), fake, None, C.byref(grads),
                           fake, 1 << 30, None) == -1
