"""Pins for the CPU oracle (no GPU).

The reference holds no golden vectors for this path, so the oracle is pinned
against: the generated-code listing for TransE (apps/kge/README.md:37-79),
the eager formulas in apps/kge/test_pytorch.py:21,40,58,74,91 evaluated with
torch library routines in fp64, closed forms and special cases that collapse
one model into another, brute-force flattening for shared negatives,
torch.autograd and finite differences for gradients.
"""
import numpy as np
import pytest
import torch

from cuke_amd import synth

RTOL = 1e-5


def close(a, b, scale=None, rtol=RTOL):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    scale = float(np.max(np.abs(b))) if scale is None else scale
    np.testing.assert_allclose(a, b, rtol=rtol, atol=rtol * max(scale, 1e-30))


def small(model, seed=0, **kw):
    spec = dict(n_ent=97, n_rel=13, dim=24, batch=32, chunk=8, n_neg=5, sigma=0.3, ent_zipf=1.1,
                gamma=3.0)
    spec.update(kw)
    return synth.custom_workload(model, seed=seed, **spec)


def T(x):
    return None if x is None else torch.from_numpy(np.asarray(x)).double()


def torch_score(model, E, R, A, h, r, t, p=2, gamma=0.0):
    """Independent fp64 restatement with torch library ops; t may be [B] or [B, N] ids."""
    eh, rr = E[h], R[r] if R is not None else None
    et = E[t]
    if et.dim() == 3:  # [B, N, d]
        eh = eh[:, None, :]
        rr = rr[:, None, :] if rr is not None else None
    half = E.shape[1] // 2
    if model == "TransE":
        return torch.linalg.vector_norm(eh - et + rr, ord=p, dim=-1)
    if model == "TransH":
        w = A[r]
        w = w[:, None, :] if et.dim() == 3 else w
        d0 = eh - et
        u = d0 + rr - torch.einsum("...a,...a->...", w, d0)[..., None] * w
        return torch.linalg.vector_norm(u, ord=p, dim=-1)
    if model == "TransR":
        M = A[r]
        d0 = eh - et
        if et.dim() == 3:
            u = torch.einsum("bni,bij->bnj", d0, M) + rr
        else:
            u = torch.einsum("ab,abc->ac", d0, M) + rr
        return torch.linalg.vector_norm(u, ord=p, dim=-1)
    if model == "DistMult":
        return (eh * rr * et).sum(-1)
    if model == "ComplEx":
        hc = torch.complex(eh[..., :half], eh[..., half:])
        rc = torch.complex(rr[..., :half], rr[..., half:])
        tc = torch.complex(et[..., :half], et[..., half:])
        return (hc * rc * tc.conj()).real.sum(-1)
    if model == "RotatE":
        hc = torch.complex(eh[..., :half], eh[..., half:])
        tc = torch.complex(et[..., :half], et[..., half:])
        rot = torch.polar(torch.ones_like(rr), rr)
        return gamma - (hc * rot - tc).abs().sum(-1)
    if model == "TransF":
        return ((eh + rr) * et).sum(-1) + ((et - rr) * eh).sum(-1)
    if model == "RESCAL":
        M = A[r]
        if et.dim() == 3:
            return torch.einsum("bj,bnj->bn", torch.einsum("bi,bij->bj", E[h], M), et)
        return torch.einsum("ab,ab->a", torch.einsum("ab,abc->ac", eh, M), et)
    raise KeyError(model)


ALL = ["TransE", "TransH", "TransR", "DistMult", "ComplEx", "RotatE", "TransF", "RESCAL"]


def test_transe_residual_bit_exact_vs_generated_listing(oracle):
    # README.md:65-79: arr[b][j] = ((E[h[b]][j] - E[t[b]][j]) + R[r[b]][j]) in fp32.
    w = synth.make_workload("cfg1_transe")
    a = w.arrays
    got = oracle.residual("TransE", a["E"], a["R"], None, a["h"], a["r"], a["t"])
    want = (a["E"][a["h"]] - a["E"][a["t"]]) + a["R"][a["r"]]
    assert want.dtype == np.float32
    assert np.array_equal(got, want)


@pytest.mark.parametrize("model", ["TransH", "TransR"])
def test_residual_vs_eager_formula_fp64(oracle, model):
    w = small(model)
    a = w.arrays
    got = oracle.residual(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"])
    E, R, A = T(a["E"]), T(a["R"]), T(a["A"])
    h, r, t = (torch.from_numpy(a[k]) for k in "hrt")
    if model == "TransH":  # test_pytorch.py:40
        want = E[h] - E[t] + R[r] - torch.einsum(
            "a,ab->ab", torch.einsum("ab,ab->a", A[r], E[h] - E[t]), A[r])
    else:  # test_pytorch.py:58
        want = torch.einsum("ab,abc->ac", E[h] - E[t], A[r]) + R[r]
    close(got, want.numpy())


@pytest.mark.parametrize("model", ALL)
@pytest.mark.parametrize("p", [1, 2])
def test_scores_vs_torch_fp64(oracle, model, p):
    w = small(model, seed=3)
    a = w.arrays
    pos, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"],
                             w.chunk, p=p, gamma=w.gamma)
    E, R, A = T(a["E"]), T(a["R"]), T(a["A"])
    h, r, t = (torch.from_numpy(a[k]) for k in "hrt")
    neg = torch.from_numpy(a["neg"]).view(w.n_chunks, w.n_neg)
    tneg = neg[torch.arange(w.batch) // w.chunk]  # [B, N]
    close(pos, torch_score(model, E, R, A, h, r, t, p, w.gamma).numpy())
    close(negs, torch_score(model, E, R, A, h, r, tneg, p, w.gamma).numpy())


@pytest.mark.parametrize("model", ALL)
def test_shared_negatives_equal_flattened_triples(oracle, model):
    # A8: out[b][k] = f(E[h[b]], R[r[b]], E[tail[(b / C) * N + k]]) -- brute force over explicit triples
    w = small(model, seed=5)
    a = w.arrays
    _, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                           gamma=w.gamma)
    B, N, C = w.batch, w.n_neg, w.chunk
    fh = np.repeat(a["h"], N)
    fr = np.repeat(a["r"], N)
    ft = np.array([a["neg"][(b // C) * N + k] for b in range(B) for k in range(N)])
    flat, _ = oracle.score(model, a["E"], a["R"], a["A"], fh, fr, ft, gamma=w.gamma)
    assert np.array_equal(negs.reshape(-1), flat)


@pytest.mark.parametrize("model", ALL)
def test_head_mode_negatives_equal_flattened_triples(oracle, model):
    # negatives that replace the head: out[b][k] = f(E[neg[(b / C) * N + k]], R[r[b]], E[t[b]]),
    # scores and sparse gradients, against the positive-only oracle on the explicit triples
    w = small(model, seed=6)
    a = w.arrays
    B, N, C = w.batch, w.n_neg, w.chunk
    _, negs = oracle.score(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], C, gamma=w.gamma,
                           neg_mode="head")
    fh = np.array([a["neg"][(b // C) * N + k] for b in range(B) for k in range(N)])
    fr, ft = np.repeat(a["r"], N), np.repeat(a["t"], N)
    flat, _ = oracle.score(model, a["E"], a["R"], a["A"], fh, fr, ft, gamma=w.gamma)
    assert np.array_equal(negs.reshape(-1), flat)

    rng = np.random.default_rng(0)
    dpos = rng.standard_normal(B).astype(np.float32)
    dneg = rng.standard_normal((B, N)).astype(np.float32)
    g = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], C, dpos, dneg,
                        neg_mode="head")
    gp = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], dpos=dpos)
    gn = oracle.backward(model, a["E"], a["R"], a["A"], fh, fr, ft, dpos=dneg.reshape(-1))

    def dense(ids, rows, n):
        out = np.zeros((n,) + rows.shape[1:], np.float64)
        out[ids] = rows
        return out
    close(dense(g.ent_ids, g.ent_rows, w.n_ent),
          dense(gp.ent_ids, gp.ent_rows, w.n_ent) + dense(gn.ent_ids, gn.ent_rows, w.n_ent))
    if g.rel_rows is not None:
        close(dense(g.rel_ids, g.rel_rows, w.n_rel),
              dense(gp.rel_ids, gp.rel_rows, w.n_rel) + dense(gn.rel_ids, gn.rel_rows, w.n_rel))
    if g.aux_rows is not None:
        close(dense(g.rel_ids, g.aux_rows, w.n_rel),
              dense(gp.rel_ids, gp.aux_rows, w.n_rel) + dense(gn.rel_ids, gn.aux_rows, w.n_rel))


def test_reference_view_layout_is_the_special_case_neg_equals_tails(oracle):
    # examples.py:1404-1444: with N == C and neg == t every positive is scored against the
    # tails of its own chunk: out[b][k] = E[h[b]] - E[t[(b / bs) * bs + k]] + R[r[b]]
    w = small("TransE", chunk=8, n_neg=8)
    a = w.arrays
    _, negs = oracle.score("TransE", a["E"], a["R"], None, a["h"], a["r"], a["t"], a["t"], 8, p=1)
    for b in (0, 7, 8, 31):
        for k in (0, 3, 7):
            u = (a["E"][a["h"][b]] - a["E"][a["t"][(b // 8) * 8 + k]]) + a["R"][a["r"][b]]
            close(negs[b, k], np.abs(u.astype(np.float64)).sum())


def test_special_cases_collapse(oracle):
    w = small("TransH", seed=7)
    a = w.arrays
    args = (a["h"], a["r"], a["t"], a["neg"], w.chunk)
    te = oracle.score("TransE", a["E"], a["R"], None, *args)
    # zero normals: TransH == TransE (bit exact: the projection term is exactly 0)
    th = oracle.score("TransH", a["E"], a["R"], np.zeros_like(a["A"]), *args)
    assert np.array_equal(te[0], th[0]) and np.array_equal(te[1], th[1])
    # identity projections: TransR == TransE
    eye = np.broadcast_to(np.eye(w.dim, dtype=np.float32), (w.n_rel, w.dim, w.dim)).copy()
    tr = oracle.score("TransR", a["E"], a["R"], eye, *args)
    close(tr[0], te[0]); close(tr[1], te[1])
    # zero imaginary parts: ComplEx == DistMult on the real halves
    half = w.dim // 2
    E0, R0 = a["E"].copy(), a["R"].copy()
    E0[:, half:] = 0; R0[:, half:] = 0
    cx = oracle.score("ComplEx", E0, R0, None, *args)
    dm = oracle.score("DistMult", E0[:, :half].copy(), R0[:, :half].copy(), None, *args)
    close(cx[0], dm[0]); close(cx[1], dm[1])
    # zero phases: RotatE == gamma - sum of complex moduli of h - t
    ro = oracle.score("RotatE", a["E"], np.zeros((w.n_rel, half), np.float32), None, *args, gamma=2.5)
    dd = a["E"][a["h"]].astype(np.float64) - a["E"][a["t"]]
    close(ro[0], 2.5 - np.hypot(dd[:, :half], dd[:, half:]).sum(1))
    # quarter-turn phases rotate (re, im) -> (-im, re)
    rq = oracle.score("RotatE", a["E"], np.full((w.n_rel, half), np.pi / 2, np.float32), None, *args)
    eh = a["E"][a["h"]].astype(np.float64); et = a["E"][a["t"]].astype(np.float64)
    close(rq[0], -np.hypot(-eh[:, half:] - et[:, :half], eh[:, :half] - et[:, half:]).sum(1))


def dense_from_sparse(ids, rows, n):
    out = np.zeros((n,) + rows.shape[1:], np.float64)
    out[ids] = rows
    return out


@pytest.mark.parametrize("model", ALL)
@pytest.mark.parametrize("p", [1, 2])
def test_gradients_vs_autograd_fp64(oracle, model, p):
    if p == 1 and model not in ("TransE", "TransH", "TransR"):
        pytest.skip("norm order only matters for the translation models")
    w = small(model, seed=11)
    a = w.arrays
    rng = np.random.default_rng(1)
    dpos = rng.standard_normal(w.batch).astype(np.float32)
    dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32)
    g = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                        dpos, dneg, p=p)
    E = T(a["E"]).requires_grad_()
    R = T(a["R"]).requires_grad_() if a["R"] is not None and a["R"].size else None
    A = T(a["A"]).requires_grad_() if a["A"] is not None else None
    h, r, t = (torch.from_numpy(a[k]) for k in "hrt")
    neg = torch.from_numpy(a["neg"]).view(w.n_chunks, w.n_neg)
    tneg = neg[torch.arange(w.batch) // w.chunk]
    L = (torch_score(model, E, R, A, h, r, t, p, w.gamma) * T(dpos)).sum() + \
        (torch_score(model, E, R, A, h, r, tneg, p, w.gamma) * T(dneg)).sum()
    L.backward()
    # ids: strictly ascending, exactly the rows that occur
    occ = np.unique(np.concatenate([a["h"], a["t"], a["neg"]]))
    assert np.array_equal(g.ent_ids, occ)
    assert np.array_equal(g.rel_ids, np.unique(a["r"]))
    tol = 2e-5 if p == 1 else 2e-5
    close(dense_from_sparse(g.ent_ids, g.ent_rows, w.n_ent), E.grad.numpy(), rtol=tol)
    if R is not None and model != "RESCAL":
        close(dense_from_sparse(g.rel_ids, g.rel_rows, w.n_rel), R.grad.numpy(), rtol=tol)
    if A is not None:
        close(dense_from_sparse(g.rel_ids, g.aux_rows, w.n_rel),
              A.grad.numpy().reshape(w.n_rel, -1), rtol=tol)


@pytest.mark.parametrize("model", ["TransH", "RotatE", "ComplEx", "TransR"])
def test_gradient_finite_difference_tiny(oracle, model):
    # central differences in fp64 through the oracle's own forward (fp32 storage, so the
    # step is large and the tolerance loose); catches a sign or index slip in bwd_one.
    w = small(model, seed=2, n_ent=9, n_rel=3, dim=6, batch=4, chunk=2, n_neg=2, norm_p=2)
    a = w.arrays
    dpos = np.ones(w.batch, np.float32)
    dneg = np.full((w.batch, w.n_neg), 0.5, np.float32)
    g = oracle.backward(model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                        dpos, dneg, p=2)

    def loss(E):
        pos, negs = oracle.score(model, E, a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                                 p=2, gamma=w.gamma)
        return float(pos.astype(np.float64).sum() + 0.5 * negs.astype(np.float64).sum())

    eps = 1e-2
    dense = dense_from_sparse(g.ent_ids, g.ent_rows, w.n_ent)
    for row in g.ent_ids[:3]:
        for col in range(w.dim):
            Ep, Em = a["E"].copy(), a["E"].copy()
            Ep[row, col] += eps; Em[row, col] -= eps
            fd = (loss(Ep) - loss(Em)) / (2 * eps)
            assert abs(fd - dense[row, col]) < 5e-2 * max(1.0, abs(fd)), (row, col, fd, dense[row, col])


def test_margin_loss_vs_torch(oracle):
    rng = np.random.default_rng(0)
    pos = rng.standard_normal(64).astype(np.float32)
    neg = rng.standard_normal((64, 9)).astype(np.float32)
    for sign in (1.0, -1.0):
        loss, dpos, dneg = oracle.margin_loss(pos, neg, 0.7, sign)
        tp = T(pos).requires_grad_(); tn = T(neg).requires_grad_()
        y = torch.full((64, 9), sign, dtype=torch.float64)
        want = torch.nn.functional.margin_ranking_loss(tp[:, None].expand(64, 9), tn, y, margin=0.7)
        want.backward()
        close(loss, want.item())
        close(dpos, tp.grad.numpy()); close(dneg, tn.grad.numpy())


def brute_inspect(idx):
    idx = [int(x) for x in idx]
    uniq = sorted(set(idx))
    perm = sorted(range(len(idx)), key=lambda i: (idx[i], i))
    seg = [0]
    for u in uniq:
        seg.append(seg[-1] + sum(1 for x in idx if x == u))
    inv = [uniq.index(x) for x in idx]
    return uniq, seg, perm, inv


@pytest.mark.parametrize("case", ["empty", "one", "all_equal", "all_distinct", "zipf", "uniform"])
def test_inspector_oracle_vs_brute_force(oracle, case):
    rng = np.random.default_rng(4)
    idx = {
        "empty": np.zeros(0, np.int64),
        "one": np.array([5], np.int64),
        "all_equal": np.full(37, 3, np.int64),
        "all_distinct": rng.permutation(64).astype(np.int64),
        "zipf": synth.zipf_indices(rng, 50, 64, 1.1),
        "uniform": rng.integers(0, 20, 61),
    }[case]
    ins = oracle.inspect(idx)
    uniq, seg, perm, inv = brute_inspect(idx)
    assert ins.unique_ids.tolist() == uniq
    assert ins.seg_offsets.tolist() == seg
    assert ins.perm.tolist() == perm
    assert ins.inverse.tolist() == inv
    assert np.array_equal(ins.unique_ids[ins.inverse], idx)


def test_build_index_properties(oracle):
    # properties of the reference's chunk-of-16 inspector (inspector.cu:68-136) on sorted input
    rng = np.random.default_rng(9)
    rel_num = 7
    r = np.sort(rng.integers(0, rel_num, 16 * 40)).astype(np.int64)
    uniq, buf, cnt, undefined = oracle.build_index(r, rel_num)
    assert not undefined
    r2 = r.reshape(-1, 16)
    for blk in range(r2.shape[0]):
        vals, counts = np.unique(r2[blk], return_counts=True)
        assert cnt[blk] in (0, 1, 2)
        for i in range(16):
            if buf[blk, i] < 16:
                assert uniq[blk, buf[blk, i]] == r2[blk, i]
            else:
                assert buf[blk, i] - 16 == r2[blk, i]
        if counts.max() >= 2:
            assert counts[list(vals).index(uniq[blk, 0])] == counts.max()
        assert all(u == rel_num for u in uniq[blk, cnt[blk]:])


def test_build_index_exhaustive_three_values(oracle):
    # every chunk made of <= 3 distinct values with all run-length splits
    rows = []
    for n0 in range(0, 17):
        for n1 in range(0, 17 - n0):
            rows.append([0] * n0 + [1] * n1 + [2] * (16 - n0 - n1))
    r = np.array(rows, np.int64).reshape(-1)
    uniq, buf, cnt, undefined = oracle.build_index(r, 5)
    assert not undefined
    for blk, row in enumerate(rows):
        vals, counts = np.unique(row, return_counts=True)
        multi = sorted([c for c in counts if c >= 2], reverse=True)
        assert cnt[blk] == min(2, len(multi))
        cached = [uniq[blk, s] for s in range(cnt[blk])]
        for i, v in enumerate(row):
            assert (buf[blk, i] < 16 and cached[buf[blk, i]] == v) or buf[blk, i] == v + 16
        if multi:
            assert counts[list(vals).index(cached[0])] == multi[0]


def lockstep_build_index(chunk, rel_num):
    """The reference's build_index kernel (apps/kge/inspection/inspector.cu:39-136) executed as written:
    sixteen threads in lockstep, one numpy array per __shared__ array, every statement applied to all
    threads at once (reads before writes, as the lanes of a wavefront execute it).  A restatement at the
    thread level, independent of the oracle's sequential one.  Returns (uniq[16], buf[16], cnt) or None
    where the kernel writes out of bounds (16 distinct values)."""
    C_, T_ = 16, 2
    tid = np.arange(C_)
    idx = np.array(chunk, dtype=np.int64)
    ord_uniq, pcount = tid.copy(), np.zeros(C_, np.int64)
    count, idx_count = np.full(C_, -1, np.int64), np.full(C_, -1, np.int64)
    # bitonic_sort(idx, ord): inspector.cu:39-66
    arr, sord = idx.copy(), tid.copy()
    k = 2
    while k <= C_:
        j = k >> 1
        while j > 0:
            ixj = tid ^ j
            a_old, o_old = arr.copy(), sord.copy()
            for t in range(C_):
                x = ixj[t]
                if x > t:
                    up = (t & k) == 0
                    if (up and a_old[t] > a_old[x]) or (not up and a_old[t] < a_old[x]):
                        arr[t], arr[x], sord[t], sord[x] = a_old[x], a_old[t], o_old[x], o_old[t]
            j >>= 1
        k <<= 1
    idx = arr
    ord_ = np.empty(C_, np.int64)
    ord_[sord] = tid
    # head flags and their inclusive scan: inspector.cu:80-88
    ibuf = np.where((tid > 0) & (idx > np.roll(idx, 1)), 1, 0).astype(np.int64)
    ibuf[0] = 0
    offset = 1
    while offset < C_:
        old = ibuf.copy()
        ibuf[offset:] = old[offset:] + old[:-offset]
        offset *= 2
    # run starts: inspector.cu:90-94
    if ibuf[C_ - 1] + 1 >= C_:
        return None  # pcount[16] = C: out of bounds
    pcount[ibuf[C_ - 1] + 1] = C_
    for t in range(1, C_):
        if idx[t] > idx[t - 1]:
            pcount[ibuf[t]] = t
    iuniq = np.full(C_, rel_num, np.int64)
    # run lengths and the tournament for the two longest: inspector.cu:97-113
    old_p = pcount.copy()
    for t in range(1, C_):
        if old_p[t] - old_p[t - 1] > 0:
            count[t - 1] = old_p[t] - old_p[t - 1]
            idx_count[t - 1] = old_p[t] - 1
    sdist = C_ // 2
    while sdist > 0:
        c_old, i_old, o_old = count.copy(), idx_count.copy(), ord_uniq.copy()
        for t in range(sdist):
            if c_old[t] < c_old[t + sdist]:
                count[t], count[t + sdist] = c_old[t + sdist], c_old[t]
                idx_count[t], idx_count[t + sdist] = i_old[t + sdist], i_old[t]
                ord_uniq[t], ord_uniq[t + sdist] = o_old[t + sdist], o_old[t]
        sdist >>= 1
    if count[1] < count[2]:
        count[1], count[2] = count[2], count[1]
        idx_count[1], idx_count[2] = idx_count[2], idx_count[1]
        ord_uniq[1], ord_uniq[2] = ord_uniq[2], ord_uniq[1]
    # cache slots for runs of at least T: inspector.cu:117-119
    for t in range(T_):
        if count[t] > T_ - 1:
            iuniq[t] = idx[idx_count[t]]
    # slot or id + C per element: inspector.cu:121-133
    new_ibuf = ibuf.copy()
    for t in range(C_):
        if ibuf[t] == ord_uniq[0] and iuniq[0] < rel_num:
            new_ibuf[t] = 0
        elif ibuf[t] == ord_uniq[1] and iuniq[1] < rel_num:
            new_ibuf[t] = 1
        else:
            new_ibuf[t] = idx[t] + C_
    cnt = 0
    for t in range(C_ - 1):
        if iuniq[t] < rel_num and iuniq[t + 1] == rel_num:
            cnt = t + 1
    return iuniq, new_ibuf[ord_], cnt


def test_build_index_equals_the_kernel_run_in_lockstep(oracle):
    """Chunks with 1 to 15 distinct values, sorted (the reference's use) and unsorted, random run lengths and
    ties between run lengths: the oracle's sequential restatement against the thread-level one."""
    rng = np.random.default_rng(21)
    rel_num = 40
    chunks = []
    for distinct in range(1, 16):
        for rep in range(40):
            vals = rng.choice(rel_num, distinct, replace=False)
            row = np.concatenate([vals, rng.choice(vals, 16 - distinct)])
            chunks.append(np.sort(row) if rep % 2 == 0 else rng.permutation(row))
    r = np.concatenate(chunks).astype(np.int64)
    uniq, buf, cnt, undefined = oracle.build_index(r, rel_num)
    assert not undefined
    for b, chunk in enumerate(chunks):
        want = lockstep_build_index(chunk, rel_num)
        assert want is not None
        assert uniq[b].tolist() == want[0].tolist(), (b, chunk.tolist())
        assert buf[b].tolist() == want[1].tolist(), (b, chunk.tolist())
        assert cnt[b] == want[2], (b, chunk.tolist())


def test_build_index_flags_sixteen_distinct(oracle):
    r = np.arange(16, dtype=np.int64)
    *_, undefined = oracle.build_index(r, 100)
    assert undefined


def test_sparse_optimizer_steps_vs_numpy(oracle):
    rng = np.random.default_rng(12)
    table = rng.standard_normal((50, 12)).astype(np.float32)
    state = rng.random(50).astype(np.float32)
    ids = np.sort(rng.choice(50, 17, replace=False)).astype(np.int64)
    rows = rng.standard_normal((17, 12)).astype(np.float32)
    want = table.astype(np.float64).copy(); want[ids] -= 0.1 * rows
    close(oracle.sparse_sgd(table, ids, rows, 0.1), want)
    st = state.astype(np.float64).copy(); st[ids] += (rows.astype(np.float64) ** 2).mean(1)
    want = table.astype(np.float64).copy(); want[ids] -= 0.1 * rows / (np.sqrt(st[ids])[:, None] + 1e-10)
    got_t, got_s = oracle.sparse_adagrad(table, state, ids, rows, 0.1)
    close(got_s, st); close(got_t, want)
    untouched = np.setdiff1d(np.arange(50), ids)
    assert np.array_equal(got_t[untouched], table[untouched])


def test_openmp_build_of_the_oracle_gives_the_checkers_results(oracle):
    """The OpenMP build (the timed multi-thread leg, and the checker of the full-size config-5 test) is the
    same source: every score comes from the same serial loop, so scores are bit-identical; gradient rows
    differ only in the order the per-thread double accumulators are added."""
    for model, p in (("TransH", 1), ("DistMult", 2), ("RotatE", 2), ("TransR", 2)):
        kw = dict(chunk=32, n_neg=24) if model != "TransR" else {}
        w = synth.custom_workload(model, n_ent=300, n_rel=7, dim=24, batch=96, norm_p=p, sigma=0.2, gamma=3.0,
                                  ent_zipf=1.1, seed=2, **kw)
        a = w.arrays
        args = (model, a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a.get("neg"), w.chunk)
        pos0, neg0 = oracle.score(*args, p=p, gamma=w.gamma)
        pos1, neg1 = oracle.score(*args, p=p, gamma=w.gamma, fast="omp")
        assert np.array_equal(pos0, pos1) and (neg0 is None or np.array_equal(neg0, neg1))
        rng = np.random.default_rng(1)
        dpos = rng.standard_normal(w.batch).astype(np.float32)
        dneg = rng.standard_normal((w.batch, w.n_neg)).astype(np.float32) if w.chunk else None
        g0 = oracle.backward(*args, dpos, dneg, p=p)
        g1 = oracle.backward(*args, dpos, dneg, p=p, fast="omp")
        for x, y in ((g0.ent_rows, g1.ent_rows), (g0.rel_rows, g1.rel_rows), (g0.aux_rows, g1.aux_rows)):
            if x is not None:
                assert np.allclose(x, y, rtol=1e-6, atol=1e-9)


def test_l1_ambiguity_mask_vs_numpy(oracle):
    """l1_ambiguous_rows counts, per row, exactly the residual elements with |u| <= eps of the triples and pairs
    that touch the row (brute force in numpy; eps chosen large enough that a fraction of the rows is marked)."""
    w = synth.custom_workload("TransH", n_ent=60, n_rel=5, dim=8, batch=24, chunk=12, n_neg=6, norm_p=1, sigma=0.2,
                              seed=4)
    a = w.arrays
    eps = 2e-3
    fe, fr, n = oracle.l1_ambiguous_rows("TransH", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                                         eps=eps)
    ue, ur = np.unique(np.concatenate([a["h"], a["t"], a["neg"]])), np.unique(a["r"])
    we, wr, total = np.zeros(ue.size, np.int64), np.zeros(ur.size, np.int64), 0
    for b in range(w.batch):
        tails = [a["t"][b]] + list(a["neg"][(b // w.chunk) * w.n_neg:(b // w.chunk + 1) * w.n_neg])
        for tl in tails:
            u = oracle.residual("TransH", a["E"], a["R"], a["A"], a["h"][b:b + 1], a["r"][b:b + 1], np.array([tl]))[0]
            k = int((np.abs(u) <= np.float32(eps)).sum())
            if k:
                total += k
                for e in (a["h"][b], tl):
                    we[np.searchsorted(ue, e)] += k
                wr[np.searchsorted(ur, a["r"][b])] += k
    assert n == total and 0 < (we > 0).sum() < we.size
    assert np.array_equal(fe, we) and np.array_equal(fr, wr)
    fe2, fr2, n2 = oracle.l1_ambiguous_rows("TransH", a["E"], a["R"], a["A"], a["h"], a["r"], a["t"], a["neg"], w.chunk,
                                            eps=eps, fast="omp")
    assert n2 == n and np.array_equal(fe2, fe) and np.array_equal(fr2, fr), "the OpenMP build counts the same"
