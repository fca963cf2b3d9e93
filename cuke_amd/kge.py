"""Host side of the KGE score path: the reference's operator surface over the HIP library.

The reference exposes each score function as a generated module whose single
``run`` takes positional sizes, embedding tensors and index tensors
(apps/kge/test_cuke.py:54,104,153,198,244) and returns a tensor; its inspector
is ``inspector(r, rel_num)`` (apps/kge/kge.py:249-271).  ``transE`` ... ``RESCAL``
and ``inspector`` below keep those names, argument orders and outputs.  On top of
that :class:`KGEModel` offers what a training step needs and the reference does
not have: scalar scores, shared negatives, and sparse row gradients.

torch is used for device memory and streams only; every computation is a kernel
of libkge_mi355.so reached through the C ABI.
"""
from __future__ import annotations

import collections
import ctypes as C
from dataclasses import dataclass

import torch

from . import _lib
from ._lib import KgeError, MODELS

__all__ = ["KGEModel", "TrainStep", "Inspection", "Forward", "SparseGrads", "inspect", "inspector", "transE",
           "transH", "transR", "transF", "RESCAL", "margin_loss", "sparse_sgd", "sparse_adagrad",
           "sparse_sgd_factored", "sparse_adagrad_factored", "KgeError"]


NEG_MODES = {"tail": 0, "head": 1}  # KGE_NEG_TAIL / KGE_NEG_HEAD


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_stream_objects: dict = {}


def _stream() -> C.c_void_p:
    if _raw_stream is not None:
        return C.c_void_p(_raw_stream(torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _current_stream(dev_index: int):
    """``torch.cuda.current_stream()`` of a loop that asks every step: the raw handle is one C call,
    and the Stream object that belongs to a handle is looked up once (torch's streams live in a pool
    for the life of the process; ``current_stream()`` itself costs about 8 us of host time)."""
    if _raw_stream is None:
        return torch.cuda.current_stream(dev_index)
    key = (dev_index, _raw_stream(dev_index))
    st = _stream_objects.get(key)
    if st is None:
        st = _stream_objects[key] = torch.cuda.current_stream(dev_index)
    return st


def _ptr(t: torch.Tensor | None) -> C.c_void_p | None:
    return None if t is None else C.c_void_p(t.data_ptr())


def _table(x, name: str, ndim: int) -> torch.Tensor:
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not x.is_cuda:
        raise KgeError(f"{name} must live on the GPU (got {x.device}); there is no CPU path")
    if x.dtype != torch.float32:
        raise TypeError(f"{name} must be float32 (got {x.dtype})")
    if x.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dimensions (got {x.dim()})")
    return x.contiguous()


def _index(x, name: str, device) -> torch.Tensor:
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if x.dtype not in (torch.int64, torch.int32):
        raise TypeError(f"{name} must be int64 or int32 (got {x.dtype})")
    if x.dim() != 1:
        raise ValueError(f"{name} must be one-dimensional")
    return x.to(device=device, dtype=torch.int64).contiguous()


@dataclass
class Inspection:
    """Sorted / deduplicated view of an index multiset (see kge_inspection in the C header)."""
    n: int
    n_rows: int
    num_unique_dev: torch.Tensor  # int32[1]
    unique_ids: torch.Tensor      # int64[n], first U valid
    seg_offsets: torch.Tensor     # int32[n+1], first U+1 valid
    perm: torch.Tensor            # int32[n]
    inverse: torch.Tensor         # int32[n]
    sorted_seg: torch.Tensor      # int32[n]
    _c: _lib.Inspection = None
    _u: int | None = None

    @property
    def num_unique(self) -> int:
        """U (copies one int from the device the first time it is asked for)."""
        if self._u is None:
            self._u = int(self.num_unique_dev.item())
        return self._u

    def ids(self) -> torch.Tensor:
        return self.unique_ids[: self.num_unique]

    def offsets(self) -> torch.Tensor:
        return self.seg_offsets[: self.num_unique + 1]


def inspect(parts, n_rows: int) -> Inspection:
    """Radix-sort and dedup the concatenation of up to four int64 index tensors."""
    if isinstance(parts, torch.Tensor):
        parts = [parts]
    if not 1 <= len(parts) <= 4:
        raise ValueError("inspect takes one to four index tensors")
    dev = parts[0].device
    parts = [_index(p, f"parts[{i}]", dev) for i, p in enumerate(parts)]
    if not parts[0].is_cuda:
        raise KgeError("inspect needs GPU tensors; there is no CPU path")
    n = sum(int(p.numel()) for p in parts)
    L = _lib.lib()
    i32 = dict(dtype=torch.int32, device=dev)
    ins = Inspection(n, int(n_rows), torch.zeros(1, **i32),
                     torch.empty(max(n, 1), dtype=torch.int64, device=dev),
                     torch.empty(n + 1, **i32), torch.empty(max(n, 1), **i32),
                     torch.empty(max(n, 1), **i32), torch.empty(max(n, 1), **i32))
    ins._c = _lib.Inspection(n, int(n_rows), ins.num_unique_dev.data_ptr(),
                             ins.unique_ids.data_ptr(), ins.seg_offsets.data_ptr(),
                             ins.perm.data_ptr(), ins.inverse.data_ptr(), ins.sorted_seg.data_ptr())
    ws_bytes = int(L.kge_inspect_workspace(n, int(n_rows)))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    ptrs = (C.c_void_p * len(parts))(*[p.data_ptr() for p in parts])
    lens = (C.c_int64 * len(parts))(*[int(p.numel()) for p in parts])
    _lib.check(L.kge_inspect(ptrs, lens, len(parts), int(n_rows), C.byref(ins._c),
                             _ptr(ws), ws_bytes, _stream()), "kge_inspect")
    ins._keep = (parts, ws)
    return ins


@dataclass
class Forward:
    """Scores plus what backward needs from the forward pass."""
    pos: torch.Tensor | None
    neg: torch.Tensor | None
    side_pos: torch.Tensor | None = None
    side_neg: torch.Tensor | None = None
    residual: torch.Tensor | None = None
    flat_pos: torch.Tensor | None = None   # projection models scored through flattened triples: all scores
    fwd_ws: torch.Tensor | None = None     # forward workspace that backward reads again (TransR with negatives)
    back_rows: torch.Tensor | None = None  # TransR: phi(residual) Proj^T rows written by the forward pass (for_backward)
    batch: tuple = ()
    neg_mode: str = "tail"
    ent_insp: Inspection | None = None
    rel_insp: Inspection | None = None


@dataclass
class SparseGrads:
    """One gradient row per distinct table row that occurs in the batch; ids ascending."""
    ent_ids: torch.Tensor
    ent_rows: torch.Tensor
    rel_ids: torch.Tensor
    rel_rows: torch.Tensor | None
    aux_rows: torch.Tensor | None
    # TransR / RESCAL with factor_max > 0 (kge_grads.aux_x / aux_q): the projection gradient of a relation
    # group of at most factor_max triples is sum_p aux_x[p]^T aux_q[p] over its sorted positions
    # p in [rel_seg_offsets[u], rel_seg_offsets[u + 1]) and its aux_rows[u] is not written
    aux_x: torch.Tensor | None = None
    aux_q: torch.Tensor | None = None
    factor_max: int = 0
    rel_seg_offsets: torch.Tensor | None = None
    _c: object = None          # the kge_grads struct these arrays were written through
    _rel_insp: object = None


class KGEModel:
    """A KGE model = its name plus its embedding tables; methods score and differentiate batches.

    model  one of TransE, TransH, TransR, DistMult, ComplEx, RotatE, TransF, RESCAL
    Eemb   [n_ent, dim] float32 (ComplEx / RotatE rows are [re | im])
    Remb   [n_rel, dim] float32 (RotatE: [n_rel, dim/2] phases; RESCAL: None)
    aux    TransH: hyperplane normals [n_rel, dim] (the reference's Pemb);
           TransR / RESCAL: projections [n_rel, dim, dim] (the reference's Proj)
    pair_sums  "matrix_cores" (default) or "vector_alus": where the shared-negative tile kernels of
           DistMult / ComplEx sum their pair products (``pair_sums`` can be reassigned between calls)
    """

    def __init__(self, model: str, Eemb, Remb=None, aux=None, norm_p: int = 2, gamma: float = 0.0,
                 pair_sums: str = "matrix_cores"):
        if model not in MODELS:
            raise ValueError(f"unknown model {model!r}; expected one of {sorted(MODELS)}")
        self.model = model
        self.E = _table(Eemb, "Eemb", 2)
        self.dev = self.E.device
        self.dim = int(self.E.shape[1])
        self.R = None if Remb is None else _table(Remb, "Remb", 2)
        self.A = None
        if model == "TransH":
            self.A = _table(aux, "aux (hyperplane normals)", 2)
        elif model in ("TransR", "RESCAL"):
            self.A = _table(aux, "aux (projection matrices)", 3)
        self.rel_dim = {"RotatE": self.dim // 2, "RESCAL": 0}.get(model, self.dim)
        if self.rel_dim and self.R is None:
            raise ValueError(f"{model} needs a relation table")
        if self.R is not None and self.rel_dim and int(self.R.shape[1]) != self.rel_dim:
            raise ValueError(f"Remb has row width {self.R.shape[1]}, {model} needs {self.rel_dim}")
        self.n_rel = int(self.R.shape[0]) if self.R is not None and self.rel_dim else \
            (int(self.A.shape[0]) if self.A is not None else 0)
        if self.A is not None:
            want = (self.n_rel, self.dim) if model == "TransH" else (self.n_rel, self.dim, self.dim)
            if tuple(self.A.shape) != want:
                raise ValueError(f"aux has shape {tuple(self.A.shape)}, {model} needs {want}")
        self.norm_p, self.gamma = int(norm_p), float(gamma)
        if pair_sums not in ("matrix_cores", "vector_alus"):
            raise ValueError("pair_sums is 'matrix_cores' or 'vector_alus'")
        self._tab = _lib.Tables(MODELS[model], self.norm_p, self.gamma,
                                _lib.PAIR_SUMS_VALU if pair_sums == "vector_alus" else 0, self.dim, self.rel_dim,
                                int(self.E.shape[0]), self.n_rel, self.E.data_ptr(),
                                self.R.data_ptr() if (self.R is not None and self.rel_dim) else None,
                                self.A.data_ptr() if self.A is not None else None)

    @property
    def pair_sums(self) -> str:
        return "vector_alus" if self._tab.flags & _lib.PAIR_SUMS_VALU else "matrix_cores"

    @pair_sums.setter
    def pair_sums(self, unit: str) -> None:
        if unit not in ("matrix_cores", "vector_alus"):
            raise ValueError("pair_sums is 'matrix_cores' or 'vector_alus'")
        self._tab.flags = _lib.PAIR_SUMS_VALU if unit == "vector_alus" else 0

    # -- helpers ---------------------------------------------------------------------------
    def _batch(self, h, r, t, neg=None, chunk=None, ent_insp=None, rel_insp=None, neg_mode="tail"):
        if neg_mode not in NEG_MODES:
            raise ValueError("neg_mode is 'tail' or 'head'")
        h, r, t = (_index(x, n, self.dev) for x, n in ((h, "h"), (r, "r"), (t, "t")))
        B = int(h.numel())
        if int(r.numel()) != B or int(t.numel()) != B:
            raise ValueError("h, r, t must have the same length")
        C_, N = 0, 0
        if neg is not None:
            neg = _index(neg.reshape(-1), "neg", self.dev)
            C_ = int(chunk) if chunk else B
            if C_ <= 0 or B % C_ != 0:
                raise ValueError(f"batch {B} is not a whole number of chunks of {C_}")
            n_chunks = B // C_
            if n_chunks == 0 or int(neg.numel()) % n_chunks != 0:
                raise ValueError("neg must hold the same number of tails for every chunk")
            N = int(neg.numel()) // n_chunks
        bat = _lib.Batch(B, h.data_ptr(), r.data_ptr(), t.data_ptr(),
                         neg.data_ptr() if neg is not None else None, C_, N,
                         C.pointer(ent_insp._c) if ent_insp is not None else None,
                         C.pointer(rel_insp._c) if rel_insp is not None else None, None, NEG_MODES[neg_mode], 0)
        return bat, (h, r, t, neg, C_, N)

    # -- reference-shaped output -------------------------------------------------------------
    def residual(self, h, r, t, rel_insp: Inspection | None = None) -> torch.Tensor:
        """[B, dim] residual vector: the reference's output for TransE / TransH / TransR."""
        bat, keep = self._batch(h, r, t, rel_insp=rel_insp)
        out = torch.empty((bat.batch, self.dim), dtype=torch.float32, device=self.dev)
        ws, nb = self._fwd_workspace(bat)
        _lib.check(_lib.lib().kge_residual_fwd(C.byref(self._tab), C.byref(bat), _ptr(out), _ptr(ws), nb,
                                               _stream()), "kge_residual_fwd")
        return out

    def _grouped_negatives_fit(self, bat) -> bool:
        """TransR with shared negatives: True if the grouped path takes this shape (its worst-case workspaces stay
        under the library's byte cap); the size query of the backward workspace answers 0 otherwise."""
        return int(_lib.lib().kge_score_bwd_workspace(C.byref(self._tab), C.byref(bat))) > 0

    def _fwd_workspace(self, bat):
        nb = int(_lib.lib().kge_score_fwd_workspace(C.byref(self._tab), C.byref(bat)))
        return torch.empty(max(nb, 1), dtype=torch.uint8, device=self.dev), nb

    # -- scalar scores ---------------------------------------------------------------------
    def score(self, h, r, t, neg=None, chunk=None, ent_insp=None, rel_insp=None, neg_mode="tail",
              for_backward: bool = False) -> Forward:
        """pos[B] and, with shared negatives, neg[B, N] scores.

        ``for_backward`` (TransR without negatives, relation inspection given, dim % 4 == 0): the forward kernel
        also forms the rows phi(residual) Proj^T while it holds the projections (``Forward.back_rows``), and
        ``backward()`` then reads no projection again.

        ``neg_mode='tail'``: neg[b, k] scores (h_b, r_b, neg_k), the reference's shared-negative layout
        (apps/examples/examples.py:1404-1444); ``'head'``: (neg_k, r_b, t_b), the head-corrupted batches of
        the reference's sampler (apps/kge/data/sampler.py:287-353)."""
        if neg is not None and self.model == "RESCAL":
            # a dot-product tile over B projected rows: (E[h] Proj[r]) . E[t'] for replaced tails,
            # E[h'] . (Proj[r] E[t]) for replaced heads; shapes outside the grouped kernels: the pairs as
            # explicit triples
            if self.dim % 4 != 0 or self.dim > 1024:
                return self._score_projected_negatives(h, r, t, neg, chunk, neg_mode)
            if rel_insp is None:
                rel_insp = inspect([_index(r, "r", self.dev)], self.n_rel)
        if neg is not None and self.model == "TransR":
            # every negative is projected once per (relation, chunk) group of the batch; needs the
            # relation groups.  Shapes outside the grouped kernels (dim % 4, dim > 1024) take the
            # flattened triples instead.
            if rel_insp is None:
                rel_insp = inspect([_index(r, "r", self.dev)], self.n_rel)
            if self.dim % 4 != 0 or self.dim > 1024:
                return self._score_projected_negatives(h, r, t, neg, chunk, neg_mode)
        bat, keep = self._batch(h, r, t, neg, chunk, ent_insp, rel_insp, neg_mode)
        if neg is not None and self.model == "TransR" and not self._grouped_negatives_fit(bat):
            # the grouped path sizes its workspaces for the worst case min(B, n_rel * n_chunks) groups; above
            # its byte cap the pairs are scored as explicit triples
            return self._score_projected_negatives(h, r, t, neg, chunk, neg_mode)
        B, N = bat.batch, bat.n_neg
        f32 = dict(dtype=torch.float32, device=self.dev)
        fw = Forward(torch.empty(B, **f32), torch.empty((B, N), **f32) if neg is not None else None,
                     batch=keep, ent_insp=ent_insp, rel_insp=rel_insp, neg_mode=neg_mode)
        if self.model == "TransH" or (self.model == "TransF" and neg is not None):
            fw.side_pos = torch.empty(B, **f32)
            if neg is not None and self.model == "TransH":
                fw.side_neg = torch.empty((2, B, N), **f32)
        if self.model in ("TransR", "RESCAL", "RotatE"):
            fw.residual = torch.empty((B, self.dim), **f32)
        if for_backward and B > 0 and _lib.lib().kge_back_rows_ok(C.byref(self._tab), C.byref(bat)):
            fw.back_rows = torch.empty((B, self.dim), **f32)
            bat.back_rows = fw.back_rows.data_ptr()
        ws, nb = self._fwd_workspace(bat)
        _lib.check(_lib.lib().kge_score_fwd(C.byref(self._tab), C.byref(bat), _ptr(fw.pos),
                                            _ptr(fw.neg), _ptr(fw.side_pos), _ptr(fw.side_neg),
                                            _ptr(fw.residual), _ptr(ws), nb, _stream()), "kge_score_fwd")
        if neg is not None and self.model == "TransR":
            fw.fwd_ws = ws  # group list and projected rows, read again by backward
        return fw

    def _score_projected_negatives(self, h, r, t, neg, chunk, neg_mode="tail") -> Forward:
        """TransR / RESCAL with shared negatives: the projection depends on the positive's relation,
        so (as in the reference's neg_transR, examples.py:1447-1480) the B x N pairs are written out
        as explicit triples behind the B positives and scored by the grouped per-relation kernels."""
        bat, (h, r, t, neg, C_, N) = self._batch(h, r, t, neg, chunk, neg_mode=neg_mode)
        B = bat.batch
        total = B * (1 + N)
        flat = [torch.empty(total, dtype=torch.int64, device=self.dev) for _ in range(3)]
        _lib.check(_lib.lib().kge_flatten_negatives(C.byref(bat), *[_ptr(x) for x in flat], _stream()),
                   "kge_flatten_negatives")
        hf, rf, tf = flat
        fw = self.score(hf, rf, tf, rel_insp=inspect([rf], self.n_rel))
        fw.flat_pos = fw.pos
        fw.neg = fw.pos[B:].view(B, N)
        fw.pos = fw.pos[:B]
        return fw

    def inspect_batch(self, h, r, t, neg=None):
        """Inspections of concat(h, t, neg) over the entity table and of r over the relations."""
        parts = [h, t] + ([neg.reshape(-1)] if neg is not None else [])
        return inspect(parts, int(self.E.shape[0])), inspect([r], max(self.n_rel, 1))

    # -- gradients ---------------------------------------------------------------------------
    def backward(self, fw: Forward, dpos=None, dneg=None, factor_max: int = 0) -> SparseGrads:
        """Sparse row gradients of sum(dpos * pos) + sum(dneg * neg).

        ``factor_max`` (TransR / RESCAL without negatives, 0..4): relation groups of at most that many
        triples leave their projection gradient factored (``SparseGrads.aux_x`` / ``aux_q``) instead of
        writing a dense dim x dim matrix; ``sparse_sgd_factored`` / ``sparse_adagrad_factored`` apply it."""
        if getattr(fw, "flat_pos", None) is not None:  # TransR / RESCAL negatives: one flat batch
            B, N = fw.neg.shape
            f32 = dict(dtype=torch.float32, device=self.dev)
            g = torch.zeros(B * (1 + N), **f32)
            if dpos is not None:
                g[:B] = dpos.to(**f32)
            if dneg is not None:
                g[B:] = dneg.to(**f32).reshape(-1)
            flat = Forward(fw.flat_pos, None, residual=fw.residual, batch=fw.batch, ent_insp=fw.ent_insp,
                           rel_insp=fw.rel_insp, fwd_ws=fw.fwd_ws)
            return self.backward(flat, g)
        h, r, t, neg, C_, N = fw.batch
        if fw.ent_insp is None or fw.rel_insp is None:
            e_insp, r_insp = self.inspect_batch(h, r, t, neg)
            fw.ent_insp = fw.ent_insp if fw.ent_insp is not None else e_insp
            fw.rel_insp = fw.rel_insp if fw.rel_insp is not None else r_insp  # (the forward pass may have planned from it)
        bat, _ = self._batch(h, r, t, neg, C_ or None, fw.ent_insp, fw.rel_insp, fw.neg_mode)
        B = bat.batch
        f32 = dict(dtype=torch.float32, device=self.dev)
        if dpos is not None:
            dpos = dpos.to(**f32).contiguous()
        if dneg is not None:
            dneg = dneg.to(**f32).contiguous()
        saved = _lib.Saved(*[(x.data_ptr() if x is not None else None) for x in
                             (fw.pos, fw.neg, fw.side_pos, fw.side_neg, fw.residual)])
        if fw.fwd_ws is not None:
            saved.fwd_workspace, saved.fwd_workspace_bytes = fw.fwd_ws.data_ptr(), int(fw.fwd_ws.numel())
        if fw.back_rows is not None:
            saved.back_rows = fw.back_rows.data_ptr()
        ent_rows = torch.empty((fw.ent_insp.n, self.dim), **f32)
        rel_rows = torch.empty((B, self.rel_dim), **f32) if self.rel_dim else None
        aux_rows = None
        if self.model == "TransH":
            aux_rows = torch.empty((B, self.dim), **f32)
        elif self.model in ("TransR", "RESCAL"):
            aux_rows = torch.empty((min(B, self.n_rel), self.dim * self.dim), **f32)
        aux_x = aux_q = None
        if factor_max:
            if self.model not in ("TransR", "RESCAL") or neg is not None:
                raise ValueError("factor_max applies to TransR / RESCAL without shared negatives")
            aux_x, aux_q = torch.empty((B, self.dim), **f32), torch.empty((B, self.dim), **f32)
        grads = _lib.Grads(_ptr(ent_rows), _ptr(rel_rows), _ptr(aux_rows), _ptr(aux_x), _ptr(aux_q), int(factor_max), 0)
        L = _lib.lib()
        ws_bytes = int(L.kge_score_bwd_workspace(C.byref(self._tab), C.byref(bat)))
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=self.dev)
        _lib.check(L.kge_score_bwd(C.byref(self._tab), C.byref(bat), C.byref(saved), _ptr(dpos),
                                   _ptr(dneg), C.byref(grads), _ptr(ws), ws_bytes, _stream()),
                   "kge_score_bwd")
        ue, ur = fw.ent_insp.num_unique, fw.rel_insp.num_unique
        return SparseGrads(fw.ent_insp.ids(), ent_rows[:ue], fw.rel_insp.ids(),
                           rel_rows[:ur] if rel_rows is not None else None,
                           aux_rows[:ur] if aux_rows is not None else None,
                           aux_x, aux_q, int(factor_max), fw.rel_insp.offsets() if factor_max else None,
                           grads, fw.rel_insp)


def margin_loss(pos: torch.Tensor, neg: torch.Tensor, margin: float, sign: float = 1.0):
    """mean_{b,k} max(0, margin - sign * (pos[b] - neg[b, k])) and its gradients (loss, dpos, dneg)."""
    B, N = neg.shape
    L = _lib.lib()
    loss = torch.empty(1, dtype=torch.float32, device=pos.device)
    dpos, dneg = torch.empty_like(pos), torch.empty_like(neg)
    ws_bytes = int(L.kge_margin_loss_workspace(B, N))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=pos.device)
    _lib.check(L.kge_margin_loss(_ptr(pos), _ptr(neg), B, N, float(margin), float(sign), _ptr(loss),
                                 _ptr(dpos), _ptr(dneg), _ptr(ws), ws_bytes, _stream()),
               "kge_margin_loss")
    return loss, dpos, dneg


def _inplace_table(table):
    """A table that is updated in place must be the caller's own memory, not a contiguous copy of it."""
    t = _table(table, "table", table.dim())
    if t.data_ptr() != table.data_ptr() or not table.is_contiguous():
        raise ValueError("table must be contiguous: it is updated in place")
    return t


def sparse_sgd(table: torch.Tensor, insp: Inspection, rows: torch.Tensor, lr: float) -> None:
    """table[id] -= lr * rows[u] for the inspection's unique ids (in place, no host sync)."""
    t = _inplace_table(table)
    _lib.check(_lib.lib().kge_sparse_sgd(_ptr(t), int(rows.shape[1]), _ptr(insp.unique_ids), _ptr(insp.num_unique_dev),
                                         int(rows.shape[0]), _ptr(rows), float(lr), _stream()), "kge_sparse_sgd")


def sparse_adagrad(table: torch.Tensor, state: torch.Tensor, insp: Inspection, rows: torch.Tensor, lr: float,
                   eps: float = 1e-10) -> None:
    """Row-wise Adagrad: state[id] += mean(g^2); table[id] -= lr * g / (sqrt(state[id]) + eps)."""
    t = _inplace_table(table)
    if not state.is_contiguous():
        raise ValueError("state must be contiguous: it is updated in place")
    _lib.check(_lib.lib().kge_sparse_adagrad(_ptr(t), _ptr(state), int(rows.shape[1]), _ptr(insp.unique_ids),
                                             _ptr(insp.num_unique_dev), int(rows.shape[0]), _ptr(rows), float(lr),
                                             float(eps), _stream()), "kge_sparse_adagrad")


def sparse_sgd_factored(proj: torch.Tensor, g: SparseGrads, lr: float) -> None:
    """Proj[id] -= lr * dM for the projection gradients of ``KGEModel.backward(..., factor_max=m)`` /
    ``TrainStep(..., factor_max=m)``: dense groups from ``aux_rows``, factored groups straight from their rows."""
    t = _inplace_table(proj)
    _lib.check(_lib.lib().kge_sparse_sgd_factored(_ptr(t), int(proj.shape[1]), C.byref(g._rel_insp._c), C.byref(g._c),
                                                  float(lr), _stream()), "kge_sparse_sgd_factored")


def sparse_adagrad_factored(proj: torch.Tensor, state: torch.Tensor, g: SparseGrads, lr: float, eps: float = 1e-10) -> None:
    """Row-wise Adagrad on the projection table from partly factored gradients (state: [n_rel])."""
    t = _inplace_table(proj)
    if not state.is_contiguous():
        raise ValueError("state must be contiguous: it is updated in place")
    _lib.check(_lib.lib().kge_sparse_adagrad_factored(_ptr(t), _ptr(state), int(proj.shape[1]), C.byref(g._rel_insp._c),
                                                      C.byref(g._c), float(lr), float(eps), _stream()),
               "kge_sparse_adagrad_factored")


# ---- the reference's positional call shapes --------------------------------------------------
# run(batch_size, dim, nnodes, Eemb, h, t, nedges, Remb, r [, r_uniq, r_buf, r_cnt] [, extra])
# The three inspector tensors are accepted and ignored: they only steer the reference kernel's
# shared-memory relation cache and do not change the result.

def _sizes_ok(batch_size, dim, Eemb, h):
    if int(batch_size) != int(h.numel()):
        raise ValueError(f"batch_size {batch_size} != len(h) {h.numel()}")
    if int(dim) != int(Eemb.shape[1]):
        raise ValueError(f"dim {dim} != Eemb row width {Eemb.shape[1]}")


def transE(batch_size, dim, nnodes, Eemb, h, t, nedges, Remb, r, *reuse):
    """apps/kge/test_cuke.py:54 -> [batch, dim] = (Eemb[h] - Eemb[t]) + Remb[r]."""
    _sizes_ok(batch_size, dim, Eemb, h)
    return KGEModel("TransE", Eemb, Remb).residual(h, r, t)


def transH(batch_size, dim, nnodes, Eemb, h, t, nedges, Remb, r, *rest):
    """apps/kge/test_cuke.py:104: (..., rel_ids, uniq, buf, cnt, projection_emb)."""
    _sizes_ok(batch_size, dim, Eemb, h)
    Pemb = rest[-1]
    return KGEModel("TransH", Eemb, Remb, Pemb).residual(h, r, t)


def transR(batch_size, dim, nnodes, Eemb, h, t, nedges, Proj, r, *rest):
    """apps/kge/test_cuke.py:153: (batch, dim, 0, E, h, t, 0, Proj, r, uniq, buf, cnt, Remb)."""
    _sizes_ok(batch_size, dim, Eemb, h)
    Remb = rest[-1]
    m = KGEModel("TransR", Eemb, Remb, Proj)
    return m.residual(h, r, t, rel_insp=inspect([r], m.n_rel))


def transF(batch_size, dim, nnodes, Eemb, h, nedges, Remb, r, *rest):
    """apps/kge/test_cuke.py:198: (batch, dim, nnodes, E, h, nedges, R, r, uniq, buf, cnt, t) -> [batch]."""
    _sizes_ok(batch_size, dim, Eemb, h)
    t = rest[-1]
    return KGEModel("TransF", Eemb, Remb).score(h, r, t).pos


def RESCAL(batch_size, dim, nnodes, Eemb, h, nedges, Proj, r, *rest):
    """apps/kge/test_cuke.py:244: (batch, dim, nnodes, E, h, nedges, Proj, r, uniq, buf, cnt, t) -> [batch]."""
    _sizes_ok(batch_size, dim, Eemb, h)
    t = rest[-1]
    m = KGEModel("RESCAL", Eemb, None, Proj)
    return m.score(h, r, t, rel_insp=inspect([r], m.n_rel)).pos


def inspector(r: torch.Tensor, rel_num: int, C_: int = 16):
    """apps/kge/kge.py:249-271: (uniq[batch/16,16], buf[batch/16,16], cnt[batch/16]) int64 for sorted r."""
    if C_ != 16:
        raise ValueError("the reference's chunk size is fixed at 16 (inspector.cu:10)")
    r = _index(r, "r", r.device)
    if not r.is_cuda:
        raise KgeError("inspector needs a GPU tensor; there is no CPU path")
    nb = int(r.numel()) // 16
    uniq = torch.zeros((nb, 16), dtype=torch.int64, device=r.device)
    buf = torch.zeros((nb, 16), dtype=torch.int64, device=r.device)
    cnt = torch.zeros((nb,), dtype=torch.int64, device=r.device)
    _lib.check(_lib.lib().kge_build_index(_ptr(r), _ptr(uniq), _ptr(buf), _ptr(cnt), int(r.numel()),
                                          int(rel_num), _stream()), "kge_build_index")
    return uniq, buf, cnt


class _InspSet:
    """Per-batch state of a TrainStep: index tensors, both inspections, their jobs and events."""


class TrainStep:
    """One forward + backward pass over a fixed-shape batch with every buffer allocated up front.

    ``run()`` enqueues: inspector over concat(h, t, neg) and over r -> scores -> (margin loss)
    -> sparse row gradients.  Nothing is allocated and nothing synchronises inside ``run()``,
    so the sequence can be captured into a HIP graph (``capture()``) and replayed.
    loss = "sum":    upstream gradients are the caller-supplied ``dpos`` / ``dneg`` (default: ones)
    loss = "margin": margin-ranking loss with ``margin`` and ``sign``
    """

    kPipelineSets = 3  # one running, one being inspected, one being refilled

    def __init__(self, model: KGEModel, h, r, t, neg=None, chunk=None, loss="sum", margin=1.0,
                 sign=1.0, dpos=None, dneg=None, neg_mode="tail", factor_max=0, back_rows=True):
        self.m = model
        dev = model.dev
        L = self.L = _lib.lib()
        f32 = dict(dtype=torch.float32, device=dev)
        i32 = dict(dtype=torch.int32, device=dev)
        _, (h, r, t, neg, C_, N) = model._batch(h, r, t, neg, chunk, neg_mode=neg_mode)
        idx0 = (h, r, t, neg)
        B = self.B = int(h.numel())
        self.N, self.C = N, C_
        self.loss_kind, self.margin, self.sign = loss, float(margin), float(sign)

        self._parts = lambda ix: [ix[0], ix[2]] + ([ix[3]] if ix[3] is not None else [])
        self.n_occ = n_occ = sum(int(p.numel()) for p in self._parts(idx0))
        self._neg_mode = neg_mode
        # forward-only scoring needs no inspection unless the relation groups drive TransR / RESCAL
        self.needs_rel_groups = model.model in ("TransR", "RESCAL")
        self._sets = [self._make_set(idx0)]
        self._cur = 0
        self._staged, self._stage_at = collections.deque(), 0
        self._pipelined = False   # the ring of run(pipeline=True) has been set up
        self._timeline = None     # set by kernel_times()
        self.side = torch.cuda.Stream(device=dev)  # default priority
        self._dev_index = dev.index if dev.index is not None else torch.cuda.current_device()
        self.pos = torch.empty(B, **f32)
        self.neg = torch.empty((B, N), **f32) if neg is not None else None
        self.side_pos = torch.empty(B, **f32) if (model.model == "TransH" or
                                                  (model.model == "TransF" and neg is not None)) else None
        self.side_neg = torch.empty((2, B, N), **f32) if (model.model == "TransH" and neg is not None) else None
        self.residual = torch.empty((B, model.dim), **f32) if model.model in ("TransR", "RESCAL", "RotatE") \
            else None
        if model.model == "TransR" and neg is not None and not model._grouped_negatives_fit(self.bat):
            raise KgeError(f"TransR with shared negatives at batch {B} x {N} negatives, dim {model.dim}, {model.n_rel} relations: "
                           "the grouped path's worst-case workspaces exceed the library's cap; score the pairs as "
                           "explicit triples (KGEModel.score) or use smaller chunks of the batch")
        # TransR without negatives: the forward kernel also writes phi(residual) Proj^T, and the backward pass
        # reads no projection again (back_rows=False: backward forms the entity gradients with its own pass)
        self.back_rows = None
        if back_rows and B > 0 and L.kge_back_rows_ok(C.byref(model._tab), C.byref(self.bat)):
            self.back_rows = torch.empty((B, model.dim), **f32)
            self._sets[0].bat.back_rows = self.back_rows.data_ptr()
        self._ws_f_bytes = int(L.kge_score_fwd_workspace(C.byref(model._tab), C.byref(self.bat)))
        self._ws_f = torch.empty(max(self._ws_f_bytes, 1), dtype=torch.uint8, device=dev)
        # TransR / RESCAL without negatives: the forward workspace holds the batch's tile plans, which a
        # staged batch gets a step ahead (stage()); every set of the ring then keeps plans of its own
        self._plans_per_set = self.needs_rel_groups and neg is None and self._ws_f_bytes > 0
        self._sets[0].ws_f = self._ws_f
        self.loss = torch.zeros(1, **f32)
        if loss == "margin":
            self.dpos, self.dneg = torch.empty(B, **f32), torch.empty((B, N), **f32)
            self._ws_l = torch.empty(max(int(L.kge_margin_loss_workspace(B, N)), 1), dtype=torch.uint8, device=dev)
        else:
            self.dpos = torch.ones(B, **f32) if dpos is None else dpos.to(**f32).contiguous()
            self.dneg = None
            if neg is not None:
                self.dneg = torch.ones((B, N), **f32) if dneg is None else dneg.to(**f32).contiguous()
        self.saved = _lib.Saved(*[(x.data_ptr() if x is not None else None) for x in
                                  (self.pos, self.neg, self.side_pos, self.side_neg, self.residual)])
        if self.needs_rel_groups and self._ws_f_bytes:  # backward reuses the forward pass's tile plans
            self.saved.fwd_workspace, self.saved.fwd_workspace_bytes = self._ws_f.data_ptr(), self._ws_f_bytes
        if self.back_rows is not None:
            self.saved.back_rows = self.back_rows.data_ptr()
        self.ent_rows = torch.empty((n_occ, model.dim), **f32)
        self.rel_rows = torch.empty((B, model.rel_dim), **f32) if model.rel_dim else None
        self.aux_rows = None
        if model.model == "TransH":
            self.aux_rows = torch.empty((B, model.dim), **f32)
        elif model.model in ("TransR", "RESCAL"):
            self.aux_rows = torch.empty((min(B, model.n_rel), model.dim * model.dim), **f32)
        self.factor_max = int(factor_max)
        self.aux_x = self.aux_q = None
        if self.factor_max:
            if model.model not in ("TransR", "RESCAL") or neg is not None:
                raise ValueError("factor_max applies to TransR / RESCAL without shared negatives")
            self.aux_x, self.aux_q = torch.empty((B, model.dim), **f32), torch.empty((B, model.dim), **f32)
        self.grads = _lib.Grads(_ptr(self.ent_rows), _ptr(self.rel_rows), _ptr(self.aux_rows), _ptr(self.aux_x),
                                _ptr(self.aux_q), self.factor_max, 0)
        self._ws_b_bytes = int(L.kge_score_bwd_workspace(C.byref(model._tab), C.byref(self.bat)))
        self._ws_b = torch.empty(max(self._ws_b_bytes, 1), dtype=torch.uint8, device=dev)
        self.graph = None

    def _make_set(self, idx):
        """Index tensors plus everything the inspector writes for them: one set per batch in flight."""
        m, L, dev = self.m, self.L, self.m.dev
        i32 = dict(dtype=torch.int32, device=dev)
        h, r, t, neg = idx

        def make_insp(n, n_rows):
            ins = Inspection(n, n_rows, torch.zeros(1, **i32), torch.empty(max(n, 1), dtype=torch.int64, device=dev),
                             torch.empty(n + 1, **i32), torch.empty(max(n, 1), **i32),
                             torch.empty(max(n, 1), **i32), torch.empty(max(n, 1), **i32))
            ins._c = _lib.Inspection(n, n_rows, ins.num_unique_dev.data_ptr(), ins.unique_ids.data_ptr(),
                                     ins.seg_offsets.data_ptr(), ins.perm.data_ptr(), ins.inverse.data_ptr(),
                                     ins.sorted_seg.data_ptr())
            ws = torch.empty(max(int(L.kge_inspect_workspace(n, n_rows)), 1), dtype=torch.uint8, device=dev)
            return ins, ws

        s = _InspSet()
        s.idx = idx
        parts = self._parts(idx)
        s.ent_insp, s.ws_e = make_insp(self.n_occ, int(m.E.shape[0]))
        s.rel_insp, s.ws_r = make_insp(self.B, max(m.n_rel, 1))
        s.jobs = (_lib.InspectJob * 2)()
        for job, ps, ins, ws in ((s.jobs[0], parts, s.ent_insp, s.ws_e), (s.jobs[1], [r], s.rel_insp, s.ws_r)):
            for q, p_ in enumerate(ps):
                job.parts[q], job.part_len[q] = p_.data_ptr(), int(p_.numel())
            job.n_parts, job.n_rows, job.out = len(ps), ins.n_rows, ins._c
            job.workspace, job.workspace_bytes = ws.data_ptr(), ws.numel()
        s.bat = _lib.Batch(self.B, h.data_ptr(), r.data_ptr(), t.data_ptr(),
                           neg.data_ptr() if neg is not None else None, self.C, self.N,
                           C.pointer(s.ent_insp._c), C.pointer(s.rel_insp._c), None, NEG_MODES[self._neg_mode], 0)
        s.bat.insp_jobs = C.addressof(s.jobs)
        if getattr(self, "back_rows", None) is not None:
            s.bat.back_rows = self.back_rows.data_ptr()
        s.fusable = bool(L.kge_fused_inspection_ok(C.byref(m._tab), C.byref(s.bat), s.jobs))
        s.insp_event = torch.cuda.Event()
        s.done_event = None  # recorded on the main stream after the last pipelined step that used this set
        s.inputs_ready = None
        return s

    def add_batch(self, h, r, t, neg=None) -> int:
        """Another batch of the same shape, with index tensors and inspections of its own (scores, gradients
        and workspaces are shared).  Returns its number for ``select()``; the batch given to the
        constructor is number 0."""
        if self._staged or self._pipelined:
            raise KgeError("add_batch() cannot be mixed with the staged pipeline")
        _, (h, r, t, neg, C_, N) = self.m._batch(h, r, t, neg, self.C or None, neg_mode=self._neg_mode)
        if int(h.numel()) != self.B or N != self.N or (neg is None) != (self.neg is None):
            raise ValueError("every batch of a TrainStep has the shape of the first one")
        self._sets.append(self._make_set((h, r, t, neg)))
        return len(self._sets) - 1

    def select(self, i: int) -> None:
        """Make batch ``i`` (see ``add_batch``) the one the next ``run()`` processes."""
        if self._staged or self._pipelined:
            raise KgeError("select() cannot be mixed with the staged pipeline")
        if not 0 <= i < len(self._sets):
            raise IndexError(i)
        self._cur = i

    # -- per-kernel timing ----------------------------------------------------------------------------
    _LABELS = {k: k.encode() for k in ("inspect", "inspect(relations)", "margin_loss")}

    def _mark(self, label: str, st) -> None:
        if self._timeline is not None:
            _lib.check(self.L.kge_timeline_mark(self._timeline, self._LABELS[label], st), "kge_timeline_mark")

    def kernel_times(self, steps: int = 10, backward: bool = True, batches=None, lead=None, fused=None):
        """[(kernel name, mean milliseconds)] of one step, in launch order: ``steps`` steps are run with an
        event recorded behind every kernel (kge_batch.timeline) and read back after each step.  Event
        records between the kernels cost a little themselves, so the sum is an upper bound of the
        step time that ``run()`` alone takes.  ``batches``: batch numbers to rotate over.  ``lead``: work
        enqueued on the stream in front of every step, so that the host has enqueued the whole step
        before the device starts on it and the intervals hold no launch gaps: a callable, or a large
        tensor that is zero-filled (which also empties the caches in front of every step).  ``fused``: as in
        ``run()``; False times the launch forms of the staged issue (no riding inspection, merged launches) with
        the inspection in front of the step on the same stream."""
        L = self.L
        tl = L.kge_timeline_create(64)
        if not tl:
            raise KgeError("kge_timeline_create failed")
        main = torch.cuda.current_stream()
        st = C.c_void_p(main.cuda_stream)
        sums, names = None, None
        ms = (C.c_float * 64)()
        self._timeline = tl
        try:
            for i in range(steps):
                if batches:
                    self.select(batches[i % len(batches)])
                self.bat.timeline = tl
                if callable(lead):
                    lead()
                elif lead is not None:
                    lead.zero_()
                _lib.check(L.kge_timeline_begin(tl, st), "kge_timeline_begin")
                try:
                    self.run(backward, overlap=False, fused=fused)
                finally:
                    self.bat.timeline = None
                main.synchronize()
                n = L.kge_timeline_elapsed(tl, ms)
                if n < 0:
                    _lib.check(n, "kge_timeline_elapsed")
                cur = [tl.contents.labels[k].decode() for k in range(n)]
                if names is None:
                    names, sums = cur, [0.0] * n
                elif cur != names:
                    raise KgeError(f"the kernel sequence changed between steps: {names} vs {cur}")
                for k in range(n):
                    sums[k] += ms[k]
        finally:
            self._timeline = None
            L.kge_timeline_destroy(tl)
        return [(nm, s / steps) for nm, s in zip(names or [], sums or [])]

    # the set of the step enqueued last (the only set unless run(pipeline=True) is used)
    idx = property(lambda self: self._sets[self._cur].idx)
    ent_insp = property(lambda self: self._sets[self._cur].ent_insp)
    rel_insp = property(lambda self: self._sets[self._cur].rel_insp)
    bat = property(lambda self: self._sets[self._cur].bat)
    _jobs = property(lambda self: self._sets[self._cur].jobs)
    insp_event = property(lambda self: self._sets[self._cur].insp_event)

    # the individual stages, each one C call
    def inspect(self, st, backward=True):
        """Both inspections in one call; forward-only steps inspect r alone, and only if needed."""
        if backward:
            _lib.check(self.L.kge_inspect_batch(self._jobs, 2, st), "kge_inspect_batch")
        elif self.needs_rel_groups:
            _lib.check(self.L.kge_inspect_batch(C.byref(self._jobs[1]), 1, st), "kge_inspect_batch")

    def forward(self, st, for_backward=True):
        bat = self.bat
        if self.back_rows is not None:  # a forward-only step does not pay for the rows of the backward pass
            bat.back_rows = self.back_rows.data_ptr() if for_backward else None
        _lib.check(self.L.kge_score_fwd(C.byref(self.m._tab), C.byref(bat), _ptr(self.pos), _ptr(self.neg),
                                        _ptr(self.side_pos), _ptr(self.side_neg), _ptr(self.residual),
                                        _ptr(self._fwd_ws()), self._ws_f_bytes, st), "kge_score_fwd")

    def _fwd_ws(self):
        """The forward workspace of the current set (its own where the sets keep their tile plans apart);
        backward is pointed at the same one."""
        cur = self._sets[self._cur]
        ws = self._ws_f
        if self._plans_per_set:
            if getattr(cur, "ws_f", None) is None:
                cur.ws_f = torch.empty(max(self._ws_f_bytes, 1), dtype=torch.uint8, device=self.m.dev)
            ws = cur.ws_f
        if self.needs_rel_groups and self._ws_f_bytes:
            self.saved.fwd_workspace = ws.data_ptr()
        return ws

    def loss_grad(self, st):
        if self.loss_kind == "margin":
            _lib.check(self.L.kge_margin_loss(_ptr(self.pos), _ptr(self.neg), self.B, self.N, self.margin,
                                              self.sign, _ptr(self.loss), _ptr(self.dpos), _ptr(self.dneg),
                                              _ptr(self._ws_l), self._ws_l.numel(), st), "kge_margin_loss")
            self._mark("margin_loss", st)

    def backward(self, st):
        _lib.check(self.L.kge_score_bwd(C.byref(self.m._tab), C.byref(self.bat), C.byref(self.saved),
                                        _ptr(self.dpos), _ptr(self.dneg), C.byref(self.grads), _ptr(self._ws_b),
                                        self._ws_b_bytes, st), "kge_score_bwd")

    # ---- pipelined issue: index tensors and inspections in a ring of sets ----
    def _ring(self):
        """Grow to kPipelineSets sets on first use (copies of the construction-time indices)."""
        self._pipelined = True
        if len(self._sets) < self.kPipelineSets:
            first = self._sets[0].idx
            while len(self._sets) < self.kPipelineSets:
                self._sets.append(self._make_set(tuple(x.clone() if x is not None else None for x in first)))
            torch.cuda.current_stream().synchronize()  # once: the copies are read from other streams
            self._stage_at = (self._cur + 1) % len(self._sets)
        return self._sets

    def next_inputs(self, stream=None):
        """The index tensors (h, r, t, neg) that the next ``stage()`` will hand to the inspector.
        ``stream`` (default: the current one) is made to wait until the last step that read them has
        finished, so the caller can refill them in place on that stream."""
        nxt = self._ring()[self._stage_at]
        if nxt.done_event is not None:
            (stream or torch.cuda.current_stream()).wait_event(nxt.done_event)
        return nxt.idx

    def stage(self, inputs_ready=None, batch=None):
        """Declare the tensors of ``next_inputs()`` final -- complete once ``inputs_ready`` (a
        torch.cuda.Event; None = already complete) has fired -- and start their inspection on the
        side stream.  ``run(pipeline=True)`` consumes staged batches oldest first.  Staging one
        batch ahead of the step that is about to run lets the inspector finish before backward asks
        for it, which also keeps the host off the slow path of waiting on a pending event.
        ``batch``: stage batch number ``batch`` of ``add_batch()`` instead of the ring's next set (its
        index tensors are used as they are; nothing is copied)."""
        if batch is None:
            sets = self._ring()
            at = self._stage_at
        else:
            if self._pipelined:
                raise KgeError("stage(batch=...) cannot be mixed with the ring of next_inputs()")
            sets, at = self._sets, int(batch)
            if not 0 <= at < len(sets) or at in self._staged:
                raise KgeError(f"batch {batch} does not exist or is already staged")
        if len(self._staged) >= max(len(sets) - 1, 1):
            raise KgeError(f"at most {max(len(sets) - 1, 1)} batches can be staged ahead of run()")
        s, side = sets[at], self.side
        if s.done_event is not None:
            side.wait_event(s.done_event)  # its inspection may still be read by an earlier step
        if inputs_ready is not None:
            side.wait_event(inputs_ready)
        s.inputs_ready = inputs_ready
        sst = C.c_void_p(side.cuda_stream)
        if self._plans_per_set:
            # the relation groups drive the forward pass: inspected and planned here, a step ahead, so
            # that run() starts with the projection kernel
            if getattr(s, "ws_f", None) is None:
                s.ws_f = torch.empty(max(self._ws_f_bytes, 1), dtype=torch.uint8, device=self.m.dev)
            # (both index sets in one batch of launches, then the plans: the step waits for all of it at once)
            _lib.check(self.L.kge_inspect_batch(s.jobs, 2, sst), "kge_inspect_batch")
            _lib.check(self.L.kge_transr_plan(C.byref(self.m._tab), C.byref(s.bat), _ptr(s.ws_f), self._ws_f_bytes, sst),
                       "kge_transr_plan")
            s.bat.plans_ready = 1  # (run() waits for insp_event, recorded below behind the plans)
        elif self.needs_rel_groups:  # (with shared negatives the forward call plans its own row list)
            _lib.check(self.L.kge_inspect_batch(C.byref(s.jobs[0]), 1, sst), "kge_inspect_batch(entities)")
        else:
            _lib.check(self.L.kge_inspect_batch(s.jobs, 2, sst), "kge_inspect_batch")
        s.insp_event.record(side)
        self._staged.append(at)
        if batch is None:
            self._stage_at = (at + 1) % len(sets)

    @property
    def fusable(self):
        """True if the inspections of this batch shape can ride inside the score kernels' launches."""
        return self._sets[self._cur].fusable

    def run(self, backward=True, overlap=True, pipeline=False, inputs_ready=None, fused=None):
        """Enqueue one step.

        fused (default whenever the batch qualifies: index sets of at most 65536 ids; shared
        negatives, or TransR / RESCAL on their grouped path): the inspector's workgroups ride in
        front of the score kernels' own workgroups in the same launches, so the whole step is one
        chain of kernels on one stream with the inspection off its critical path.  TransR /
        RESCAL inspect the relations first (the forward pass is planned from their groups); only
        the entity inspection rides.

        Otherwise, with overlap, the inspector runs on a side stream while the main stream
        computes scores and per-occurrence gradients; backward waits for it right before its
        segmented reduction.  TransR / RESCAL need the relation groups in the forward pass, so
        their relation inspection stays on the main stream.

        pipeline=True runs the oldest batch handed over with ``stage()`` (staging the tensors of
        ``next_inputs()`` first, with ``inputs_ready``, if none is waiting).  Index tensors and
        inspections live in a ring of sets, so the side stream never waits for the step before.
        Results (``sparse_grads()``, ``pos`` ...) are those of the step enqueued last.  Not
        capturable into one graph: the dependencies cross steps."""
        main = _current_stream(self._dev_index)
        st = C.c_void_p(main.cuda_stream)
        for s_ in self._sets:  # cached unique counts belong to the batches of earlier steps
            s_.ent_insp._u = s_.rel_insp._u = None
        if not pipeline:
            self.bat.plans_ready = 0  # the forward call plans for itself
        if fused is None:
            fused = backward and not pipeline and self.fusable
        if fused:
            if not (backward and self.fusable) or pipeline or self._staged:
                raise KgeError("fused inspection needs a backward step over a batch that qualifies "
                               "(TrainStep.fusable), outside the staged pipeline")
            bat = self.bat
            bat.insp_ready, bat.fuse_inspection = None, 1
            try:
                if self.needs_rel_groups:  # the forward pass is planned from the relation groups
                    _lib.check(self.L.kge_inspect_batch(C.byref(self._jobs[1]), 1, st), "kge_inspect_batch(relations)")
                    self._mark("inspect(relations)", st)
                self.forward(st)
                self.loss_grad(st)
                self.backward(st)
            finally:
                bat.fuse_inspection = 0
            self._record_done(main)
            return
        if not (backward and overlap):
            self.bat.insp_ready = None
            self.inspect(st, backward)
            if backward or self.needs_rel_groups:
                self._mark("inspect", st)
            self.forward(st, backward)
            if backward:
                self.loss_grad(st)
                self.backward(st)
            return
        if pipeline:
            if not self._staged:
                self.stage(inputs_ready)
            self._cur = self._staged.popleft()
            cur = self._sets[self._cur]
            if cur.inputs_ready is not None:
                main.wait_event(cur.inputs_ready)  # the score kernels read the index tensors too
            if self._plans_per_set:
                # Relation groups, tile plans and the entity inspection of this batch were all enqueued by stage(), a
                # step ahead, on the side stream: ONE wait on the event recorded behind the last of them covers the
                # forward pass (plans) and the backward pass (entity inspection); a second wait in front of the
                # reduction would cost its 2-3 us for an event that has long fired.
                main.wait_event(cur.insp_event)
                cur.bat.insp_ready = None
                self.forward(st)
                self.loss_grad(st)
                self.backward(st)
                self._record_done(main, pipeline)
                return
            elif self.needs_rel_groups:
                _lib.check(self.L.kge_inspect_batch(C.byref(cur.jobs[1]), 1, st), "kge_inspect_batch(relations)")
        else:
            if self._staged:
                raise KgeError("staged batches are waiting: use run(pipeline=True)")
            cur, side = self._sets[self._cur], self.side
            sst = C.c_void_p(side.cuda_stream)
            side.wait_stream(main)
            if self.needs_rel_groups:
                _lib.check(self.L.kge_inspect_batch(C.byref(cur.jobs[1]), 1, st), "kge_inspect_batch(relations)")
                _lib.check(self.L.kge_inspect_batch(C.byref(cur.jobs[0]), 1, sst), "kge_inspect_batch(entities)")
            else:
                _lib.check(self.L.kge_inspect_batch(cur.jobs, 2, sst), "kge_inspect_batch")
            cur.insp_event.record(side)
        cur.bat.insp_ready = cur.insp_event.cuda_event
        self.forward(st)
        self.loss_grad(st)
        self.backward(st)
        self._record_done(main, pipeline)

    def _record_done(self, main, force=False):
        """Marks the end of the step that read the current set, for the ring's reuse check."""
        cur = self._sets[self._cur]
        if force or (len(self._sets) > 1 and not torch.cuda.is_current_stream_capturing()):
            if cur.done_event is None:
                cur.done_event = torch.cuda.Event()
            cur.done_event.record(main)

    def capture(self, backward=True):
        """Record run() into a HIP graph; replay() then launches the whole step at once."""
        self.run(backward)  # warm-up outside capture (module loading, lazy init)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.run(backward)
        self.graph = g
        return g

    def replay(self):
        self.graph.replay()

    def capture_staged(self, cur: int, nxt: int, backward=True):
        """One HIP graph with two branches: the step of batch ``cur`` on the capturing stream and, beside it on
        the side stream, the inspection of batch ``nxt`` (TransR / RESCAL: its relation groups and tile plans
        too).  Replaying the graphs (cur, nxt) = (0, 1), (1, 2), ... one after the other is the staged issue
        of ``stage(batch=...)`` / ``run(pipeline=True)`` with one launch per step: the inspection of batch
        ``cur`` was made by the replay before (graph launches on one stream run one after the other), so
        nothing inside the graph waits for it.  Before the first replay batch ``cur`` of the first graph has
        to be inspected once: ``prime_staged(cur)``."""
        if self._staged or self._pipelined:
            raise KgeError("capture_staged() cannot be mixed with the staged pipeline")
        self.prime_staged(cur)
        self.prime_staged(nxt)
        self._run_staged_pair(cur, nxt, backward)  # warm-up outside capture (module loading, lazy init)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._run_staged_pair(cur, nxt, backward)
        return g

    def use_batch(self, i: int) -> None:
        """Point ``sparse_grads()`` and the inspection properties at batch ``i`` (after replaying a graph of
        ``capture_staged(i, ...)``, which Python does not see)."""
        self._cur = i
        for s_ in self._sets:
            s_.ent_insp._u = s_.rel_insp._u = None

    def prime_staged(self, i: int) -> None:
        """Inspect (and, for TransR / RESCAL, plan) batch ``i`` on the current stream: what the side branch of
        the graph before would have done."""
        self._inspect_ahead(self._sets[i], C.c_void_p(torch.cuda.current_stream().cuda_stream))

    def _inspect_ahead(self, s, sst) -> None:
        if self._plans_per_set:
            if getattr(s, "ws_f", None) is None:
                s.ws_f = torch.empty(max(self._ws_f_bytes, 1), dtype=torch.uint8, device=self.m.dev)
            _lib.check(self.L.kge_inspect_batch(C.byref(s.jobs[1]), 1, sst), "kge_inspect_batch(relations)")
            _lib.check(self.L.kge_transr_plan(C.byref(self.m._tab), C.byref(s.bat), _ptr(s.ws_f), self._ws_f_bytes, sst),
                       "kge_transr_plan")
            s.bat.plans_ready = 1
            _lib.check(self.L.kge_inspect_batch(C.byref(s.jobs[0]), 1, sst), "kge_inspect_batch(entities)")
        elif self.needs_rel_groups:
            _lib.check(self.L.kge_inspect_batch(C.byref(s.jobs[0]), 1, sst), "kge_inspect_batch(entities)")
        else:
            _lib.check(self.L.kge_inspect_batch(s.jobs, 2, sst), "kge_inspect_batch")

    def _run_staged_pair(self, cur: int, nxt: int, backward: bool) -> None:
        main, side = torch.cuda.current_stream(), self.side
        st = C.c_void_p(main.cuda_stream)
        side.wait_stream(main)                                   # fork
        self._inspect_ahead(self._sets[nxt], C.c_void_p(side.cuda_stream))
        self.use_batch(cur)
        bat = self.bat
        bat.insp_ready, bat.fuse_inspection = None, 0
        if self.needs_rel_groups and not self._plans_per_set:    # (shared negatives: groups needed by the forward call)
            _lib.check(self.L.kge_inspect_batch(C.byref(self._jobs[1]), 1, st), "kge_inspect_batch(relations)")
        self.forward(st, backward)
        if backward:
            self.loss_grad(st)
            self.backward(st)
        main.wait_stream(side)                                   # join

    # ---- the staged issue from native code: one library call per step ----
    def _native_state(self):
        """kge_step_batch per batch (events created once) and the kge_step_buffers of this TrainStep."""
        if getattr(self, "_native", None) is not None:
            return self._native
        main = torch.cuda.current_stream()

        def event():
            ev = torch.cuda.Event()
            ev.record(main)       # (torch creates the underlying event at its first record)
            return ev

        batches = []
        for s_ in self._sets:
            sb = _lib.StepBatch()
            sb.bat = s_.bat
            sb.bat.insp_ready, sb.bat.fuse_inspection, sb.bat.plans_ready, sb.bat.timeline = None, 0, 0, None
            sb.bat.back_rows = self.back_rows.data_ptr() if self.back_rows is not None else None
            if self._plans_per_set:
                if getattr(s_, "ws_f", None) is None:
                    s_.ws_f = torch.empty(max(self._ws_f_bytes, 1), dtype=torch.uint8, device=self.m.dev)
                sb.fwd_workspace, sb.fwd_workspace_bytes = s_.ws_f.data_ptr(), self._ws_f_bytes
            s_.native_events = [event() for _ in range(3)]
            sb.inspected, sb.planned, sb.released = (e.cuda_event for e in s_.native_events)
            sb.released_valid = 0
            batches.append(sb)
        buf = _lib.StepBuffers()
        for name in ("pos", "neg", "side_pos", "side_neg", "residual", "dpos", "dneg"):
            t = getattr(self, name)
            setattr(buf, name, t.data_ptr() if t is not None else None)
        buf.fwd_workspace, buf.fwd_workspace_bytes = self._ws_f.data_ptr(), self._ws_f_bytes
        if self.loss_kind == "margin":
            buf.loss, buf.margin, buf.sign = self.loss.data_ptr(), self.margin, self.sign
            buf.loss_workspace, buf.loss_workspace_bytes = self._ws_l.data_ptr(), self._ws_l.numel()
        buf.grads = self.grads
        buf.bwd_workspace, buf.bwd_workspace_bytes = self._ws_b.data_ptr(), self._ws_b_bytes
        torch.cuda.synchronize()
        self._native = (batches, buf)
        return self._native

    def run_native(self, cur, nxt) -> None:
        """The staged issue in ONE library call (kge_train_step_staged): the step of batch ``cur`` on the current
        stream and, on the side stream, the inspection of batch ``nxt`` (TransR / RESCAL: its tile plans too) for
        the call that follows.  ``cur=None`` only stages ``nxt`` (in front of the first step); ``nxt=None`` only
        runs ``cur``.  Same launches in the same order as ``stage(batch=nxt)`` + ``run(pipeline=True)``, hence
        the same results bit for bit; what it saves is the host's time per step."""
        if self._staged or self._pipelined:
            raise KgeError("run_native() cannot be mixed with the staged pipeline")
        batches, buf = self._native_state()
        st = C.c_void_p(_current_stream(self._dev_index).cuda_stream)
        _lib.check(self.L.kge_train_step_staged(C.byref(self.m._tab), C.byref(batches[cur]) if cur is not None else None,
                                                C.byref(batches[nxt]) if nxt is not None else None, C.byref(buf), st,
                                                C.c_void_p(self.side.cuda_stream)), "kge_train_step_staged")
        if cur is not None:
            self.use_batch(cur)

    def sparse_grads(self) -> SparseGrads:
        ue, ur = self.ent_insp.num_unique, self.rel_insp.num_unique
        return SparseGrads(self.ent_insp.unique_ids[:ue], self.ent_rows[:ue], self.rel_insp.unique_ids[:ur],
                           self.rel_rows[:ur] if self.rel_rows is not None else None,
                           self.aux_rows[:ur] if self.aux_rows is not None else None,
                           self.aux_x, self.aux_q, self.factor_max,
                           self.rel_insp.seg_offsets[:ur + 1] if self.factor_max else None, self.grads, self.rel_insp)
