"""ctypes binding of libkge_mi355.so (the C ABI declared in include/kge_mi355.h).

There is no CPU or PyTorch fallback: if the HIP library has not been built the
first call raises.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libkge_mi355.so")

MODELS = {"TransE": 0, "TransH": 1, "TransR": 2, "DistMult": 3, "ComplEx": 4, "RotatE": 5,
          "TransF": 6, "RESCAL": 7}


class KgeError(RuntimeError):
    pass


class Tables(C.Structure):
    _fields_ = [("model", C.c_int32), ("norm_p", C.c_int32), ("gamma", C.c_float),
                ("flags", C.c_int32), ("dim", C.c_int64), ("rel_dim", C.c_int64),
                ("n_ent", C.c_int64), ("n_rel", C.c_int64),
                ("ent", C.c_void_p), ("rel", C.c_void_p), ("aux", C.c_void_p)]


class Inspection(C.Structure):
    _fields_ = [("n", C.c_int64), ("n_rows", C.c_int64), ("num_unique", C.c_void_p),
                ("unique_ids", C.c_void_p), ("seg_offsets", C.c_void_p), ("perm", C.c_void_p),
                ("inverse", C.c_void_p), ("sorted_seg", C.c_void_p)]


class InspectJob(C.Structure):
    _fields_ = [("parts", C.c_void_p * 4), ("part_len", C.c_int64 * 4), ("n_parts", C.c_int32),
                ("reserved", C.c_int32), ("n_rows", C.c_int64), ("out", Inspection),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class Timeline(C.Structure):
    _fields_ = [("begin", C.c_void_p), ("events", C.POINTER(C.c_void_p)), ("labels", C.POINTER(C.c_char_p)),
                ("capacity", C.c_int32), ("count", C.c_int32), ("dropped", C.c_int32), ("reserved", C.c_int32)]


PAIR_SUMS_VALU = 1  # kge_tables.flags


class Batch(C.Structure):
    _fields_ = [("batch", C.c_int64), ("h", C.c_void_p), ("r", C.c_void_p), ("t", C.c_void_p),
                ("neg", C.c_void_p), ("chunk", C.c_int64), ("n_neg", C.c_int64),
                ("ent_insp", C.POINTER(Inspection)), ("rel_insp", C.POINTER(Inspection)),
                ("insp_ready", C.c_void_p), ("neg_mode", C.c_int32), ("fuse_inspection", C.c_int32),
                ("insp_jobs", C.c_void_p), ("timeline", C.POINTER(Timeline)),
                ("plans_ready", C.c_int32), ("reserved", C.c_int32), ("back_rows", C.c_void_p)]


class Saved(C.Structure):
    _fields_ = [("pos", C.c_void_p), ("neg", C.c_void_p), ("side_pos", C.c_void_p),
                ("side_neg", C.c_void_p), ("residual", C.c_void_p),
                ("fwd_workspace", C.c_void_p), ("fwd_workspace_bytes", C.c_size_t), ("back_rows", C.c_void_p)]


class Grads(C.Structure):
    _fields_ = [("ent_rows", C.c_void_p), ("rel_rows", C.c_void_p), ("aux_rows", C.c_void_p),
                ("aux_x", C.c_void_p), ("aux_q", C.c_void_p), ("aux_factor_max", C.c_int32), ("reserved", C.c_int32)]


class StepBatch(C.Structure):
    _fields_ = [("bat", Batch), ("fwd_workspace", C.c_void_p), ("fwd_workspace_bytes", C.c_size_t),
                ("inspected", C.c_void_p), ("planned", C.c_void_p), ("released", C.c_void_p),
                ("released_valid", C.c_int32), ("reserved", C.c_int32)]


class StepBuffers(C.Structure):
    _fields_ = [("pos", C.c_void_p), ("neg", C.c_void_p), ("side_pos", C.c_void_p), ("side_neg", C.c_void_p),
                ("residual", C.c_void_p), ("fwd_workspace", C.c_void_p), ("fwd_workspace_bytes", C.c_size_t),
                ("loss", C.c_void_p), ("margin", C.c_float), ("sign", C.c_float), ("loss_workspace", C.c_void_p),
                ("loss_workspace_bytes", C.c_size_t), ("dpos", C.c_void_p), ("dneg", C.c_void_p), ("grads", Grads),
                ("bwd_workspace", C.c_void_p), ("bwd_workspace_bytes", C.c_size_t)]


EXPORTS = {
    # name: (restype, argtypes)
    "kge_strerror": (C.c_char_p, [C.c_int]),
    "kge_abi_version": (C.c_int, []),
    "kge_timeline_create": (C.POINTER(Timeline), [C.c_int32]),
    "kge_timeline_destroy": (None, [C.POINTER(Timeline)]),
    "kge_timeline_begin": (C.c_int, [C.POINTER(Timeline), C.c_void_p]),
    "kge_timeline_mark": (C.c_int, [C.POINTER(Timeline), C.c_char_p, C.c_void_p]),
    "kge_timeline_elapsed": (C.c_int, [C.POINTER(Timeline), C.POINTER(C.c_float)]),
    "kge_residual_fwd": (C.c_int, [C.POINTER(Tables), C.POINTER(Batch), C.c_void_p, C.c_void_p, C.c_size_t,
                                   C.c_void_p]),
    "kge_score_fwd_workspace": (C.c_size_t, [C.POINTER(Tables), C.POINTER(Batch)]),
    "kge_transr_plan": (C.c_int, [C.POINTER(Tables), C.POINTER(Batch), C.c_void_p, C.c_size_t, C.c_void_p]),
    "kge_score_fwd": (C.c_int, [C.POINTER(Tables), C.POINTER(Batch), C.c_void_p, C.c_void_p,
                                C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "kge_inspect_workspace": (C.c_size_t, [C.c_int64, C.c_int64]),
    "kge_inspect": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(C.c_int64), C.c_int, C.c_int64,
                              C.POINTER(Inspection), C.c_void_p, C.c_size_t, C.c_void_p]),
    "kge_inspect_batch": (C.c_int, [C.POINTER(InspectJob), C.c_int, C.c_void_p]),
    "kge_fused_inspection_ok": (C.c_int, [C.POINTER(Tables), C.POINTER(Batch), C.POINTER(InspectJob)]),
    "kge_back_rows_ok": (C.c_int, [C.POINTER(Tables), C.POINTER(Batch)]),
    "kge_margin_loss_workspace": (C.c_size_t, [C.c_int64, C.c_int64]),
    "kge_margin_loss": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_float,
                                  C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_size_t, C.c_void_p]),
    "kge_margin_loss_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_float,
                                         C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "kge_score_bwd_workspace": (C.c_size_t, [C.POINTER(Tables), C.POINTER(Batch)]),
    "kge_score_bwd": (C.c_int, [C.POINTER(Tables), C.POINTER(Batch), C.POINTER(Saved), C.c_void_p,
                                C.c_void_p, C.POINTER(Grads), C.c_void_p, C.c_size_t, C.c_void_p]),
    "kge_build_index": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                  C.c_int64, C.c_void_p]),
    "kge_flatten_negatives": (C.c_int, [C.POINTER(Batch), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "kge_sparse_sgd": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_float,
                                 C.c_void_p]),
    "kge_sparse_adagrad": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64,
                                     C.c_void_p, C.c_float, C.c_float, C.c_void_p]),
    "kge_sparse_sgd_factored": (C.c_int, [C.c_void_p, C.c_int64, C.POINTER(Inspection), C.POINTER(Grads), C.c_float,
                                          C.c_void_p]),
    "kge_sparse_adagrad_factored": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.POINTER(Inspection), C.POINTER(Grads),
                                              C.c_float, C.c_float, C.c_void_p]),
    "kge_train_step_staged": (C.c_int, [C.POINTER(Tables), C.POINTER(StepBatch), C.POINTER(StepBatch), C.POINTER(StepBuffers),
                                        C.c_void_p, C.c_void_p]),
    "kge_sample_negatives": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_uint64, C.c_uint64, C.c_void_p]),
    "kge_check_indices": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]),
}

_lib = None


ABI_VERSION = 7  # layout of the ctypes structures above; must match kge_abi_version()


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise KgeError(
                f"{LIB_PATH} is missing: build it with `python -m cuke_amd.build` "
                "(hipcc, gfx950). There is no fallback path.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        if handle.kge_abi_version() != ABI_VERSION:
            raise KgeError(f"{LIB_PATH} has ABI version {handle.kge_abi_version()}, this package expects "
                           f"{ABI_VERSION}: rebuild it with `python -m cuke_amd.build`")
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise KgeError(f"{what}: {lib().kge_strerror(rc).decode()} ({rc})")
