"""MI355X-native KGE score-function kernels behind the cuke apps/kge operator surface."""
from .kge import (KGEModel, TrainStep, Inspection, Forward, SparseGrads, inspect, inspector, margin_loss,
                  sparse_sgd, sparse_adagrad, transE, transH, transR, transF, RESCAL, KgeError)
from .data import KGDataset, TrainSampler

__all__ = ["KGEModel", "TrainStep", "Inspection", "Forward", "SparseGrads", "inspect", "inspector",
           "margin_loss", "sparse_sgd", "sparse_adagrad", "transE", "transH", "transR", "transF", "RESCAL",
           "KGDataset", "TrainSampler", "KgeError"]
