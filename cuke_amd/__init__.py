"""MI355X-native KGE score-function kernels behind the cuke apps/kge operator surface."""
from .kge import (KGEModel, TrainStep, Inspection, Forward, SparseGrads, inspect, inspector, margin_loss,
                  transE, transH, transR, transF, RESCAL, KgeError)

__all__ = ["KGEModel", "TrainStep", "Inspection", "Forward", "SparseGrads", "inspect", "inspector",
           "margin_loss", "transE", "transH", "transR", "transF", "RESCAL", "KgeError"]
