"""Execution of a schedule on the stages of one rank."""

from .block import HipStageBlock, Variable
from .engine import Engine, GraphedStep, compute_loss
from .offload import PinnedHostTensorPool, StageOffloader

__all__ = ["Engine", "GraphedStep", "HipStageBlock", "Variable", "StageOffloader", "PinnedHostTensorPool", "compute_loss"]
