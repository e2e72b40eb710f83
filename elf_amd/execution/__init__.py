"""Execution of a schedule on the stages of one rank."""

from .autograd_block import AutogradStageBlock
from .block import HipStageBlock, StageBlockBase, Variable
from .engine import Engine, GraphedStep, compute_loss
from .offload import PinnedHostTensorPool, StageOffloader

__all__ = ["Engine", "GraphedStep", "HipStageBlock", "AutogradStageBlock", "StageBlockBase", "Variable", "StageOffloader", "PinnedHostTensorPool", "compute_loss"]
