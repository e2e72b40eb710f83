"""Schedulers for computations and communications, and their registry entries (same keys as the
reference's elf/scheduling/__init__.py:11-85)."""

from .scheduling import *  # noqa: F401,F403
from .scheduling import schedule_to_str, check_schedule_validity, OpOptions, Operation, OperationType
from .comm_scheduling import *  # noqa: F401,F403
from .schedulers import *  # noqa: F401,F403
from . import schedulers as _s, comm_scheduling as _c
from ..registry import SCHEDULERS, COMM_SCHEDULERS

SCHEDULERS.register(["afab", "gpipe"], _s.generate_afab_schedule, "All Forward All Backward as in GPipe https://arxiv.org/abs/1811.06965")
SCHEDULERS.register(["1f1b", "megatron"], _s.generate_1f1b_schedule, "One Forward One Backward as in PipeDream https://arxiv.org/abs/1806.03377")
SCHEDULERS.register("hanayo", _s.generate_hanayo_schedule, "Hanayo schedule as in https://dl.acm.org/doi/10.1145/3581784.3607073")
SCHEDULERS.register("full_remat", _s.generate_full_remat_schedule, "GPipe with every forward fully checkpointed, for memory-constrained setups.")
SCHEDULERS.register("zbh1", _s.generate_zbh1_schedule, "ZB-H1 schedule as in https://arxiv.org/abs/2401.10241")
SCHEDULERS.register("zbh2", _s.generate_zbh2_schedule, "ZB-H2 schedule as in https://arxiv.org/abs/2401.10241")
SCHEDULERS.register("zbv", _s.generate_zbv_schedule, "ZB-V schedule as in https://arxiv.org/abs/2401.10241 (2 stages per device, nmb = 2 * devices).")
SCHEDULERS.register("inference", _s.generate_inference_schedule, "Inference schedule. Forward pass only.")
SCHEDULERS.register("fixed", _s.FixedSchedule, "Fixed schedule. Use a dictionary to specify the schedule.")


def _auto_placeholder(*_):
	"""Stands for "solve the remat ILP for every base scheduler and keep the best"; it is replaced
	by an AutoScheduler when a memory budget is given, and produces no schedule on its own."""
	return None


SCHEDULERS.register("auto", _auto_placeholder, "Solves the remat ILP for all base schedulers and uses the best objective value (needs memory_budget).")

COMM_SCHEDULERS.register("topo", _c.topological_sort, "Topological sort of the communications. No optimizations are performed.")
COMM_SCHEDULERS.register("simulation", _c.smart_topological_sort, "Simulate execution to schedule communications together across ranks.")
COMM_SCHEDULERS.register("pipelined", _c.pipelined_topological_sort, "Pipelines receive -> compute -> send to utilize compute/comm overlapping.")
