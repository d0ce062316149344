"""Bridge between the communication plan and the compute kernels: a plan is lowered to
per-rank, per-buffer wave schedules whose flattened rows are the kernels' arguments."""

from .lowering import lower_comm_plan_to_raw_schedules  # noqa: F401
from .tile_schedule import Mod1DSchedule, RawSchedule, SimplifiedSchedule, TileBlock, TileCoord  # noqa: F401
