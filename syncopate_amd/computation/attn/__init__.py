from .template import attention, attention_forward, build_waves_and_signals_divisible  # noqa: F401
from .work_plan import WorkPlan, plan_attention_work  # noqa: F401
