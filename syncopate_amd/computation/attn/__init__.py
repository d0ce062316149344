from .template import attention, attention_forward, build_waves_and_signals_divisible  # noqa: F401
