"""syncopate_amd — MI355X-native chunk-scheduled compute kernels behind Syncopate's host API.

Host side (pure Python): communication IR, plan builders, signal planning,
lowering to per-rank wave schedules.  Device side: hand-written gfx950 HIP
kernels reached through the C ABI of csrc/libsyncopate_hip.so.
"""

__version__ = "0.1.0"
