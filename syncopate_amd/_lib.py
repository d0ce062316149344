"""ctypes binding of libsyncopate_hip.so (the C ABI declared in include/syncopate_hip.h).

There is no fallback: if the library has not been built, or a call returns a
non-zero code, this module raises.  torch is imported before the library is
opened so that both use the same HIP runtime.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_float, c_int32, c_int64, c_uint32, c_uint64, c_void_p
from pathlib import Path
from typing import Optional

import torch  # noqa: F401  (must precede CDLL: loads the HIP runtime the kernels run on)

# SYNCOPATE_HIP_LIBRARY names another build of the library (for comparing two builds on one device)
LIB_PATH = Path(os.environ.get("SYNCOPATE_HIP_LIBRARY") or Path(__file__).resolve().parent / "csrc" / "libsyncopate_hip.so")

SYN_DTYPE_BF16 = 0
SYN_DTYPE_FP16 = 1
SYN_EINVAL = -22
SYN_ERANGE = -34
SYN_EALIGN = -75
SYN_E2BIG = -7
SYN_STATIC_MAX_WAVES = 4096
SYN_STATUS_WORDS = 4
SYN_STATUS_SPIN_TIMEOUT = 1
SYN_GEMM_XCD_REMAP = 1
SYN_GEMM_EIGHT_WAVES = 2
SYN_GEMM_RING_PIPE = 4
SYN_GEMM_NO_K_STAGGER = 8
SYN_GEMM_TWO_STAGE = 16
SYN_GEMM_MFMA_32X32 = 32
SYN_GEMM_ACQUIRE_ALWAYS = 64
SYN_ATTN_PAIR_Q_BLOCKS = 1
SYN_ATTN_XCD_REMAP = 2
SYN_ATTN_CHAIN_Q_BLOCKS = 4
SYN_ATTN_ACQUIRE_ALWAYS = 8
SYN_ATTN_WORK_LIST = 16
SYN_ATTN_WORK_PAIR_MASK = 0x0FFFFFFF
SYN_ATTN_WORK_CONTINUES = 0x10000000
SYN_ATTN_WORK_SOLE_WRITER = 0x20000000
SYN_STATUS_BAD_PAIRING = 2
SYN_STATUS_BAD_CHAIN = 3
SYN_BOX_COPY, SYN_BOX_ADD_ATOMIC, SYN_BOX_ADD_EXCLUSIVE = range(3)
SYN_ELEM_BF16, SYN_ELEM_FP16, SYN_ELEM_FP32, SYN_ELEM_1B, SYN_ELEM_2B, SYN_ELEM_4B, SYN_ELEM_8B = range(7)

_ERRORS = {
    SYN_EINVAL: "SYN_EINVAL (malformed argument or unsupported configuration)",
    SYN_ERANGE: "SYN_ERANGE (wave table addresses tiles or flags outside the operands)",
    SYN_EALIGN: "SYN_EALIGN (pointer or extent not aligned as the kernel needs)",
    SYN_E2BIG: "SYN_E2BIG (more waves than the static counter array of syn_gemm_producer_static holds: "
               f"{SYN_STATIC_MAX_WAVES})",
}


class SyncopateHipError(RuntimeError):
    def __init__(self, fn: str, code: int):
        self.fn = fn
        self.code = code
        what = _ERRORS.get(code, f"hipError_t {code}" if code > 0 else f"error {code}")
        super().__init__(f"{fn} failed: {what}")


class GemmDesc(ctypes.Structure):
    _fields_ = [
        ("a", c_void_p),
        ("b", c_void_p),
        ("c", c_void_p),
        ("flags", c_void_p),
        ("wave_sizes", c_void_p),
        ("wave_offsets", c_void_p),
        ("signal_offsets", c_void_p),
        ("counters", c_void_p),
        ("visit_log", c_void_p),
        ("status", c_void_p),
        ("num_waves", c_int32),
        ("M", c_int32),
        ("N", c_int32),
        ("K", c_int32),
        ("dtype", c_int32),
        ("block_m", c_int32),
        ("block_n", c_int32),
        ("block_k", c_int32),
        ("group_m", c_int32),
        ("num_sms", c_int32),
        ("cum_tiles", c_int64),
        ("spin_timeout_us", c_int64),
        ("options", c_uint32),
    ]


class GemmRemote(ctypes.Structure):
    _fields_ = [
        ("a_peers", c_void_p),
        ("a_target_rank", c_void_p),
        ("c_peers", c_void_p),
        ("c_target_rank", c_void_p),
        ("c_dst_offsets", c_void_p),
        ("c_ld", c_int32),
        ("c_atomic_add", c_int32),
        ("k_ranges", c_void_p),
    ]


class AttnDesc(ctypes.Structure):
    _fields_ = [
        ("q", c_void_p),
        ("k", c_void_p),
        ("v", c_void_p),
        ("o", c_void_p),
        ("lse", c_void_p),
        ("lock", c_void_p),
        ("first", c_void_p),
        ("flags", c_void_p),
        ("wave_offsets", c_void_p),
        ("wave_sizes", c_void_p),
        ("cum_wave_sizes", c_void_p),
        ("signal_offsets", c_void_p),
        ("visit_log", c_void_p),
        ("status", c_void_p),
        ("num_waves", c_int32),
        ("Z", c_int32),
        ("H", c_int32),
        ("Sq", c_int32),
        ("Skv", c_int32),
        ("D", c_int32),
        ("dtype", c_int32),
        ("block_m", c_int32),
        ("block_n", c_int32),
        ("causal", c_int32),
        ("num_programs", c_int32),
        ("sm_scale", c_float),
        ("cum_tiles", c_int64),
        ("spin_timeout_us", c_int64),
        ("q_strides", c_int64 * 3),
        ("k_strides", c_int64 * 3),
        ("v_strides", c_int64 * 3),
        ("o_strides", c_int64 * 3),
        ("counters", c_void_p),
        ("options", c_int32),
        ("wait_flags", c_void_p),
        ("wait_signal_offsets", c_void_p),
        ("work_list", c_void_p),
    ]


# name -> (restype, argtypes); mirrors include/syncopate_hip.h one to one
_SIGNATURES = {
    "syn_gemm_consumer": (c_int32, [POINTER(GemmDesc), c_void_p]),
    "syn_gemm_producer": (c_int32, [POINTER(GemmDesc), c_void_p]),
    "syn_gemm_producer_static": (c_int32, [POINTER(GemmDesc), c_void_p]),
    "syn_gemm_static_counters_peek": (c_int32, [c_void_p, c_int32]),
    "syn_gemm_consumer_producer": (c_int32, [POINTER(GemmDesc), c_void_p, c_void_p, c_void_p]),
    "syn_gemm_remote_binding": (c_int32, [POINTER(GemmDesc), POINTER(GemmRemote), c_void_p]),
    "syn_gemm_check_waves": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_int64, c_int64],
    ),
    "syn_gemm_grid": (c_int32, [c_int64, c_int32, c_int32, c_int32, c_int32, c_int32]),
    "syn_ring_reduce": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int64, c_int64, c_int32, c_int32, c_void_p],
    ),
    "syn_ring_reduce_strided": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_int32, c_int64, c_int64, c_int32, c_int32, c_void_p],
    ),
    "syn_attn_fwd": (c_int32, [POINTER(AttnDesc), c_void_p]),
    "syn_attn_check_work_list": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_int64, c_int32, c_int32],
    ),
    "syn_attn_check_waves": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_int32, c_int64, c_int64],
    ),
    "syn_copy_async": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "syn_copy_kernel_async": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "syn_copy_flag_async": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, ctypes.c_uint64, c_void_p, c_int32,
                                      c_void_p]),
    "syn_copy_flag_list_async": (c_int32, [c_void_p, c_int32, c_void_p, c_int32, c_void_p]),
    "syn_box_copy_async": (c_int32, [c_void_p, c_void_p, c_int32, POINTER(c_int64), POINTER(c_int64),
                                     POINTER(c_int64), c_int32, c_int32, c_int32, c_void_p]),
    "syn_flag_set": (c_int32, [c_void_p, c_uint64, c_void_p]),
    "syn_flag_write_value": (c_int32, [c_void_p, c_uint64, c_void_p]),
    "syn_flag_wait": (c_int32, [c_void_p, c_uint64, c_int64, c_void_p, c_void_p]),
    "syn_delay_us": (c_int32, [c_int64, c_void_p]),
    "syn_stream_create_cu_mask": (c_int32, [POINTER(ctypes.c_uint32), ctypes.c_uint32, POINTER(c_void_p)]),
    "syn_stream_destroy": (c_int32, [c_void_p]),
    "syn_where_async": (c_int32, [c_void_p, c_int32, c_int32, c_void_p]),
    "syn_probe_mfma_rate": (c_int32, [c_void_p, c_int32, c_int32, c_int32, c_void_p]),
    "syn_probe_read_streams": (c_int32, [c_void_p, ctypes.c_int64, ctypes.c_int64, c_int32, c_int32, c_void_p, c_void_p]),
    "syn_probe_read_streams_skewed": (c_int32, [c_void_p, ctypes.c_int64, ctypes.c_int64, c_int32, c_void_p, c_void_p]),
    "syn_probe_attn_slot": (c_int32, [c_void_p, ctypes.c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p]),
    "syn_version": (c_int32, []),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Open the built library (once) and declare every entry point's signature."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m syncopate_amd.build` "
            "(the HIP extension is the only implementation; there is no CPU fallback)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(fn: str, code: int) -> None:
    if code != 0:
        raise SyncopateHipError(fn, int(code))


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return SYN_DTYPE_BF16
    if dtype == torch.float16:
        return SYN_DTYPE_FP16
    raise TypeError(f"unsupported element type {dtype}; the kernels take bfloat16 or float16")


def stream_handle(stream: Optional["torch.cuda.Stream"] = None) -> int:
    s = stream if stream is not None else torch.cuda.current_stream()
    return int(s.cuda_stream)
