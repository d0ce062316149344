"""Tile-visit order of the chunk-scheduled kernels, restated on the CPU (oracle: test infrastructure).

Follows the reference's device index math:
  * get_pid_mn                syncopate/computation/gemm/template.py:10-18
  * persistent wave walk      syncopate/computation/gemm/template.py:69-136
                              (generated twin: transform/transformer.py:759-879)
  * attention wave lookup     syncopate/computation/attn/template.py:39-44,80-121
                              (generated twin: transform/transformer.py:555-660)
"""

from __future__ import annotations

from typing import Dict, List, Sequence, Tuple


def get_pid_mn(tile_id: int, num_pid_m: int, num_pid_n: int, group_size_m: int) -> Tuple[int, int]:
    """Grouped ordering inside one wave (template.py:10-18)."""
    num_pid_in_group = group_size_m * num_pid_n
    group_id = tile_id // num_pid_in_group
    first_pid_m = group_id * group_size_m
    size_m = min(num_pid_m - first_pid_m, group_size_m)
    pid_m = first_pid_m + (tile_id % size_m)
    pid_n = (tile_id % num_pid_in_group) // size_m
    return pid_m, pid_n


def gemm_num_tiles(cum_tiles: int, M: int, N: int, BM: int, BN: int) -> int:
    """cdiv(cum_tiles, BM*BN) when cum_tiles is given, else the full grid
    (transform/transformer.py:1003-1031)."""
    if cum_tiles:
        return -(-cum_tiles // (BM * BN))
    return (-(-M // BM)) * (-(-N // BN))


def gemm_tile_visits(
    wave_sizes: Sequence[Sequence[int]],
    wave_offsets: Sequence[Sequence[int]],
    signal_offsets: Sequence[int],
    *,
    M: int,
    N: int,
    BM: int,
    BN: int,
    group_m: int,
    num_sms: int,
    cum_tiles: int = 0,
) -> List[Dict[str, int]]:
    """For every tile id, in tile-id order: which program visits it, at which
    iteration, in which wave, which (pid_m, pid_n) it is, and which flag (if any)
    the program waits on just before it (template.py:69-136).

    Sizes and offsets are in elements and are floor-divided by the block sizes,
    as the kernel does (template.py:82-87,113-116).
    """
    num_tiles = gemm_num_tiles(cum_tiles, M, N, BM, BN)
    grid = min(num_sms, num_tiles)
    visits: List[Dict[str, int]] = [dict() for _ in range(num_tiles)]
    for pid in range(grid):
        tiles_here = num_tiles // num_sms + (1 if pid < num_tiles % num_sms else 0)
        wave = 0
        past = 0
        cur_m = wave_sizes[0][0] // BM
        cur_n = wave_sizes[0][1] // BN
        off_m = wave_offsets[0][0] // BM
        off_n = wave_offsets[0][1] // BN
        cur_tiles = cur_m * cur_n
        sig = signal_offsets[0]
        # the program waits on wave 0's flag before its loop (template.py:90-97)
        pending_wait = sig if sig >= 0 else -1
        for it in range(tiles_here):
            tile_id = pid + it * num_sms
            new_wave = False
            while tile_id >= past + cur_tiles:
                past += cur_tiles
                wave += 1
                cur_m = wave_sizes[wave][0] // BM
                cur_n = wave_sizes[wave][1] // BN
                off_m = wave_offsets[wave][0] // BM
                off_n = wave_offsets[wave][1] // BN
                cur_tiles = cur_m * cur_n
                sig = signal_offsets[wave]
                new_wave = True
            waited = pending_wait
            pending_wait = -1
            if new_wave and sig >= 0:
                waited = sig
            pm, pn = get_pid_mn(tile_id - past, cur_m, cur_n, group_m)
            visits[tile_id] = {
                "tile_id": tile_id,
                "pid": pid,
                "iter": it,
                "wave": wave,
                "pid_m": pm + off_m,
                "pid_n": pn + off_n,
                "waited_signal": waited,
            }
    return visits


def attn_tile_work(
    tile_id: int,
    wave_offsets: Sequence[Sequence[int]],
    wave_sizes: Sequence[Sequence[int]],
    cum_wave_sizes: Sequence[int],
    signal_offsets: Sequence[int],
    *,
    block_m: int = 128,
    block_n: int = 128,
) -> Dict[str, int]:
    """tile id -> (wave, z, h, q block, kv block range, signal); generated-kernel
    units: Q/KV entries in elements, cum in Z*H*Q elements
    (transform/transformer.py:561-601; template.py:80-121 with get_pid_range :39-44).
    """
    wave = None
    for i, cum in enumerate(cum_wave_sizes):
        if cum // block_m > tile_id:
            wave = i
            break
    if wave is None:
        raise IndexError(f"tile id {tile_id} is beyond the last wave")
    prev = 0 if wave == 0 else cum_wave_sizes[wave - 1] // block_m
    t = tile_id - prev
    size_z, size_h, size_q, size_kv = wave_sizes[wave]
    off_z, off_h, off_q, off_kv = wave_offsets[wave]
    nq = size_q // block_m
    q = t % nq
    h = (t // nq) % size_h
    z = t // (nq * size_h)
    kv_lo = off_kv // block_n
    return {
        "wave": wave,
        "z": z + off_z,
        "h": h + off_h,
        "q_block": q + off_q // block_m,
        "kv_lo": kv_lo,
        "kv_hi": kv_lo + size_kv // block_n,
        "signal": signal_offsets[wave],
    }
