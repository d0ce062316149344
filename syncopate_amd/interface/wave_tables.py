"""Host glue: RawSchedule -> the flat wave tables the compute kernels take.

The reference keeps these few lines inside its end-to-end test scripts; here
they are library functions.  All results are plain Python lists (one row per
wave) so that they can be compared, logged, or turned into int32 tensors.

    gemm_consumer_tables      tests/test_ag_gemm_gen.py:137-150
    gemm_producer_tables      tests/test_gemm_rs_transform.py:113-122
    allgather_attn_tables     tests/test_allgather_attn_transform.py:63-84
    all2all_attn_tables       tests/test_all2all_attn_transform.py:58-117
"""

from __future__ import annotations

from typing import Dict, List, NamedTuple, Tuple

from .tile_schedule import RawSchedule


class GemmWaveTables(NamedTuple):
    block_offsets: List[List[int]]   # [num_waves, 2] elements
    block_shapes: List[List[int]]    # [num_waves, 2] elements
    signal_offsets: List[int]        # [num_waves]
    cum_tiles: int                   # sum rows*cols, elements


class AttnWaveTables(NamedTuple):
    wave_offsets: List[List[int]]    # [num_waves, 4] (Z, H, Q, KV), Q/KV in elements
    wave_sizes: List[List[int]]      # [num_waves, 4]
    signal_offsets: List[int]        # [num_waves]
    cum_wave_sizes: List[int]        # inclusive prefix sum of Z*H*Q elements
    cum_tiles: int


def gemm_consumer_tables(schedule: RawSchedule, n_per_rank: int) -> GemmWaveTables:
    """AG+GEMM: the schedule of the gathered A [M, K] names row blocks; the GEMM works on
    C [M, N_per_rank], so the column entry is replaced by the full local N."""
    offsets = schedule.gen_block_offset_lists()
    shapes = schedule.gen_block_shape_lists()
    for off, shape in zip(offsets, shapes):
        off[1] = 0
        shape[1] = n_per_rank
    cum_tiles = sum(int(s[0]) * int(s[1]) for s in shapes)
    return GemmWaveTables(offsets, shapes, schedule.gen_signal_lists(), cum_tiles)


def gemm_producer_tables(schedule: RawSchedule) -> GemmWaveTables:
    """GEMM+RS: the schedule of the partial C [M, N] ("src") is used as it is."""
    shapes = schedule.gen_block_shape_lists()
    cum_tiles = sum(int(s[0]) * int(s[1]) for s in shapes)
    return GemmWaveTables(schedule.gen_block_offset_lists(), shapes, schedule.gen_signal_lists(), cum_tiles)


def plan_layout_spec(layout: str, B: int, H: int, SEQ: int, DIM: int, stacked: int = 2
                     ) -> Tuple[Tuple[int, ...], int, Dict[str, int]]:
    """Shape of the stacked K/V (stacked=2) or Q/K/V (stacked=3) comm buffer, its sequence
    axis, and the axis index of batch / head / seq (tests/test_allgather_attn_transform.py:51-60)."""
    if layout == "bhsd":
        return (stacked, B, H, SEQ, DIM), 3, {"batch": 1, "head": 2, "seq": 3}
    if layout == "bshd":
        return (stacked, B, SEQ, H, DIM), 2, {"batch": 1, "head": 3, "seq": 2}
    raise ValueError(f"Unknown layout {layout}")


def allgather_attn_tables(schedule: RawSchedule, seq_per_rank: int, axes: Dict[str, int]) -> AttnWaveTables:
    """All-gather (swizzle / ring / double ring) of K/V: one wave per arrived KV chunk, all of
    the local Q (seq_per_rank rows) against it."""
    b, h, s = axes["batch"], axes["head"], axes["seq"]
    offsets, sizes, cums, total = [], [], [], 0
    for off, shape in zip(schedule.gen_block_offset_lists(), schedule.gen_block_shape_lists()):
        offsets.append([off[b], off[h], 0, off[s]])
        sizes.append([shape[b], shape[h], seq_per_rank, shape[s]])
        total += shape[b] * shape[h] * seq_per_rank
        cums.append(total)
    return AttnWaveTables(offsets, sizes, schedule.gen_signal_lists(), cums, total)


def all2all_attn_tables(schedule: RawSchedule, axes: Dict[str, int]) -> AttnWaveTables:
    """All-to-all (Ulysses) of stacked Q/K/V: sequence chunk w of Q, K and V arrives with
    wave w.  Arrival w unlocks (Q_w x KV_w), and for every earlier p: (Q_p x KV_w) and
    (Q_w x KV_p) — all gated by wave w's flag:

            KV_0 KV_1 KV_2
        Q_0   0    1    2
        Q_1   1    1    2
        Q_2   2    2    2
    """
    b, h, s = axes["batch"], axes["head"], axes["seq"]
    src_offsets = schedule.gen_block_offset_lists()
    src_shapes = schedule.gen_block_shape_lists()
    src_signals = schedule.gen_signal_lists()
    offsets, sizes, signals, cums, total = [], [], [], [], 0

    def emit(q_wave: int, kv_wave: int, gate: int, batch_head_from: int, count_q_from: int) -> None:
        nonlocal total
        o_bh, s_bh = src_offsets[batch_head_from], src_shapes[batch_head_from]
        offsets.append([o_bh[b], o_bh[h], src_offsets[q_wave][s], src_offsets[kv_wave][s]])
        sizes.append([s_bh[b], s_bh[h], src_shapes[q_wave][s], src_shapes[kv_wave][s]])
        signals.append(src_signals[gate])
        total += s_bh[b] * s_bh[h] * src_shapes[count_q_from][s]
        cums.append(total)

    for w in range(len(src_shapes)):
        emit(w, w, w, w, w)
        for p in range(w):
            # the reference counts the programs of both cross terms with the other chunk's
            # length (test_all2all_attn_transform.py:103,110); equal for uniform chunks
            emit(p, w, w, p, w)
            emit(w, p, w, p, p)
    return AttnWaveTables(offsets, sizes, signals, cums, total)


def attn_producer_tables(schedule: RawSchedule, axes: Dict[str, int], kv_len: int) -> AttnWaveTables:
    """Attention that PRODUCES the source of an all-to-all along the sequence axis: one wave per
    outgoing sequence chunk of the output, every q block of it against the whole K/V; the signals
    are the COMPUTE_DONE flags the kernel sets (tests/test_attn_all2all_transform.py:57-85)."""
    b, h, s = axes["batch"], axes["head"], axes["seq"]
    offsets, sizes, cums, total = [], [], [], 0
    for off, shape in zip(schedule.gen_block_offset_lists(), schedule.gen_block_shape_lists()):
        offsets.append([off[b], off[h], off[s], 0])
        sizes.append([shape[b], shape[h], shape[s], kv_len])
        total += shape[b] * shape[h] * shape[s]
        cums.append(total)
    return AttnWaveTables(offsets, sizes, schedule.gen_signal_lists(), cums, total)
