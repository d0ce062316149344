"""Which tile shape the chunk-scheduled GEMM should run on, given how the chunks arrive.

The reference fixes the shape at the call site (BLOCK_SIZE_M/N kwargs; 128x256 by default,
syncopate/computation/gemm/template.py:193-220) and sweeps it by hand
(tests/test_ag_gemm_tile_size_sensitivity.py).  Here the same kwargs exist; this module picks them.

Two regimes:

* The chunks arrive faster than the GEMM eats them (copies at HBM speed, or everything resident).  The step is
  the kernel, and the fastest kernel wins: 256x256 tiles (the least LDS traffic per product).
* The chunks arrive slower than the GEMM eats them (one xGMI link per peer: 16.8 MB in ~110 us against ~45 us of
  GEMM per chunk).  The step is the producer plus what is left to compute when the LAST chunk has landed, and that
  is `rounds x tile time`: the last chunk's tiles on `programs` programs.  A 256x256 tile of K = 8192 takes a
  compute unit ~165 us and the last chunk's 56 tiles keep 56 of 224 programs busy for all of it; 128x128 tiles are
  224 per chunk - one full round - and 256x128 tiles are 112, half a round of a tile that takes ~65 us.  The wave order exists for this regime
  (gemm/template.py:69-136): the shape has to let a wave fill the machine.
"""

from __future__ import annotations

from typing import Iterable, Optional, Tuple

# Cost of one round of tiles of each shape (K = 8192, microseconds; only the ratios matter).
# RESIDENT_COST: every program busy - from the resident 8192 x 8192 x 3584 GEMM on 224 programs (256x256: 2 rounds in
# 326 us; 128x256 / 256x128: 4 rounds in 376 / 367 us; 128x128: 8 rounds in 540 us).
# LAST_ROUND_COST: the round that is left when the last chunk lands - measured as the step's time beyond the
# producer's with one link's delay per chunk (209 / 88 / 85 / 92 us, of which ~20 us are the flag's way to the
# kernel, the epilogue and the stream join).  Half-empty rounds run faster than full ones: the idle compute units
# leave their share of the power budget and of the memory system to the busy ones.
RESIDENT_COST = {(256, 256): 163.0, (128, 256): 94.0, (256, 128): 92.0, (128, 128): 67.5}
LAST_ROUND_COST = {(256, 256): 189.0, (128, 256): 68.0, (256, 128): 65.0, (128, 128): 72.0}
TILE_COST = RESIDENT_COST


def rounds(rows: int, cols: int, bm: int, bn: int, programs: int) -> int:
    tiles = (rows // bm) * (cols // bn)
    return -(-tiles // programs)


def choose_tile(chunk_rows: int, n: int, programs: int, *, producer_bound: bool,
                shapes: Optional[Iterable[Tuple[int, int]]] = None) -> Tuple[int, int]:
    """(BLOCK_SIZE_M, BLOCK_SIZE_N) for a GEMM whose A arrives in chunks of `chunk_rows` rows against N = `n`.

    `producer_bound`: the chunks arrive slower than the GEMM consumes them.  Then the shape with the shortest
    `rounds(last chunk) x tile cost` that divides the chunk is taken; otherwise the shape with the lowest cost per
    element, 256x256.
    """
    candidates = [s for s in (shapes or TILE_COST) if chunk_rows % s[0] == 0 and n % s[1] == 0]
    if not candidates:
        raise ValueError(f"no tile shape divides a chunk of {chunk_rows} rows x {n} columns")
    if not producer_bound:
        return min(candidates, key=lambda s: RESIDENT_COST[s] / (s[0] * s[1]))

    def left_over(s):
        r = rounds(chunk_rows, n, s[0], s[1], programs)
        return (r - 1) * RESIDENT_COST[s] + LAST_ROUND_COST[s]

    return min(candidates, key=lambda s: (left_over(s), -s[0] * s[1]))


def choose_xcd_remap(bm: int, bn: int) -> bool:
    """Whether the programs of one XCD should take consecutive tiles (SYN_GEMM_XCD_REMAP), for a launcher that was not
    told.  Measured on the resident 8192 x 8192 x 3584 consumer: 128x256, 256x128 and 128x128 tiles gain 4-10 % from
    the remap (224 programs: 373 / 369 / 502 us against 409 / 385 / 559); 256x256 tiles gain nothing on 224 programs
    (340 either way) and LOSE 9 % on 256 (365 against 336 us); the 8192 x 8192 x 3584 producer on 256x256 tiles is
    the same either way (335 us)."""
    return (bm, bn) != (256, 256)
