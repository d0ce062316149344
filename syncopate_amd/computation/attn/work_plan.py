"""Work lists for the paired attention kernel (SYN_ATTN_WORK_LIST): which program visits which tiles.

The wave tables fix what a tile IS - tile id -> (wave, z, h, q block, kv range), the reference's mapping
(syncopate/computation/attn/template.py:39-44, 80-121).  The reference leaves which program runs a tile to
the hardware's workgroup scheduler (one program per tile, `grid = cum_tiles / BLOCK_M`,
tests/test_all2all_attn_transform.py:120-146).  A persistent launch has to choose, and the choice decides
three things at once:

* balance - under a causal mask the visits of the all-to-all table differ in cost by a factor of eight
  (a visit ends at the diagonal) and a quarter of them cost nothing;
* how often a pair of q blocks is merged into the output - visits to the same q blocks that one program makes
  in a row are one SEGMENT: the running maxima, sums and output stay in registers, and the q blocks are merged
  (or, if no other segment writes them, simply stored) once;
* what a program can do while a chunk has not arrived - a program makes its visits in list order and waits for
  each visit's flag, so a list follows the order of the waves.

`plan_attention_work` cuts every q-block pair's visits (in table order) into segments no longer than asked,
places the segments on programs - longest first onto the least loaded program, a head's segments on that head's
share of the programs - and orders each program's segments by wave.  Everything here is host logic on plain integers; the result is the int32
word list of include/syncopate_hip.h (SYN_ATTN_WORK_LIST).
"""

from __future__ import annotations

import heapq
from typing import Dict, List, NamedTuple, Optional, Sequence, Tuple

WORK_PAIR_MASK = 0x0FFFFFFF
WORK_CONTINUES = 0x10000000
WORK_SOLE_WRITER = 0x20000000


class Visit(NamedTuple):
    pair: int            # tiles 2 * pair and 2 * pair + 1
    wave: int
    key: Tuple[int, int, int]     # (z, h, lower q block)
    kv_blocks: int       # kv blocks the pair walks (0: wholly above the diagonal)


class WorkPlan(NamedTuple):
    words: List[int]                 # num_programs + 1 offsets, then the entries
    num_programs: int
    program_entries: List[List[int]]   # the entries per program (flag bits included)
    program_cost: List[int]          # kv blocks per program
    segments: int
    merged_segments: int             # segments that share their q blocks with another one


def table_visits(wave_offsets: Sequence[Sequence[int]], wave_sizes: Sequence[Sequence[int]],
                 cum_wave_sizes: Sequence[int], *, causal: bool, block_m: int = 128, block_n: int = 128
                 ) -> List[Visit]:
    """Every pair of tiles of the table with what it costs; ValueError for tables the paired kernel does not take."""
    visits: List[Visit] = []
    prev = 0
    for w, cum in enumerate(cum_wave_sizes):
        cum = int(cum)
        if cum == 0:
            break                       # zero rows pad the end of a table
        first_tile, tiles = prev // block_m, (cum - prev) // block_m
        prev = cum
        off, size = [int(x) for x in wave_offsets[w]], [int(x) for x in wave_sizes[w]]
        nq, size_h = size[2] // block_m, size[1]
        if nq % 2 or first_tile % 2:
            raise ValueError(f"wave {w}: the paired kernel needs an even number of q blocks per wave")
        lo, length = off[3] // block_n, size[3] // block_n
        if causal and (lo % 2 or (off[2] // block_m) % 2):
            raise ValueError(f"wave {w}: under a causal mask q and kv ranges must begin at even blocks")
        for t in range(0, tiles, 2):
            z = t // (nq * size_h) + off[0]
            h = (t // nq) % size_h + off[1]
            qb = t % nq + off[2] // block_m
            walked = min(length, qb + 2 - lo) if causal else length
            visits.append(Visit((first_tile + t) // 2, w, (z, h, qb), max(walked, 0)))
    return visits


def plan_attention_work(wave_offsets, wave_sizes, cum_wave_sizes, *, causal: bool, num_programs: int,
                        max_visits: Optional[int] = None, max_blocks: Optional[float] = None,
                        group_heads: bool = True, list_masked_visits: bool = False,
                        segment_overhead: float = 1.0, merge_overhead: float = 3.0,
                        block_m: int = 128, block_n: int = 128) -> WorkPlan:
    """The work list for `num_programs` programs (see the module text).

    `max_visits`: longest segment in visits (None: no limit).
    `max_blocks`: longest segment in kv blocks; "fair" = a program's fair share of all kv blocks (None: no limit).
    A pair of q blocks whose visits exceed a limit is cut from its LAST visit backwards into pieces as long as the
    limits allow, the remainder at the front (under a causal mask the front holds the short visit on the diagonal:
    the pieces are whole, the remainders come in all sizes and fill the programs up).
    `group_heads`: where the programs divide evenly among the (z, h) of the table, each gets a run of neighbouring
    programs - under the XCD remap one or a few XCDs, through whose L2 that head's K and V then pass.
    `list_masked_visits`: also list the visits that lie wholly above a causal diagonal (they are then logged in
    the visit log and skipped); left out otherwise.
    `segment_overhead`, `merge_overhead`: what a segment costs beyond its kv blocks, in kv blocks - its start
    (flag, Q, first fills) and, for a segment that shares its q blocks, the merge under their locks.
    """
    if num_programs <= 0:
        raise ValueError("num_programs must be positive")
    visits = table_visits(wave_offsets, wave_sizes, cum_wave_sizes, causal=causal, block_m=block_m, block_n=block_n)
    chains: Dict[Tuple[int, int, int], List[Visit]] = {}
    masked: List[Visit] = []
    for v in visits:
        if v.kv_blocks == 0:
            masked.append(v)
        else:
            chains.setdefault(v.key, []).append(v)
    if max_blocks == "fair":
        max_blocks = sum(v.kv_blocks for v in visits) / num_programs

    segments: List[List[Visit]] = []
    shared: Dict[Tuple[int, int, int], bool] = {}
    for key, chain in chains.items():
        pieces: List[List[Visit]] = []
        piece: List[Visit] = []
        blocks = 0
        for v in reversed(chain):
            if piece and ((max_visits is not None and len(piece) >= max_visits) or
                          (max_blocks is not None and blocks + v.kv_blocks > max_blocks)):
                pieces.append(piece[::-1])
                piece, blocks = [], 0
            piece.append(v)
            blocks += v.kv_blocks
        pieces.append(piece[::-1])
        segments.extend(reversed(pieces))
        shared[key] = len(pieces) > 1

    def cost(seg: List[Visit]) -> float:
        return sum(v.kv_blocks for v in seg) + segment_overhead + (merge_overhead if shared[seg[0].key] else 0.0)

    # which programs a segment may go to: its head's share of them, or all
    heads = sorted({key[:2] for key in chains})
    if group_heads and heads and num_programs % len(heads) == 0:
        share = num_programs // len(heads)
        pool_of = {head: n for n, head in enumerate(heads)}
        heaps = [[(0.0, p) for p in range(n * share, (n + 1) * share)] for n in range(len(heads))]
    else:
        pool_of = {head: 0 for head in heads}
        heaps = [[(0.0, p) for p in range(num_programs)]]

    # longest first onto the least loaded program of the pool; ties go to the lower program id, so that the
    # equally long segments of one wave (consecutive pairs) end up side by side, at the same place in their lists
    order = sorted(range(len(segments)), key=lambda i: (-cost(segments[i]), segments[i][0].pair))
    placed: List[List[int]] = [[] for _ in range(num_programs)]
    for i in order:
        heap = heaps[pool_of[segments[i][0].key[:2]]]
        load, p = heapq.heappop(heap)
        placed[p].append(i)
        heapq.heappush(heap, (load + cost(segments[i]), p))

    program_entries: List[List[int]] = []
    program_cost: List[int] = []
    for p in range(num_programs):
        mine = sorted(placed[p], key=lambda i: (segments[i][0].wave, segments[i][0].pair))
        entries: List[int] = []
        for i in mine:
            seg = segments[i]
            for n, v in enumerate(seg):
                word = v.pair
                if n + 1 < len(seg):
                    word |= WORK_CONTINUES
                if n == 0 and not shared[v.key]:
                    word |= WORK_SOLE_WRITER
                entries.append(word)
        program_entries.append(entries)
        program_cost.append(sum(v.kv_blocks for i in mine for v in segments[i]))
    if list_masked_visits:
        # dealt round-robin; kept in wave order inside each program's list by a stable merge on the wave index
        for n, v in enumerate(masked):
            program_entries[n % num_programs].append(v.pair)
        wave_of = {v.pair: v.wave for v in visits}
        for p in range(num_programs):
            program_entries[p] = _merge_by_wave(program_entries[p], wave_of)

    words: List[int] = [0]
    for entries in program_entries:
        words.append(words[-1] + len(entries))
    for entries in program_entries:
        words.extend(entries)
    return WorkPlan(words, num_programs, program_entries, program_cost, len(segments),
                    sum(1 for seg in segments if shared[seg[0].key]))


def _merge_by_wave(entries: List[int], wave_of: Dict[int, int]) -> List[int]:
    """Order a program's entries by the wave of each SEGMENT's first visit, keeping segments whole."""
    groups: List[List[int]] = []
    open_group = False
    for word in entries:
        if open_group:
            groups[-1].append(word)
        else:
            groups.append([word])
        open_group = bool(word & WORK_CONTINUES)
    groups.sort(key=lambda g: wave_of[g[0] & WORK_PAIR_MASK])
    return [word for g in groups for word in g]
