"""Launchers of the chunked-KV flash-attention kernel (MI355X HIP, through the C ABI).

Two call forms, as in the reference:

* ``attention(q, k, v, sm_scale, wave_dicts)`` — the hand-written template's
  launcher (syncopate/computation/attn/template.py:366-439).  Table entries
  along Q and KV are in BLOCKS, `cum_wave_sizes` counts programs, tables may be
  padded with zero rows to a power of two (template.py:567-641).
* ``attention_forward(q, k, v, sm_scale, *, wave_offsets, wave_sizes,
  cum_wave_sizes, signal_ptr, signal_offsets, NUM_WAVES, cum_tiles)`` — the
  launcher the transform pass generates (syncopate/computation/transform/
  transformer.py:1125-1137; used in tests/test_allgather_attn_transform.py:206-214).
  Table entries along Q and KV are in ELEMENTS and `cum_wave_sizes`/`cum_tiles`
  count Z*H*Q elements.

Layout: q, o [Z, H, Sq, D]; k, v [Z, H, Skv, D] ("bhsd", the default), or q, o [Z, Sq, H, D];
k, v [Z, Skv, H, D] ("bshd", the reference's example_attn_bshd.py); D = 128 contiguous; bf16 or
fp16.  Views with other batch / head / row strides (slices of a stacked comm buffer) are fine.
"""

from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from ... import _lib
from .._launch import (
    acquire_always,
    recall_note,
    remember_note,
    TableLike,
    already_checked,
    as_device_table,
    flag_buffer,
    host_copy,
    host_ptr,
    launches_on_stream,
    zeroed_int32,
    remember_checked,
    require_cuda,
    status_words,
)

from .work_plan import WorkPlan, plan_attention_work

BLOCK_M = 128
BLOCK_N = 128
DEFAULT_SPIN_TIMEOUT_US = 2_000_000


@launches_on_stream
def attention_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sm_scale: float,
    *,
    wave_offsets: TableLike,
    wave_sizes: TableLike,
    cum_wave_sizes: TableLike,
    signal_ptr: torch.Tensor,
    signal_offsets: TableLike,
    NUM_WAVES: Optional[int] = None,
    cum_tiles: Optional[int] = None,
    causal: bool = False,
    layout: str = "bhsd",
    num_programs: int = 0,
    counter_ptr: Optional[torch.Tensor] = None,
    output_buffer: Optional[torch.Tensor] = None,
    consumer_signal_ptr: Optional[torch.Tensor] = None,
    consumer_signal_offsets: Optional[TableLike] = None,
    pair_q_blocks: bool = False,
    xcd_remap: bool = False,
    chain_q_blocks: bool = False,
    work_plan: Optional[WorkPlan] = None,
    form: str = "explicit",
    out: Optional[torch.Tensor] = None,
    return_lse: bool = False,
    visit_log: Optional[torch.Tensor] = None,
    spin_timeout_us: int = DEFAULT_SPIN_TIMEOUT_US,
    stream: Optional[torch.cuda.Stream] = None,
):
    """Chunk-gated attention forward; returns o (and the base-2 lse if asked).

    `causal` is an extension over the reference (which is non-causal): kv blocks
    above the diagonal are skipped, the diagonal block is masked.
    `num_programs` > 0 runs that many persistent workgroups over the tile ids
    instead of one workgroup per tile.
    `counter_ptr` (int32, one zeroed word per wave) selects the producer form the transform
    pass generates for attention that feeds an all-to-all
    (tests/test_attn_all2all_transform.py:182-214): no flag is waited for; every finished tile
    bumps its wave's counter and the tile that completes a wave sets the wave's flag in
    `signal_ptr`.  `output_buffer` (alias of `out`) is the reference's name for the comm buffer
    the result is written into.
    `consumer_signal_ptr` / `consumer_signal_offsets` (with `counter_ptr`): a second flag array
    and the index per wave (-1: none) that the producer form waits for before it reads a wave's K
    and V - the transform pass with both roles enabled (tests/test_all2all_attn_all2all.py:192-210).
    `pair_q_blocks` (an extension): one workgroup of eight wavefronts takes two consecutive q
    blocks and runs them half a kv block apart, the softmax of one beside the matrix products of
    the other, both reading K and V from the same LDS blocks.  Every wave must hold an even
    number of q blocks (with `causal`: q and kv ranges that begin at even blocks); not with `counter_ptr`.
    `xcd_remap` (an extension): the workgroups of one XCD take consecutive tiles (the q blocks of
    one head), so that a head's K and V are fetched into one L2 instead of eight.
    `chain_q_blocks` (an extension, with `pair_q_blocks`): for tables whose waves all list the same
    (z, h, q) ranges and differ in the kv range and the flag only (the all-gather attention).  With
    as many programs as a wave has pairs of q blocks - `num_programs` must be that number, or 0 to
    have it filled in - a program's tiles are one pair of q blocks in wave after wave, so it keeps
    the running maxima, sums and output in registers from one wave's kv range to the next (each
    behind its flag) and writes every q block once, without locks or merges.  Programs, tiles and
    their order are those of the persistent launch with that `num_programs`.  A ValueError for
    tables of another shape.
    `work_plan` (an extension, with `pair_q_blocks`; `plan_attention_work` makes one): which program visits which
    tiles, in which order, and which consecutive visits to the same q blocks are one segment whose sums stay in
    registers (include/syncopate_hip.h, SYN_ATTN_WORK_LIST).  `num_programs` is the plan's.  The tile -> work
    mapping is the tables'; the visit log shows on which program each tile ran.
    `form="auto"` (what `attention()` passes): where none of the three options above, `causal`, `counter_ptr` or
    `visit_log` is given, the launcher reads the tables and takes the fastest form they allow - two q blocks per
    workgroup with the XCD remap where every wave holds an even number of q blocks, chained where the waves
    also share their (z, h, q) ranges and `num_programs` is 0 or the pairs of a wave.  Where the waves cover
    different q ranges (the all-to-all table), and with `causal` (and none of the other options), it plans the
    visits itself where the tables pair up: `plan_attention_work` for one program per compute unit (or
    `num_programs`), segments cut to a program's fair share of the kv blocks; the plan is remembered with the
    caller's device tables.  Results are the same
    to rounding; what differs is which program a tile runs on, which only `visit_log` shows.
    """
    dev = require_cuda(q, k, v, signal_ptr)
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("q, k and v must share one element type")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be 4-D")
    if layout not in ("bhsd", "bshd"):
        raise ValueError(f"Unknown layout {layout}")
    HEAD_DIM_Q, HEAD_DIM_K, HEAD_DIM_V = q.shape[-1], k.shape[-1], v.shape[-1]
    assert HEAD_DIM_Q == HEAD_DIM_K and HEAD_DIM_K == HEAD_DIM_V
    if HEAD_DIM_K != 128:
        raise ValueError("the gfx950 kernel is specialised for head_dim 128")
    h_ax, s_ax = (1, 2) if layout == "bhsd" else (2, 1)
    Z, H, Sq, D = q.shape[0], q.shape[h_ax], q.shape[s_ax], q.shape[3]
    if (k.shape[0], k.shape[h_ax]) != (Z, H) or v.shape != k.shape:
        raise ValueError("k and v must have q's batch and head extents and one shape")
    Skv = k.shape[s_ax]

    def strides(t: torch.Tensor):
        if t.stride(3) != 1 or any(t.stride(ax) % 8 for ax in (0, 1, 2)):
            raise ValueError("the head dimension must be contiguous and rows 16-byte aligned")
        return (ctypes.c_int64 * 3)(t.stride(0), t.stride(h_ax), t.stride(s_ax))

    flags = flag_buffer(signal_ptr)

    offs = as_device_table(wave_offsets, dev, 4)
    sizes = as_device_table(wave_sizes, dev, 4)
    cums = as_device_table(cum_wave_sizes, dev, None)
    sigs = as_device_table(signal_offsets, dev, None)
    num_waves = cums.numel() if NUM_WAVES is None else int(NUM_WAVES)
    if min(offs.shape[0], sizes.shape[0], cums.numel(), sigs.numel()) < num_waves:
        raise ValueError("wave tables are shorter than NUM_WAVES")

    lib = _lib.load()
    tables = (wave_offsets, wave_sizes, cum_wave_sizes, signal_offsets)   # the caller's objects
    caller_owned = all(isinstance(t, torch.Tensor) and t.is_cuda
                       for t in (wave_offsets, wave_sizes, cum_wave_sizes, signal_offsets))
    if pair_q_blocks and counter_ptr is not None:
        raise ValueError("pair_q_blocks does not go with counter_ptr")
    if chain_q_blocks and not pair_q_blocks:
        raise ValueError("chain_q_blocks goes with pair_q_blocks")
    if chain_q_blocks and causal:
        raise ValueError("chain_q_blocks does not go with causal: plan the visits with plan_attention_work")
    if work_plan is not None and (not pair_q_blocks or chain_q_blocks):
        raise ValueError("work_plan goes with pair_q_blocks and without chain_q_blocks")
    num_programs = int(num_programs)
    if work_plan is not None:
        if num_programs not in (0, work_plan.num_programs):
            raise ValueError(f"the work plan is for {work_plan.num_programs} programs")
        num_programs = work_plan.num_programs
    host_tables = None
    if form not in ("explicit", "auto"):
        raise ValueError("form must be 'explicit' or 'auto'")
    def planned_by_the_launcher(with_mask: bool):
        """A work plan for these tables (one program per compute unit, or `num_programs`; segments cut to a program's
        fair share of the kv blocks), remembered with the caller's device tables; False where the tables do not pair up."""
        nonlocal host_tables
        units = num_programs or torch.cuda.get_device_properties(dev).multi_processor_count
        note = f"work plan, causal {int(with_mask)}, {units} programs"
        plan = recall_note(tables, note) if caller_owned else None
        if plan is None:
            host_tables = host_tables or (host_copy(offs), host_copy(sizes), host_copy(cums), host_copy(sigs))
            try:
                plan = plan_attention_work(host_tables[0][:num_waves].tolist(), host_tables[1][:num_waves].tolist(),
                                           host_tables[2][:num_waves].tolist(), causal=with_mask, num_programs=units,
                                           max_blocks="fair")
            except ValueError:
                plan = False
            if caller_owned:
                remember_note(tables, note, plan)
        return plan

    if form == "auto" and causal and not (pair_q_blocks or chain_q_blocks or xcd_remap or counter_ptr is not None
                                          or consumer_signal_ptr is not None or visit_log is not None
                                          or work_plan is not None):
        # under a causal mask the visits differ in cost and many cost nothing: a planned launch where the tables pair
        # up, the one-tile-per-program kernel where they do not
        plan = planned_by_the_launcher(True)
        if plan:
            pair_q_blocks = xcd_remap = True
            work_plan, num_programs = plan, plan.num_programs
    if form == "auto" and not (pair_q_blocks or chain_q_blocks or xcd_remap or causal or counter_ptr is not None
                               or consumer_signal_ptr is not None or visit_log is not None):
        choice = recall_note(tables, "attention form") if caller_owned else None
        if choice is None:
            host_tables = host_tables or (host_copy(offs), host_copy(sizes), host_copy(cums), host_copy(sigs))
            ho, hs, hc, _ = host_tables
            real = [i for i in range(num_waves) if int(hc[i]) > 0]
            even = bool(real) and all(int(hs[i, 2]) % (2 * BLOCK_M) == 0 for i in real)
            same = even and all(ho[i, :3].tolist() == ho[real[0], :3].tolist() and
                                hs[i, :3].tolist() == hs[real[0], :3].tolist() for i in real)
            pairs = int(hs[real[0], 0]) * int(hs[real[0], 1]) * int(hs[real[0], 2]) // (2 * BLOCK_M) if same else 0
            choice = (even, pairs)
            if caller_owned:
                remember_note(tables, "attention form", choice)
        even, pairs = choice
        if even:
            pair_q_blocks = xcd_remap = True
            if pairs and num_programs in (0, pairs):
                chain_q_blocks, num_programs = True, pairs
            elif not pairs:
                # waves over different q ranges (the all-to-all table): the visits to a pair of q blocks are planned as
                # segments that keep their sums in registers, instead of one merge into the output per visit
                plan = planned_by_the_launcher(False)
                if plan:
                    work_plan, num_programs = plan, plan.num_programs
    given_programs = num_programs
    if chain_q_blocks and num_programs <= 0 and caller_owned:
        # filled in by an earlier call on these tables; `already_checked` below vouches for it
        num_programs = recall_note(tables, "chain programs") or 0
    params = (num_waves, Z, H, Sq, Skv, cum_tiles, flags.numel(), bool(pair_q_blocks), bool(causal),
              None if work_plan is None else id(work_plan), num_programs if chain_q_blocks else None)
    if cum_tiles is None or (chain_q_blocks and num_programs <= 0) or \
            not (caller_owned and already_checked(tables, params)):
        ho, hs, hc, hg = host_tables or (host_copy(offs), host_copy(sizes), host_copy(cums), host_copy(sigs))
        if cum_tiles is None:
            cum_tiles = int(hc[:num_waves].max().item())
        if pair_q_blocks and any(int(hs[i, 2]) % (2 * BLOCK_M) for i in range(num_waves) if int(hc[i]) > 0):
            raise ValueError("pair_q_blocks needs an even number of q blocks in every wave")
        if pair_q_blocks and causal and any(int(ho[i, 2]) % (2 * BLOCK_M) or int(ho[i, 3]) % (2 * BLOCK_N)
                                            for i in range(num_waves) if int(hc[i]) > 0):
            raise ValueError("pair_q_blocks with causal needs q and kv ranges that begin at even blocks")
        if work_plan is not None:
            words = torch.tensor(work_plan.words, dtype=torch.int32)
            _lib.check(
                "syn_attn_check_work_list",
                lib.syn_attn_check_work_list(host_ptr(ho), host_ptr(hs), host_ptr(hc), num_waves, BLOCK_M, BLOCK_N,
                                             1 if causal else 0, host_ptr(words), words.numel(),
                                             work_plan.num_programs, 1 if visit_log is not None and causal else 0),
            )
        if chain_q_blocks:
            real = [i for i in range(num_waves) if int(hc[i]) > 0]
            if not real or any(ho[i, :3].tolist() != ho[real[0], :3].tolist() or
                               hs[i, :3].tolist() != hs[real[0], :3].tolist() for i in real):
                raise ValueError("chain_q_blocks needs the same (z, h, q) ranges in every wave")
            pairs = int(hs[real[0], 0]) * int(hs[real[0], 1]) * int(hs[real[0], 2]) // (2 * BLOCK_M)
            if given_programs <= 0:
                num_programs = pairs
            elif num_programs != pairs:
                raise ValueError(f"chain_q_blocks needs num_programs = {pairs}, the pairs of q blocks of one wave")
            params = params[:-1] + (num_programs,)
            if caller_owned:
                remember_note(tables, "chain programs", num_programs)
        _lib.check(
            "syn_attn_check_waves",
            lib.syn_attn_check_waves(host_ptr(ho), host_ptr(hs), host_ptr(hc), host_ptr(hg), num_waves,
                                     Z, H, Sq, Skv, BLOCK_M, BLOCK_N, int(cum_tiles), flags.numel()),
        )
        if caller_owned:
            remember_checked(tables, params[:5] + (cum_tiles,) + params[6:])

    if output_buffer is not None:
        if out is not None and out is not output_buffer:
            raise ValueError("give out or output_buffer, not both")
        out = output_buffer
    if counter_ptr is not None:
        if counter_ptr.dtype != torch.int32 or counter_ptr.device != dev or not counter_ptr.is_contiguous() \
                or counter_ptr.numel() < num_waves:
            raise ValueError("counter_ptr must be a contiguous int32 tensor with one word per wave on q's device")
    wait_flags = wait_sigs = None
    if (consumer_signal_ptr is None) != (consumer_signal_offsets is None):
        raise ValueError("consumer_signal_ptr and consumer_signal_offsets go together")
    if consumer_signal_ptr is not None:
        if counter_ptr is None:
            raise ValueError("without counter_ptr, signal_ptr itself is what the kernel waits for")
        wait_flags = flag_buffer(consumer_signal_ptr)
        wait_sigs = as_device_table(consumer_signal_offsets, dev, None)
        # read back once per table object: a device-to-host copy per launch would wait for the stream to drain
        owned = isinstance(consumer_signal_offsets, torch.Tensor) and consumer_signal_offsets.is_cuda
        note = f"indices to wait for, {num_waves} waves, {wait_flags.numel()} flags"
        if not (owned and recall_note([consumer_signal_offsets], note)):
            hw = host_copy(wait_sigs)
            if wait_sigs.numel() < num_waves or int(hw[:num_waves].min()) < -1 or \
                    int(hw[:num_waves].max()) >= wait_flags.numel():
                raise ValueError("consumer_signal_offsets must hold one index into consumer_signal_ptr (or -1) per wave")
            if owned:
                remember_note([consumer_signal_offsets], note, True)
    o = torch.empty(q.shape, dtype=q.dtype, device=dev) if out is None else out
    if o.shape != q.shape or o.dtype != q.dtype:
        raise ValueError("out must match q")
    # lse (base 2), lock and first-writer marker: the reference's M / guard / first
    # (template.py:382-384), one lock per 128-row q block
    lse = torch.empty((Z, H, Sq), device=dev, dtype=torch.float32)
    scratch = zeroed_int32((2, Z, H, Sq // BLOCK_M), dev)
    tiles = int(cum_tiles) // BLOCK_M
    if visit_log is not None:
        if visit_log.dtype != torch.int32 or visit_log.numel() < 8 * tiles or not visit_log.is_contiguous():
            raise ValueError(f"visit_log must be a contiguous int32 tensor of at least {8 * tiles} words")

    desc = _lib.AttnDesc(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), o=o.data_ptr(), lse=lse.data_ptr(),
        lock=scratch[0].data_ptr(), first=scratch[1].data_ptr(), flags=flags.data_ptr(),
        wave_offsets=offs.data_ptr(), wave_sizes=sizes.data_ptr(), cum_wave_sizes=cums.data_ptr(),
        signal_offsets=sigs.data_ptr(),
        visit_log=None if visit_log is None else visit_log.data_ptr(),
        status=status_words(dev).data_ptr(),
        num_waves=num_waves, Z=Z, H=H, Sq=Sq, Skv=Skv, D=D, dtype=_lib.dtype_code(q.dtype),
        block_m=BLOCK_M, block_n=BLOCK_N, causal=1 if causal else 0, num_programs=int(num_programs),
        sm_scale=float(sm_scale), cum_tiles=int(cum_tiles), spin_timeout_us=int(spin_timeout_us),
        q_strides=strides(q), k_strides=strides(k), v_strides=strides(v), o_strides=strides(o),
        counters=None if counter_ptr is None else counter_ptr.data_ptr(),
        options=(_lib.SYN_ATTN_PAIR_Q_BLOCKS if pair_q_blocks else 0) | (_lib.SYN_ATTN_XCD_REMAP if xcd_remap else 0)
        | (_lib.SYN_ATTN_CHAIN_Q_BLOCKS if chain_q_blocks else 0) | (_lib.SYN_ATTN_WORK_LIST if work_plan is not None else 0)
        | (_lib.SYN_ATTN_ACQUIRE_ALWAYS
           if acquire_always(consumer_signal_ptr if consumer_signal_ptr is not None else signal_ptr) else 0),
        wait_flags=None if wait_flags is None else wait_flags.data_ptr(),
        wait_signal_offsets=None if wait_sigs is None else wait_sigs.data_ptr(),
        work_list=None if work_plan is None else _device_words(work_plan, dev).data_ptr(),
    )
    with torch.cuda.device(dev):
        _lib.check("syn_attn_fwd", lib.syn_attn_fwd(ctypes.byref(desc), _lib.stream_handle(stream)))
    return (o, lse) if return_lse else o


# a plan's words on a device, kept with the plan object
_plan_words: Dict[tuple, tuple] = {}


def _device_words(plan: WorkPlan, dev: torch.device) -> torch.Tensor:
    key = (id(plan), dev.index)
    entry = _plan_words.get(key)
    if entry is None or entry[0] is not plan:
        if len(_plan_words) > 256:
            _plan_words.clear()
        entry = (plan, torch.tensor(plan.words, dtype=torch.int32, device=dev))
        _plan_words[key] = entry
    return entry[1]


def attention(q, k, v, sm_scale, wave_dicts: Dict, BLOCK_M=128, BLOCK_N=128, NUM_BUFFERS=2,
              NUM_MMA_WARPS=8, NUM_MMA_GROUPS=2, **kwargs):
    """Hand-template call form (template.py:366-439): tables in block units."""
    if BLOCK_M != 128 or BLOCK_N != 128:
        raise ValueError("the gfx950 kernel uses 128x128 blocks")
    dev = q.device
    offs = as_device_table(wave_dicts["wave_offsets"], dev, 4).clone()
    sizes = as_device_table(wave_dicts["wave_sizes"], dev, 4).clone()
    cums = as_device_table(wave_dicts["cum_wave_sizes"], dev, None).clone()
    # blocks -> elements along Q and KV; programs -> Z*H*Q elements
    scale = torch.tensor([1, 1, BLOCK_M, BLOCK_N], dtype=torch.int32, device=dev)
    offs *= scale
    sizes *= scale
    cums *= BLOCK_M
    signal_ptr = wave_dicts["signal_ptr"]
    if signal_ptr.element_size() != 8:
        # the reference's "everything resident" helper hands out int32 ones (template.py:622)
        signal_ptr = signal_ptr.to(torch.int64)
    return attention_forward(
        q, k, v, sm_scale,
        wave_offsets=offs, wave_sizes=sizes, cum_wave_sizes=cums,
        signal_ptr=signal_ptr, signal_offsets=wave_dicts["signal_offsets"],
        NUM_WAVES=wave_dicts.get("CUM_CHUNK_BLOCK"), **{"form": "auto", **kwargs})


def build_waves_and_signals_divisible(Z, H, N_CTX_Q, N_CTX_KV, *, BLOCK_M=128, BLOCK_N=128, w=4,
                                      device="cuda"):
    """Split only along KV into `w` equal waves, everything resident (all flags set):
    the table shape of the reference's `_build_waves_and_signals_divisible`
    (template.py:567-641), block units, padded with zero rows to a power of two.
    """
    if N_CTX_Q % BLOCK_M or N_CTX_KV % BLOCK_N or w <= 0:
        raise ValueError("sequence lengths must be multiples of the block sizes and w positive")
    nq = N_CTX_Q // BLOCK_M
    nkv = N_CTX_KV // BLOCK_N
    if nkv % w:
        raise ValueError(f"(N_CTX_KV/BLOCK_N)={nkv} must be divisible by w({w})")
    per = nkv // w
    padded = 1 if w <= 1 else 1 << ((w - 1).bit_length())
    offsets, sizes, cums = [], [], []
    for i in range(w):
        offsets.append([0, 0, 0, i * per])
        sizes.append([Z, H, nq, per])
        cums.append((i + 1) * Z * H * nq)
    for _ in range(padded - w):
        offsets.append([0, 0, 0, 0])
        sizes.append([0, 0, 0, 0])
        cums.append(0)
    return dict(
        wave_offsets=torch.tensor(offsets, dtype=torch.int32, device=device).flatten(),
        wave_sizes=torch.tensor(sizes, dtype=torch.int32, device=device).flatten(),
        cum_wave_sizes=torch.tensor(cums, dtype=torch.int32, device=device),
        signal_ptr=torch.ones(padded, dtype=torch.int64, device=device),
        signal_offsets=torch.zeros(padded, dtype=torch.int32, device=device),
        CUM_CHUNK_BLOCK=padded,
        num_pid_q=nq,
        num_pid_kv_total=nkv,
        kv_per_wave=per,
        w=w,
    )
