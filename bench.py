"""Benchmark of the chunk-scheduled compute path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only ag_gemm,reduce,...]

The headline step is one fused all-gather+GEMM iteration of rank 0 of a simulated mesh of 8
(M, K, N = 8192, 8192, 3584): flags reset, the 7 peer chunks of A (1024 x 8192 bf16 each)
copied into the symmetric buffer on a side stream in the order the lowered schedule
prescribes (copy, then flag), the consumer GEMM (8192 x 8192 x 3584) on the compute stream
waiting on each chunk's flag.  All operands are resident in HBM before the timed region.
The W warm-up steps follow SETTLE_STEPS further untimed steps (an idle device's clocks settle
over the first ~10 ms of work); the timed region is exactly K steps.  Prints ONE JSON line.

Beside the headline the same line carries the other workloads of the path, each with the number
of launches its figure averages over: the matrix-pipe ceiling of the board (a loop of nothing
but MFMAs, constant and random operands) and the consumer kernel on zero operands, the producer
throttled to a link's rate, the chunked reduce, the GEMM+RS producer and the fused GEMM+RS step
(producer, pushes gated by its flags, reduce), all-gather attention (resident and with the kv
chunks arriving behind flags), all-to-all attention (causal; resident and gated), box copies,
and CPU baselines of the same workloads on the host's cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402

MFMA_BF16_PEAK_TFLOPS = 2500.0      # MI355X dense bf16
HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the kernels below come from hardware-counter runs, which serialise
# kernels and therefore cannot be taken while the benchmark itself runs; the readings are kept
# in this tracked file together with the commands that made them.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")

# AG+GEMM, the headline configuration
M, K, N, WORLD, RANK = 8192, 8192, 3584, 8, 0
BM, BN, BK, GROUP_M = 256, 256, 64, 8
NUM_SMS = 224                        # 448 tiles = 2 per program; 32 of the 256 CUs stay free for the
                                     # copy kernels of the producer
SETTLE_STEPS = 40                    # untimed steps ahead of the W warm-up steps: the clocks of an idle device
                                     # take some ten milliseconds of this work to settle (20 steps behind 5
                                     # warm-up steps measure 0.49 ms per step, behind 40 of them 0.43 ms)
XCD_REMAP = False                    # consecutive tile ids on one XCD (see --xcd-remap)
LEAD_OPS = 3                         # ops of the side stream the consumer launch waits for: two chunks copied, the
                                     # first one's flag set (the second flag lands while the first tiles run)
EIGHT_WAVES = False                  # 256-thread workgroups: one wavefront per SIMD, 128x128 of C each
LEAD_COPY_BLOCKS = 0                 # see --lead-copy-blocks
LIST_BLOCKS = 0                      # see --list-blocks
LEAD_ON_COMPUTE_STREAM = False       # see --lead-on-compute-stream
LINK_CHUNK_US = 110                  # one 16.8 MB chunk over one xGMI link (~153 GB/s)

SECTIONS = ("ag_gemm", "throttled", "mfma_ceiling", "library", "reduce", "box_copies", "gemm_rs", "attn_ag", "attn_a2a",
            "attn_slot", "cpu")


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _timed(fn, launches, warmup, stream=None):
    """Average milliseconds of `launches` calls of fn(i), timed as one batch between two events."""
    stream = torch.cuda.current_stream() if stream is None else stream
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    begin, end = _events(2)
    begin.record(stream)
    for i in range(launches):
        fn(i)
    end.record(stream)
    torch.cuda.synchronize()
    return begin.elapsed_time(end) / launches


def _table(rows, device):
    return torch.tensor(rows, dtype=torch.int32, device=device)


# ----------------------------------------------------------------------------------- AG+GEMM

def build_ag_gemm(device, copy_blocks=0, split_units=0, fuse_flags=False, link_delay_us=0, lead_copy_blocks=0,
                  flag_write_values=False, list_blocks=0):
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import gemm_consumer_tables

    t0 = time.perf_counter()
    plans = {r: build_all_gather_plan_1d_swizzle((M, K), torch.bfloat16, 0, WORLD, r, "a", "pull")
             for r in range(WORLD)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    schedule = lower_comm_plan_to_raw_schedules(gen)[RANK]["a"]
    info = gen.generate_code_for_plan()
    compile_ms = (time.perf_counter() - t0) * 1e3
    info.local_world_size = info.world_size
    if split_units:
        # the device split in two: `split_units` compute units for the producer's copy kernels, the
        # consumer on the stream that owns the rest
        info.need_green_ctx, info.num_copy_sms = True, split_units
    tables = gemm_consumer_tables(schedule, N)

    torch.manual_seed(0)
    a = (0.02 * torch.randn(M, K, device=device)).bfloat16()
    b = (0.02 * torch.randn(N, K, device=device)).bfloat16()
    # two flag sets: the reset of one iteration's flags happens behind the next one's copies
    ctx = CommContext(RANK, info, device=device, copy_blocks=copy_blocks, flag_sets=2, fuse_flags=fuse_flags,
                      link_delay_us=link_delay_us, lead_copy_blocks=lead_copy_blocks, flag_write_values=flag_write_values,
                      list_blocks=list_blocks)
    rows = M // WORLD
    for r in range(WORLD):     # every rank's symmetric buffer holds its own shard
        ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
    dev_tables = dict(
        cur_wave_sizes=_table(tables.block_shapes, device),
        wave_offsets=_table(tables.block_offsets, device),
        signal_offsets=_table(tables.signal_offsets, device),
        cum_tiles=tables.cum_tiles,
    )
    c = torch.empty(M, N, dtype=torch.bfloat16, device=device)
    return dict(a=a, b=b, c=c, ctx=ctx, tables=dev_tables, compile_ms=compile_ms)


def run_ag_gemm(state, steps, warmup, resident_only=False, use_graph=True, lead_ops=None):
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm

    lead_ops = LEAD_OPS if lead_ops is None else lead_ops
    ctx, b, c, tables = state["ctx"], state["b"], state["c"], state["tables"]
    symm = ctx.comm_buffers["a"][RANK]
    stream = torch.cuda.current_stream()

    def consumer(flag_words, a_operand=symm, b_operand=b):
        gemm(a_operand, b_operand, c, WORLD, NUM_SMS, BM, BN, BK, GROUP_M, signal_ptr=flag_words, xcd_remap=XCD_REMAP,
             eight_waves=EIGHT_WAVES, **tables)

    def fused_step():
        cur = torch.cuda.current_stream()
        ctx.reset_signals()               # switches to the zeroed flag set
        ctx.start_after(cur)
        ctx.execute(lead_ops=lead_ops, lead_on=cur if LEAD_ON_COMPUTE_STREAM else None)
        if lead_ops:
            ctx.wait_lead(cur)            # the kernel starts behind the first chunk copies (3x faster before it does)
        consumer(ctx.recv_signal_bufs[RANK])
        ctx.end_before(cur)

    # One step is ~25 launches (7 copies, 7 flag writes, flag reset, stream joins, the GEMM):
    # replayed as a HIP graph so that the host's launch rate is not what gets measured (kernels
    # and memcpy nodes only).  The graph holds two steps, since consecutive steps use alternate
    # flag sets; the warm-up replays it, the timed region replays it steps/2 times (the first
    # replay of a graph pays for its instantiation on the device: ~1.5 ms for 20 steps' nodes,
    # which a graph of all timed steps replayed once would book as 60 us per step); an odd step
    # count ends with one step launched from the host.
    def capture(n):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(n):
                fused_step()
        return graph

    if resident_only:
        # counter runs serialise kernels: a gated consumer would wait for copies that can only
        # start after it.  Only the producer runs, so that the gathered buffer is complete.
        use_graph = False
        ctx.reset_signals()
        ctx.start_after(stream)
        ctx.execute()
        ctx.end_before(stream)
    else:
        fused_step()
        fused_step()
    torch.cuda.synchronize()
    pair_graph = capture(2) if use_graph else None

    # ---- gated run: the step the metric is quoted on ----
    wall_ms = gated_kernel_ms = no_lead_kernel_ms = None
    if not resident_only:
        for _ in range(SETTLE_STEPS // 2 + (warmup + 1) // 2):
            if use_graph:
                pair_graph.replay()
            else:
                fused_step()
                fused_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if pair_graph is not None:           # EXACTLY `steps` fused steps, nothing else on the streams
            for _ in range(steps // 2):
                pair_graph.replay()
            if steps % 2:
                fused_step()
        else:
            for _ in range(steps):
                fused_step()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        # the same steps once more, launched from the host, with HIP events around the consumer
        # launch (event markers perturb the overlap slightly, so they stay out of the timed region
        # above); then a few with the kernel launched together with the first copy instead of
        # behind the leading chunks
        def kernel_ms(count, lead):
            begin, end = _events(count), _events(count)
            for i in range(count):
                ctx.reset_signals()
                ctx.start_after(stream)
                ctx.execute(lead_ops=lead, lead_on=stream if (lead and LEAD_ON_COMPUTE_STREAM) else None)
                if lead:
                    ctx.wait_lead(stream)
                begin[i].record(stream)
                consumer(ctx.recv_signal_bufs[RANK])
                end[i].record(stream)
                ctx.end_before(stream)
            torch.cuda.synchronize()
            return sum(s.elapsed_time(e) for s, e in zip(begin, end)) / count
        gated_kernel_ms = kernel_ms(steps, lead_ops)
        no_lead_kernel_ms = kernel_ms(min(steps, 20), 0) if lead_ops else gated_kernel_ms
    check_status()
    ctx.check_status()

    # ---- same kernel, every chunk resident and every flag already set ----
    # (a flag array of the benchmark's own: declared trusted, as the executor's are - nothing here reads a chunk
    # before its flag - so that resident and gated launches run the same code path)
    from syncopate_amd.computation._launch import trust_flags
    resident_flags = torch.ones_like(ctx.recv_signal_bufs[RANK])
    trust_flags(resident_flags)

    def resident_ms(a_operand=symm, b_operand=b):
        for _ in range(warmup):
            consumer(resident_flags, a_operand, b_operand)
        torch.cuda.synchronize()
        begin, end = _events(steps), _events(steps)
        for i in range(steps):
            begin[i].record(stream)
            consumer(resident_flags, a_operand, b_operand)
            end[i].record(stream)
        torch.cuda.synchronize()
        return sum(s.elapsed_time(e) for s, e in zip(begin, end)) / steps

    resident_kernel_ms = resident_ms()
    check_status()
    if resident_only:
        wall_ms = gated_kernel_ms = no_lead_kernel_ms = resident_kernel_ms
    state["resident_ms_fn"] = resident_ms
    return wall_ms, gated_kernel_ms, no_lead_kernel_ms, resident_kernel_ms


def run_throttled(device, steps):
    """The same fused step with the producer throttled to one link's rate: a delay in front of
    every chunk copy brings a chunk to ~LINK_CHUNK_US, the time 16.8 MB take over one xGMI link.
    Seven chunks in sequence then take longer than the GEMM: the step is bound by the producer,
    and what the wave order buys is that only the last chunk's tiles are left when it lands - if
    the tile shape lets that chunk fill the machine.  Every shape is timed; `choose_tile` picks."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import choose_tile, gemm

    delay = LINK_CHUNK_US - 28          # a chunk copy beside the running GEMM takes ~28 us
    state = build_ag_gemm(device, link_delay_us=delay)
    ctx, b, c, tables = state["ctx"], state["b"], state["c"], state["tables"]
    symm = ctx.comm_buffers["a"][RANK]
    stream = torch.cuda.current_stream()

    def step_for(bm, bn):
        def step(i):
            ctx.reset_signals()
            ctx.start_after(stream)
            ctx.execute()
            gemm(symm, b, c, WORLD, NUM_SMS, bm, bn, BK, GROUP_M, signal_ptr=ctx.recv_signal_bufs[RANK],
                 xcd_remap=XCD_REMAP, eight_waves=EIGHT_WAVES, **tables)
            ctx.end_before(stream)
        return step

    # the producer alone: the same op list with nothing to overlap
    def comm_only(i):
        ctx.reset_signals()
        ctx.start_after(stream)
        ctx.execute()
        ctx.end_before(stream)
    comm_ms = _timed(comm_only, steps, 3, stream)
    by_shape = {}
    for bm, bn in ((256, 256), (128, 256), (256, 128), (128, 128)):
        ms = _timed(step_for(bm, bn), steps, 5, stream)
        check_status()
        ctx.check_status()
        rows = torch.arange(0, M, 257, device=device)
        ref = state["a"][rows].float() @ b.float().t()
        err = ((c[rows].float() - ref).abs().max() / ref.abs().max()).item()
        by_shape[f"{bm}x{bn}"] = {"ms_per_step": ms, "exposed_compute_ms": ms - comm_ms, "max_rel_err_vs_fp32": err}
    comm_after_ms = _timed(comm_only, steps, 3, stream)
    bm, bn = choose_tile(M // WORLD, N, NUM_SMS, producer_bound=True)
    chosen = by_shape[f"{bm}x{bn}"]
    del state
    return {"launches": steps, "link_delay_us_per_chunk": delay, "tile": f"{bm}x{bn}",
            "tile_choice": "choose_tile(chunk rows, N, programs, producer_bound=True): fewest rounds x tile time for the last chunk",
            "ms_per_step": chosen["ms_per_step"], "producer_alone_ms": comm_ms, "producer_alone_after_ms": comm_after_ms,
            "exposed_compute_ms": chosen["exposed_compute_ms"], "by_tile": by_shape}


def traffic_calibration(device):
    """One launch of the library's plain copy kernel over 64 MiB: under a counter run its
    FETCH_SIZE / WRITE_SIZE readings give the scale of those counters (65536 KiB each way)."""
    from syncopate_amd import _lib

    lib = _lib.load()
    nbytes = 64 << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device=device).fill_(1)
    dst = torch.empty_like(src)
    _lib.check("syn_copy_kernel_async",
               lib.syn_copy_kernel_async(dst.data_ptr(), src.data_ptr(), nbytes, 1024,
                                         torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()


def check_ag_gemm(state):
    """Spot-check the last step's output against torch on the GPU (fp32 accumulate)."""
    a, b, c = state["a"], state["b"], state["c"]
    rows = torch.arange(0, M, 257, device=a.device)
    ref = a[rows].float() @ b.float().t()
    err = ((c[rows].float() - ref).abs().max() / ref.abs().max()).item()
    gathered = torch.equal(state["ctx"].comm_buffers["a"][RANK], a)
    return err, gathered


# ---------------------------------------------------------------------------- matrix-pipe ceiling

def run_mfma_ceiling(device, state, launches=8):
    """What the matrix pipes of this board sustain: a loop of nothing but the GEMM's MFMA on
    register-resident operands, one workgroup of four wavefronts per compute unit, with constant
    and with random operands (the board is power-limited: toggling operand bits cost clock);
    and the consumer kernel itself, every chunk resident, on operands that are all zero."""
    from syncopate_amd import _lib

    lib = _lib.load()
    sink = torch.empty(256 * 256, dtype=torch.float32, device=device)
    stream = _lib.stream_handle(torch.cuda.current_stream())
    iters = 2000
    out = {"launches": launches, "mfma": "v_mfma_f32_16x16x32_bf16, 8x8 accumulators per wavefront, 128 per round (the 256x256 tile's "
                                          "K loop); mfma_32x32x16_*: v_mfma_f32_32x32x16_bf16, 4x4 accumulators, 64 per round",
           "rounds_per_launch": iters}
    for workgroups in (256, NUM_SMS):
        for pattern, name in ((5, "constant"), (6, "random"), (1, "mfma_32x32x16_constant"), (2, "mfma_32x32x16_random")):
            def probe(i):
                _lib.check("syn_probe_mfma_rate", lib.syn_probe_mfma_rate(sink.data_ptr(), workgroups, iters, pattern, stream))
            ms = _timed(probe, launches, 3)
            out[f"{name}_operands_{workgroups}_workgroups_tflops"] = workgroups * 4.0 * iters * 64 * 32768 / ms / 1e9
    if state is not None and "resident_ms_fn" in state:
        zeros_a, zeros_b = torch.zeros_like(state["a"]), torch.zeros_like(state["b"])
        ms = state["resident_ms_fn"](zeros_a, zeros_b)
        out["consumer_kernel_zero_operands_tflops"] = 2.0 * M * N * K / ms / 1e9
        out["consumer_kernel_zero_operands_ms"] = ms
    return out


def run_library_baselines(device, state):
    """The vendor libraries on the same operands, for scale (not part of the path: they take whole,
    resident operands and know nothing of chunks or flags): torch.matmul (hipBLASLt) on the two
    GEMM shapes, torch's scaled_dot_product_attention on the two attention shapes."""
    import torch.nn.functional as F

    # the board's clock settles over the first ~80 launches after other work (it rises): timed behind as many
    out = {"launches": 100, "warmup_launches": 80}
    a, b = state["a"], state["b"]
    ms = _timed(lambda i: torch.matmul(a, b.t()), 100, 80)
    out["matmul_8192x8192x3584_tflops"] = 2.0 * M * N * K / ms / 1e9
    a2 = (0.02 * torch.randn(8192, 3584, device=device)).bfloat16()
    b2 = (0.02 * torch.randn(8192, 3584, device=device)).bfloat16()
    ms = _timed(lambda i: torch.matmul(a2, b2.t()), 100, 80)
    out["matmul_8192x3584x8192_tflops"] = 2.0 * 8192 * 8192 * 3584 / ms / 1e9
    za, zb = torch.zeros_like(a), torch.zeros_like(b)
    ms = _timed(lambda i: torch.matmul(za, zb.t()), 100, 80)
    out["matmul_8192x8192x3584_zero_operands_tflops"] = 2.0 * M * N * K / ms / 1e9
    del a2, b2, za, zb
    q = torch.randn(1, 32, 4096, 128, device=device).bfloat16()
    k = torch.randn(1, 32, 32768, 128, device=device).bfloat16()
    v = torch.randn(1, 32, 32768, 128, device=device).bfloat16()
    ms = _timed(lambda i: F.scaled_dot_product_attention(q, k, v), 5, 2)
    out["sdpa_4096x32768_32_heads_tflops"] = 4.0 * 32 * 4096 * 32768 * 128 / ms / 1e9
    q = torch.randn(1, 4, 16384, 128, device=device).bfloat16()
    k, v = torch.randn_like(q), torch.randn_like(q)
    ms = _timed(lambda i: F.scaled_dot_product_attention(q, k, v, is_causal=True), 5, 2)
    out["sdpa_16384_causal_4_heads_tflops"] = 2.0 * 4 * 16384 * 16384 * 128 / ms / 1e9
    return out


# --------------------------------------------------------------------------------------- reduce

def run_reduce(device, steps, warmup):
    """GEMM+RS chunked reduce of the headline GEMM+RS configuration: 8 x (1024, 8192) bf16 -> (1024, 8192).
    Launches rotate over three sets of operands (3 x 151 MB, more than the 256 MB of memory-side
    cache) so that every launch streams from HBM; the batch is timed as a whole."""
    from syncopate_amd.computation.reduce import padded_receive_buffer, ring_reduce

    world, rows, n, sets = 8, 1024, 8192, 3
    torch.manual_seed(1)
    recv = [torch.randn(world, rows, n, device=device).bfloat16() for _ in range(sets)]
    local = [torch.randn(world * rows, n, device=device).bfloat16() for _ in range(sets)]
    out = [torch.empty(rows, n, dtype=torch.bfloat16, device=device) for _ in range(sets)]
    ms = _timed(lambda i: ring_reduce(recv[i % sets], out[i % sets], local[i % sets], RANK), steps, max(warmup, sets))
    nbytes = (world + 1) * rows * n * 2          # 8 reads + 1 write of a (1024, 8192) bf16 block
    # the same with the eight received blocks 16 MiB + 4 KiB apart (a caller's own receive buffer; the executor's
    # symmetric buffers keep the reference's contiguous layout, whose byte offsets the op lists carry)
    padded = [padded_receive_buffer(world, rows, n, torch.bfloat16, device) for _ in range(sets)]
    for dst, src in zip(padded, recv):
        dst.copy_(src)
    padded_ms = _timed(lambda i: ring_reduce(padded[i % sets], out[i % sets], local[i % sets], RANK), steps, max(warmup, sets))
    return ms, nbytes, padded_ms


def run_hbm_read_ceiling(device, launches=30):
    """What the memory system gives the reduce's READS (`syn_probe_read_streams`: the reduce's loop with an
    exclusive-or in place of the adds and no result stream, 512 workgroups like the reduce): one linear
    stream; eight streams 16 MiB apart, which is where the reference's layout [W, rows, N] puts the
    eight partial blocks of (1024, 8192) bf16; and the same eight streams 16 MiB + 4 KiB apart.  Launches
    rotate over three regions (3 x 134 MB, more than the memory-side cache)."""
    from syncopate_amd import _lib

    lib = _lib.load()
    stream_bytes, sets, blocks = 16 << 20, 3, 512
    span = 8 * (stream_bytes + 4096)
    torch.manual_seed(5)
    pool = torch.randint(0, 2 ** 31 - 1, (sets * span // 4,), dtype=torch.int32, device=device)
    sink = torch.zeros(4 * blocks, dtype=torch.int32, device=device)

    def probe(region, nbytes, stride, streams):
        _lib.check("syn_probe_read_streams", lib.syn_probe_read_streams(pool.data_ptr() + region * span, nbytes, stride,
                                                                         streams, blocks, sink.data_ptr(),
                                                                         _lib.stream_handle(None)))

    forms = {"one_stream_128MiB": (8 * stream_bytes, 0, 1), "eight_streams_16MiB_apart": (stream_bytes, stream_bytes, 8),
             "eight_streams_16MiB_plus_4KiB_apart": (stream_bytes, stream_bytes + 4096, 8)}
    result = {"launches": launches, "bytes_read_per_launch": 8 * stream_bytes}
    for name, (nbytes, stride, streams) in forms.items():
        ms = _timed(lambda i: probe(i % sets, nbytes, stride, streams), launches, sets)
        result[name + "_GBps"] = 8 * stream_bytes / (ms * 1e-3) / 1e9

    # the eight streams 16 MiB apart again, read the way the reduce walks them: skewed by one 4 KB block per stream
    def skewed(region):
        _lib.check("syn_probe_read_streams_skewed",
                   lib.syn_probe_read_streams_skewed(pool.data_ptr() + region * span, stream_bytes, stream_bytes, blocks,
                                                     sink.data_ptr(), _lib.stream_handle(None)))
    ms = _timed(lambda i: skewed(i % sets), launches, sets)
    result["eight_streams_16MiB_apart_skewed_walk_GBps"] = 8 * stream_bytes / (ms * 1e-3) / 1e9
    return result


def run_box_copies(device, steps, warmup):
    """Box copies on compute units (the SM copy ops of reduce-scatter by direct reduction): one
    rank's (8192, 8192) bf16 partial product added into / copied onto a result of the same shape
    with 256 workgroups.  Operands rotate over three sets (6 x 134 MB) so that every launch
    streams from HBM.  Returns {form: (ms, HBM bytes per launch)}."""
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.communication.descriptor import ReduceOp

    rows, n, sets, blocks = 8192, 8192, 3, 256
    torch.manual_seed(3)
    src = [torch.randn(rows, n, device=device).bfloat16() for _ in range(sets)]
    dst = [torch.zeros(rows, n, dtype=torch.bfloat16, device=device) for _ in range(sets)]
    nbytes = rows * n * 2
    forms = {"copy": (None, False, 2 * nbytes), "add_exclusive": (ReduceOp.SUM, True, 3 * nbytes),
             "add_atomic": (ReduceOp.SUM, False, 3 * nbytes)}
    result = {}
    for name, (op, exclusive, traffic) in forms.items():
        ms = _timed(lambda i: persistent_copy_last_contig(src[i % sets], dst[i % sets], num_sms=blocks, reduce_op=op,
                                                          exclusive=exclusive), steps, max(warmup, sets))
        result[name] = (ms, traffic)
    return result


# -------------------------------------------------------------------------------------- GEMM+RS

def run_gemm_rs(device, steps, warmup, gated=True):
    """GEMM+RS of rank 0 of 8: partial C (8192, 8192) = A (8192, 3584) B^T in wave order 1..7, 0 with
    per-wave counters and flags.  Timed twice: the producer kernel alone, and the fused step the
    reference times (tests/test_gemm_rs.py:196-244) - producer on the compute stream, the pushes
    of the finished chunks to their owners on a side stream, each behind its wave's COMPUTE_DONE
    flag, then the chunked reduce of the 7 received partials and the rank's own block."""
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.comm_runtime.communication_context import CommContext
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm_producer
    from syncopate_amd.computation.reduce import ring_reduce
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import gemm_producer_tables

    m, k, n, world = 8192, 3584, 8192, 8
    rows = m // world
    plans = {r: build_all_to_all_plan(shape=(m, n), dtype=torch.bfloat16, mesh_size=world, rank=r, src_buffer="src",
                                      dst_buffer="dst", transfer_kind="push", compute_producer=True)
             for r in range(world)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    tables = gemm_producer_tables(lower_comm_plan_to_raw_schedules(gen)[RANK]["src"])
    info = gen.generate_code_for_plan()
    info.local_world_size = info.world_size
    ctx = CommContext(RANK, info, device=device)
    torch.manual_seed(3)
    a = (0.02 * torch.randn(m, k, device=device)).bfloat16()
    b = (0.02 * torch.randn(n, k, device=device)).bfloat16()
    src, dst = ctx.comm_buffers["src"][RANK], ctx.comm_buffers["dst"][RANK]
    dst.copy_(torch.randn(world, rows, n, device=device).bfloat16())       # what the peers pushed
    out = torch.empty(rows, n, dtype=torch.bfloat16, device=device)
    sizes, offsets = _table(tables.block_shapes, device), _table(tables.block_offsets, device)
    signals = _table(tables.signal_offsets, device)
    counters = torch.zeros(world, dtype=torch.int32, device=device)
    main = torch.cuda.current_stream()

    def producer(flags, programs=256, xcd_remap=True):
        counters.zero_()
        # 1024 tiles of 256 x 256: four full rounds of 256 programs.  With the remap an XCD's 32 tiles of a
        # round are 4 x 8 neighbours (12 panels of A and B through its L2 instead of 18).
        gemm_producer(a, b, src, flags, sizes, offsets, signals, programs, 256, 256, BK, GROUP_M,
                      cum_tiles=tables.cum_tiles, counter_buffer=counters, xcd_remap=xcd_remap, eight_waves=EIGHT_WAVES)

    alone_flags = torch.zeros(world, dtype=torch.int64, device=device)
    _timed(lambda i: producer(alone_flags), max(3, steps // 4), warmup)        # clocks settle
    producer_ms = _timed(lambda i: producer(alone_flags), steps, warmup)
    assert alone_flags.tolist() == [1] * world
    no_remap_ms = _timed(lambda i: producer(alone_flags, xcd_remap=False), steps, warmup)

    if not gated:
        return {"launches": steps, "producer_ms": producer_ms, "producer_ms_without_xcd_remap": no_remap_ms,
                "flop": 2.0 * m * n * k}

    def fused(programs):
        ctx.reset_signals()
        ctx.start_after(main)
        producer(ctx.compute_signal_bufs[RANK], programs)
        ctx.execute(neglect_local=True)
        ctx.end_before(main)
        ring_reduce(dst, out, src, RANK)

    # On one GPU the pushes are copy kernels that need compute units: beside 256 persistent programs
    # they only run once the producer has finished; 224 programs leave them 32 units but cost the
    # GEMM a fifth round of tiles.  Both are timed; a node's copy engines need neither.
    fused_by_programs = {programs: _timed(lambda i: fused(programs), steps, max(3, warmup // 4)) for programs in (224, 256)}
    fused_ms = min(fused_by_programs.values())
    check_status()
    ctx.check_status()
    sample = torch.arange(7, rows, 97, device=device)
    acc = src[RANK * rows:(RANK + 1) * rows][sample].clone()
    for i in range(1, world):
        acc = acc + dst[(RANK + i) % world][sample]
    reduce_matches = torch.equal(out[sample], acc)
    pushed = all(torch.equal(ctx.comm_buffers["dst"][p][RANK], src[p * rows:(p + 1) * rows]) for p in (1, 4, 7))
    # The reference's other GEMM+RS form (template_rs.py:212-290, tests/test_gemm_rs_direct_reduce.py): no pushes and no
    # reduce kernel - the GEMM's epilogue adds every tile into its owner's (1024, 8192) result with packed 16-bit
    # float atomics.  This rank's launch alone, all 256 compute units (the peers' atomics would arrive beside it);
    # the owners' buffers are eight local allocations here and keep accumulating over the timed launches.
    from syncopate_amd.computation.gemm import gemm_rs_producer_persistent
    owners = [torch.zeros(rows, n, dtype=torch.bfloat16, device=device) for _ in range(world)]
    targets = [row // rows for row, _ in tables.block_offsets]
    owner_table = _table(targets, device)
    def direct():
        gemm_rs_producer_persistent(a, b, owners, sizes, offsets, owner_table, world, world, 256, 256, 256, BK, GROUP_M)
    direct()
    torch.cuda.synchronize()
    direct_matches = True
    for p in (1, 4, RANK):
        ref = a[p * rows + 5:p * rows + 6].float() @ b.float().t()
        direct_matches = direct_matches and bool(((owners[p][5:6].float() - ref).abs().max() / ref.abs().max()) < 1e-2)
    direct_ms = _timed(lambda i: direct(), steps, max(3, warmup // 4))
    check_status()
    # A third form, from the same per-wave peer bindings with a plain store (RemoteBinding without a reduction,
    # transform/transformer.py:1158-1178): the epilogue writes every tile straight into this rank's slot of its
    # owner's receive buffer - no pushes, so nothing beside the GEMM needs compute units and all 256 programs run -
    # and the chunked reduce follows.  The same bytes land in the same places as in the fused step.
    from syncopate_amd.computation.gemm import gemm_remote
    peers = ctx.comm_buffers["dst"]
    slots = [src[RANK * rows:(RANK + 1) * rows] if p == RANK else peers[p][RANK] for p in range(world)]
    slot_offsets = torch.tensor(tables.block_offsets, dtype=torch.int32)
    slot_offsets[:, 0] = 0                       # rows are wave-local in the owner's slot, columns keep their place
    slot_offsets, owner_of_wave = slot_offsets.to(device), _table(targets, device)
    for p in (1, 4, 7):
        peers[p][RANK].zero_()

    def stored(reduce=True):
        gemm_remote(a, b, slots, 256, 256, 256, BK, GROUP_M, cur_wave_sizes=sizes, wave_offsets=offsets, M=m,
                    target_rank=owner_of_wave, dst_offsets=slot_offsets, cum_tiles=tables.cum_tiles)
        if reduce:
            ring_reduce(dst, out, src, RANK)
    stored()
    torch.cuda.synchronize()
    stored_matches = all(torch.equal(peers[p][RANK], src[p * rows:(p + 1) * rows]) for p in (1, 4, 7))
    acc = src[RANK * rows:(RANK + 1) * rows][sample].clone()
    for i in range(1, world):
        acc = acc + dst[(RANK + i) % world][sample]
    stored_matches = stored_matches and torch.equal(out[sample], acc)
    stored_ms = _timed(lambda i: stored(), steps, max(3, warmup // 4))
    stored_gemm_ms = _timed(lambda i: stored(reduce=False), steps, max(3, warmup // 4))
    check_status()
    return {"launches": steps, "producer_ms": producer_ms, "producer_ms_without_xcd_remap": no_remap_ms,
            "flop": 2.0 * m * n * k, "fused_step_ms": fused_ms,
            "fused_step_ms_by_programs": {str(k_): v for k_, v in fused_by_programs.items()},
            "reduce_matches": bool(reduce_matches), "pushed_chunks_match": bool(pushed),
            "direct_reduce_form_ms": direct_ms, "direct_reduce_form_matches": direct_matches,
            "remote_store_form_ms": stored_ms, "remote_store_form_gemm_ms": stored_gemm_ms,
            "remote_store_form_matches": bool(stored_matches)}


# ------------------------------------------------------------------------------------ attention

def _gated_attention(q, staged_kv, buf, arrival, chunk, tables, launches, device, causal=False, pair=False,
                     programs=0, copy_units=32, xcd_remap=False):
    """Attention over `buf` (stacked K, V of shape [2, B, H, S, D]) while the kv chunks arrive:
    chunk arrival[0] is resident, the others are copied from `staged_kv` by a side-stream
    producer in arrival order - a box copy on `copy_units` compute units, then the chunk's flag.
    The kernel runs `programs` persistent workgroups so that the copies find compute units."""
    from syncopate_amd import _lib
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status, trust_flags
    from syncopate_amd.computation.attn import attention_forward

    lib = _lib.load()
    D = q.shape[-1]
    main = torch.cuda.current_stream()
    side = pick_side_streams(1, main, device)[0]
    flags = torch.zeros(len(arrival), dtype=torch.int64, device=device)
    trust_flags(flags)
    out = torch.empty_like(q)
    signals = tables["signal_offsets"].tolist()
    own = arrival[0]
    buf.zero_()
    buf[:, :, :, own * chunk:(own + 1) * chunk].copy_(staged_kv[:, :, :, own * chunk:(own + 1) * chunk])

    def step(i):
        flags.zero_()
        side.wait_stream(main)
        # The kernel is launched first: its persistent workgroups then hold `programs` compute units and the
        # copy kernels get the rest.  A copy kernel that starts first spreads its small workgroups over many
        # compute units, none of which can take an attention workgroup (all registers of a SIMD) until it ends.
        attention_forward(q, buf[0], buf[1], D ** -0.5, out=out, signal_ptr=flags, causal=causal, pair_q_blocks=pair,
                          num_programs=programs, xcd_remap=xcd_remap, **tables)
        with torch.cuda.stream(side):
            for wave in range(1, len(arrival)):
                c = arrival[wave]
                persistent_copy_last_contig(staged_kv[:, :, :, c * chunk:(c + 1) * chunk],
                                            buf[:, :, :, c * chunk:(c + 1) * chunk], num_sms=copy_units)
                _lib.check("syn_flag_set", lib.syn_flag_set(flags.data_ptr() + 8 * signals[wave], 1,
                                                            _lib.stream_handle(side)))
        main.wait_stream(side)

    ms = _timed(step, launches, 2)
    check_status()
    return ms, out


def run_attention_ag(device, launches=5, gated=True):
    """All-gather attention at the headline ring / all-gather configuration: 4096 local q rows, 32 heads,
    against 32768 kv rows as 8 chunks of 4096 in double-ring arrival order, head dim 128; two q
    blocks per workgroup in opposite phases (pair_q_blocks).  Resident (every flag set) in the chained form
    and in the forms that merge after every tile, and gated (224 persistent programs that merge: the
    stand-in producer's copy kernels need the other 32 compute units)."""
    from syncopate_amd.computation._launch import check_status, trust_flags
    from syncopate_amd.computation.attn import attention_forward

    B, H, Sq, Skv, D, chunks = 1, 32, 4096, 32768, 128, 8
    torch.manual_seed(2)
    q = torch.randn(B, H, Sq, D, device=device).bfloat16()
    kv = torch.randn(2, B, H, Skv, D, device=device).bfloat16()
    chunk = Skv // chunks
    arrival = [0, 1, 7, 6, 4, 5, 3, 2]
    cums = [(i + 1) * B * H * Sq for i in range(chunks)]
    tables = dict(wave_offsets=_table([[0, 0, 0, o * chunk] for o in arrival], device),
                  wave_sizes=_table([[B, H, Sq, chunk]] * chunks, device), cum_wave_sizes=_table(cums, device),
                  signal_offsets=_table([-1, 0, 4, 1, 5, 2, 6, 3], device), cum_tiles=cums[-1])
    ones = torch.ones(chunks, dtype=torch.int64, device=device)
    trust_flags(ones)
    out = torch.empty_like(q)
    def resident(**kw):
        return _timed(lambda i: attention_forward(q, kv[0], kv[1], D ** -0.5, out=out, pair_q_blocks=True,
                                                  signal_ptr=ones, **tables, **kw), launches, 3)
    resident()                      # clocks settle
    # one program per pair of q blocks of a wave (512), each XCD's on consecutive pairs (the q blocks of two
    # heads at a time, whose K and V then pass through that XCD's L2 only); a program walks through the
    # eight chunks with its sums in registers and writes its q blocks once
    ms = resident(xcd_remap=True, chain_q_blocks=True)
    check_status()
    # the reference's protocol: 256 persistent workgroups, every tile merged into the output under its q block's lock
    merged_ms = resident(xcd_remap=True, num_programs=256)
    plain_ms = resident()           # one workgroup per pair of q blocks, dealt round-robin over the XCDs
    persistent_ms = resident(num_programs=224, xcd_remap=True)
    s = (q[0, 7].float() @ kv[0, 0, 7].float().t()) * D ** -0.5
    ref = torch.softmax(s, dim=-1) @ kv[1, 0, 7].float()
    err = ((out[0, 7].float() - ref).abs().max() / ref.abs().max()).item()
    result = {"launches": launches, "ms": ms, "flop": 4.0 * B * H * Sq * Skv * D, "max_rel_err_vs_fp32": err,
              "form": "chain_q_blocks, 512 programs, xcd_remap", "ms_256_programs_merge_per_tile": merged_ms,
              "ms_224_programs_resident": persistent_ms, "ms_one_workgroup_per_pair_no_xcd_remap": plain_ms}
    if not gated:
        return result
    buf = torch.empty_like(kv)
    gated_ms, gated_out = _gated_attention(q, kv, buf, arrival, chunk, tables, launches, device, pair=True, programs=224,
                                           xcd_remap=True)
    gated_err = ((gated_out[0, 7].float() - ref).abs().max() / ref.abs().max()).item()
    # the device warms up over these launches (consecutive launches of one kernel get 1 % slower each): the resident
    # form is timed again behind the gated one and the overhead is quoted against the mean of the two
    persistent_after_ms = resident(num_programs=224, xcd_remap=True)
    baseline_ms = 0.5 * (persistent_ms + persistent_after_ms)
    result.update({"ms_gated": gated_ms, "gated_max_rel_err_vs_fp32": gated_err,
                   "gathered_kv_matches": bool(torch.equal(buf, kv)),
                   "ms_224_programs_resident_after_gated": persistent_after_ms,
                   "flag_wait_overhead_pct": 100.0 * (gated_ms - baseline_ms) / baseline_ms,
                   "gated_tflops": result["flop"] / (gated_ms * 1e-3) / 1e12})
    return result


def run_attention_a2a(device, launches=10, gated=True):
    """All-to-all (Ulysses) attention of rank 0 of 8: the whole sequence of 16384, 4 local heads, head
    dim 128, causal; Q, K and V arrive as 8 sequence chunks of 2048 (the rank's own first), and
    arrival w unlocks (Q_w x KV_w), (Q_p x KV_w) and (Q_w x KV_p) for every earlier p: 64 waves.
    The launch is planned (work_plan.plan_attention_work): one program per compute unit, every head's visits on
    two XCDs, visits to the same q blocks in a row as one segment, segments cut to a program's fair share.
    Resident, and with the chunks copied in behind flags.  flop counts the causal half."""
    from syncopate_amd import _lib
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.common_descriptors import build_all_to_all_plan_dim
    from syncopate_amd.communication.comm_runtime.persistent_copy import persistent_copy_last_contig
    from syncopate_amd.communication.comm_runtime.streams import pick_side_streams
    from syncopate_amd.computation._launch import check_status, trust_flags
    from syncopate_amd.computation.attn import attention_forward, plan_attention_work
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules
    from syncopate_amd.interface.wave_tables import all2all_attn_tables

    world, B, H, S_local, D = 8, 1, 32, 2048, 128
    H_local, S = H // world, world * S_local
    plans = {r: build_all_to_all_plan_dim(shape=(3, B, H, S_local, D), dtype=torch.bfloat16, mesh_size=world, rank=r,
                                          src_buffer="src", dst_buffer="dst", src_split_axis=3, dst_split_axis=2,
                                          transfer_kind="pull", compute_producer=False) for r in range(world)}
    gen = CommGenerator(plans)
    gen.plan_signals()
    host = all2all_attn_tables(lower_comm_plan_to_raw_schedules(gen)[RANK]["dst"], {"batch": 1, "head": 2, "seq": 3})
    tables = dict(wave_offsets=_table(host.wave_offsets, device), wave_sizes=_table(host.wave_sizes, device),
                  cum_wave_sizes=_table(host.cum_wave_sizes, device), signal_offsets=_table(host.signal_offsets, device),
                  cum_tiles=host.cum_tiles)
    num_flags = max(host.signal_offsets) + 1
    torch.manual_seed(4)
    qkv = torch.randn(3, B, H_local, S, D, device=device).bfloat16()
    scale = D ** -0.5
    # the benchmark owns these flag arrays and keeps the kernels' precondition: nothing reads a chunk before its flag
    ones = torch.ones(num_flags, dtype=torch.int64, device=device)
    flags = torch.zeros(num_flags, dtype=torch.int64, device=device)
    trust_flags(ones, flags)
    out = torch.empty_like(qkv[0])

    def plan_for(causal, programs, **limits):
        return plan_attention_work(host.wave_offsets, host.wave_sizes, host.cum_wave_sizes, causal=causal,
                                   num_programs=programs, **limits)

    def planned(plan, causal, signal=ones, src=qkv, sm_scale=scale):
        return attention_forward(src[0], src[1], src[2], sm_scale, out=out, signal_ptr=signal, causal=causal,
                                 pair_q_blocks=True, xcd_remap=True, work_plan=plan, **tables)

    causal_plan = plan_for(True, 256, max_blocks="fair")
    plain_plan = plan_for(False, 256)
    gated_plan = plan_for(True, 224, max_visits=1)
    # (planning is host work of a few tens of milliseconds during which the device idles and its clock drops:
    # every timed region here follows some 15 ms of the same kernel)
    warm = 40
    ms = _timed(lambda i: planned(causal_plan, True), launches, warm)
    # the reference's tests run this flow with sm_scale = 1.0 (tests/test_all2all_attn_transform.py:297)
    unit_ms = _timed(lambda i: planned(causal_plan, True, sm_scale=1.0), launches, warm // 2)
    check_status()
    noncausal_ms = _timed(lambda i: planned(plain_plan, False), launches, warm // 2)
    # the reference's launch shape: one program per tile, the hardware's scheduler deals them
    one_tile_ms = _timed(lambda i: attention_forward(qkv[0], qkv[1], qkv[2], scale, out=out, signal_ptr=ones, causal=True,
                                                     **tables), launches, warm // 2)
    rows = torch.arange(3, S, 61, device=device)

    def error(sm_scale, head=1):
        s = (qkv[0, 0, head][rows].float() @ qkv[1, 0, head].float().t()) * sm_scale
        s = s.masked_fill(torch.arange(S, device=device)[None, :] > rows[:, None], float("-inf"))
        ref = torch.softmax(s, dim=-1) @ qkv[2, 0, head].float()
        return ((out[0, head][rows].float() - ref).abs().max() / ref.abs().max()).item()

    planned(causal_plan, True)
    err = error(scale)
    planned(causal_plan, True, sm_scale=1.0)
    err_unit = error(1.0)

    result = {"launches": launches, "waves": len(host.signal_offsets), "ms_causal": ms, "ms_non_causal": noncausal_ms,
              "form": "planned: 256 programs, head groups, segments cut to a fair share, xcd_remap",
              "plan_causal": {"segments": causal_plan.segments, "merged_segments": causal_plan.merged_segments,
                              "kv_blocks_per_program_max": max(causal_plan.program_cost),
                              "kv_blocks_per_program_fair": sum(causal_plan.program_cost) / 256},
              "flop_causal": 2.0 * B * H_local * S * S * D, "flop_non_causal": 4.0 * B * H_local * S * S * D,
              "max_rel_err_vs_fp32": err, "ms_causal_sm_scale_1": unit_ms, "max_rel_err_vs_fp32_sm_scale_1": err_unit,
              "ms_causal_one_program_per_tile": one_tile_ms}
    result["causal_tflops"] = result["flop_causal"] / (ms * 1e-3) / 1e12
    result["non_causal_tflops"] = result["flop_non_causal"] / (noncausal_ms * 1e-3) / 1e12
    if not gated:
        return result

    # gated: Q, K and V of sequence chunk w land together, then flag w.  224 programs, so that the stand-in
    # producer's copy kernels find compute units, and a plan of single visits: a chunk's work is then spread over
    # as many programs as it has visits, and what is left to do when the last chunk lands is one visit per program.
    lib = _lib.load()
    main = torch.cuda.current_stream()
    side = pick_side_streams(1, main, device)[0]
    buf = torch.zeros_like(qkv)
    # arrival order of the sequence chunks and each arrival's flag: the (Q_w x KV_w) waves of the table
    diag = [i for i in range(len(host.signal_offsets))
            if host.wave_offsets[i][2] == host.wave_offsets[i][3] and host.wave_sizes[i][2] == host.wave_sizes[i][3]]
    arrivals = [(host.wave_offsets[i][2] // S_local, host.signal_offsets[i]) for i in diag]

    # producer (a): one box copy of the stacked buffer per chunk, then the flag kernel - two kernels per chunk
    def copy_then_flag():
        for c, sig in arrivals:
            persistent_copy_last_contig(qkv[:, :, :, c * S_local:(c + 1) * S_local],
                                        buf[:, :, :, c * S_local:(c + 1) * S_local], num_sms=32)
            if sig >= 0:
                _lib.check("syn_flag_set", lib.syn_flag_set(flags.data_ptr() + 8 * sig, 1, _lib.stream_handle(side)))

    # producer (b): ONE kernel of 32 workgroups that walks the list of every chunk's twelve rows-of-a-head and
    # raises a chunk's flag behind its last piece - no kernel boundary, with its cache write-back and
    # invalidate, while the attention kernel runs
    records = []
    for c, sig in arrivals:
        pieces = [(t, h) for t in range(3) for h in range(H_local)]
        for n, (t, h) in enumerate(pieces):
            src_rows = qkv[t, 0, h, c * S_local:(c + 1) * S_local]
            dst_rows = buf[t, 0, h, c * S_local:(c + 1) * S_local]
            flag = flags.data_ptr() + 8 * sig if (n + 1 == len(pieces) and sig >= 0) else 0
            records.append([dst_rows.data_ptr(), src_rows.data_ptr(), src_rows.numel() * 2 // 16, flag, 1, 0])
    records = torch.tensor(records, dtype=torch.int64, device=device)
    tickets = torch.zeros(records.shape[0], dtype=torch.int32, device=device)

    def one_list_kernel():
        _lib.check("syn_copy_flag_list_async",
                   lib.syn_copy_flag_list_async(records.data_ptr(), records.shape[0], tickets.data_ptr(), 32,
                                                _lib.stream_handle(side)))

    def gated_ms(producer):
        def step(i):
            flags.zero_()
            side.wait_stream(main)
            # the kernel first: its persistent programs then hold 224 compute units and the copies get the rest
            planned(gated_plan, True, signal=flags, src=buf)
            with torch.cuda.stream(side):
                producer()
            main.wait_stream(side)
        buf.zero_()
        t = _timed(step, launches, 5)
        check_status()
        return t, bool(torch.equal(buf, qkv)), error(scale)

    resident_before = _timed(lambda i: planned(gated_plan, True), launches, warm)
    list_ms, list_ok, list_err = gated_ms(one_list_kernel)
    resident_between = _timed(lambda i: planned(gated_plan, True), launches, 5)
    pair_ms, pair_ok, pair_err = gated_ms(copy_then_flag)
    resident_after = _timed(lambda i: planned(gated_plan, True), launches, 5)
    # the device's clock moves over these launches: each gated form is quoted against the resident runs around it
    result.update({"gated_form": "224 programs, single visits; producer: one list kernel of 32 workgroups",
                   "ms_causal_224_programs_resident": [resident_before, resident_between, resident_after],
                   "ms_causal_gated": list_ms, "gated_max_rel_err_vs_fp32": max(list_err, pair_err),
                   "gathered_qkv_matches": list_ok and pair_ok,
                   "flag_wait_overhead_pct": 100.0 * (list_ms / (0.5 * (resident_before + resident_between)) - 1.0),
                   "gated_causal_tflops": result["flop_causal"] / (list_ms * 1e-3) / 1e12,
                   "ms_causal_gated_copy_kernel_and_flag_kernel_per_chunk": pair_ms,
                   "flag_wait_overhead_pct_copy_kernel_and_flag_kernel_per_chunk":
                       100.0 * (pair_ms / (0.5 * (resident_between + resident_after)) - 1.0)})
    return result


# -------------------------------------------------------------------------------- CPU baselines

def run_attention_slot(device, launches=10):
    """What the pieces of the paired attention kernel's slot cost beside each other (`syn_probe_attn_slot`): the 64
    MFMAs of a slot on register operands, fed from LDS through the kernel's reads, beside the other group's softmax,
    with the fills, with the first fragments of a phase asked for early, on constant and on random operands, and with
    the products as pairs of 16x16x32 MFMAs instead of 32x32x16 ones.  Per
    configuration: time and shader-clock cycles per slot, the clock the device held (cycles / time), and the rate
    the slot's products run at, as a fraction of the matrix pipes' peak.  2048 matrix-pipe cycles per slot."""
    from syncopate_amd import _lib

    lib = _lib.load()
    workgroups, iters = 256, 2000
    pool = torch.randn((workgroups * 65536 + (32 << 20)) // 2, device=device).bfloat16()
    sink = torch.empty(workgroups * 512, dtype=torch.float32, device=device)
    cycles = torch.zeros(2, dtype=torch.int64, device=device)
    stream = _lib.stream_handle(torch.cuda.current_stream())
    PRODUCTS, SOFTMAX, LDS, FILLS, PREFETCH, RANDOM, PRIVATE, NARROW = 1, 2, 4, 8, 16, 32, 64, 128
    configs = (("products_register_operands", PRODUCTS),
               ("products_from_lds", PRODUCTS | LDS),
               ("softmax_alone", SOFTMAX),
               ("products_from_lds_beside_softmax", PRODUCTS | LDS | SOFTMAX),
               ("products_from_lds_beside_softmax_with_fills", PRODUCTS | LDS | SOFTMAX | FILLS),
               ("same_fragments_asked_for_a_phase_early", PRODUCTS | LDS | SOFTMAX | FILLS | PREFETCH),
               ("same_fills_that_miss_the_l2", PRODUCTS | LDS | SOFTMAX | FILLS | PRIVATE),
               ("products_register_operands_random", PRODUCTS | RANDOM),
               ("products_from_lds_random", PRODUCTS | LDS | RANDOM),
               ("products_from_lds_beside_softmax_random", PRODUCTS | LDS | SOFTMAX | RANDOM),
               ("products_from_lds_beside_softmax_with_fills_random", PRODUCTS | LDS | SOFTMAX | FILLS | RANDOM),
               ("same_fragments_asked_for_a_phase_early_random", PRODUCTS | LDS | SOFTMAX | FILLS | PREFETCH | RANDOM),
               # the same slot with every 32x32x16 product as two 16x16x32 products (the form the kernel uses)
               ("narrow_products_register_operands_random", PRODUCTS | RANDOM | NARROW),
               ("narrow_products_from_lds_beside_softmax_random", PRODUCTS | LDS | SOFTMAX | RANDOM | NARROW),
               ("narrow_products_from_lds_beside_softmax_with_fills_random", PRODUCTS | LDS | SOFTMAX | FILLS | RANDOM | NARROW),
               ("narrow_products_from_lds_beside_softmax_with_fills", PRODUCTS | LDS | SOFTMAX | FILLS | NARROW))
    out = {"workgroups": workgroups, "slots_per_launch": iters, "launches": launches, "matrix_pipe_cycles_per_slot": 2048}
    flop_per_slot = workgroups * 4 * 64 * 32768.0
    for name, what in (("warm-up", configs[-2][1]),) + configs:
        def probe(i):
            _lib.check("syn_probe_attn_slot", lib.syn_probe_attn_slot(pool.data_ptr(), pool.numel() * 2, workgroups, iters, what,
                                                                     sink.data_ptr(), cycles.data_ptr(), stream))
        ms = _timed(probe, launches, 2)
        if name == "warm-up":           # the clock the device holds depends on what it has just been doing
            continue
        cyc = cycles.tolist()
        per_slot = max(cyc) / iters
        entry = {"ns_per_slot": ms * 1e6 / iters, "cycles_per_slot": per_slot, "clock_GHz": per_slot / (ms * 1e6 / iters)}
        if what & PRODUCTS:
            entry["products_tflops"] = flop_per_slot / (ms * 1e-3 / iters) / 1e12
            entry["products_pct_bf16_mfma_peak"] = 100.0 * entry["products_tflops"] / MFMA_BF16_PEAK_TFLOPS
        out[name] = entry
    return out


def _host_cpu():
    """What the CPU baselines ran on: the model string, the cores the host shows and the threads used.  A one-GPU box
    of the pool gives a job 16 cores whatever the host shows (OMP_NUM_THREADS is 16 there), so the baselines use
    at most that many threads."""
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    threads = min(16, os.cpu_count() or 1)
    return {"cpu_model": model, "host_cores": os.cpu_count(), "threads": threads,
            "threads_note": "capped at the 16 cores a one-GPU job of this pool is given"}


def cpu_baseline(state):
    """torch CPU matmul over the gathered operands (fp32 values of the same bf16 inputs):
    a bounded sample of the same GEMM — a band of rows of A against all of B."""
    from oracle import numerics

    host = _host_cpu()
    threads = host["threads"]
    torch.set_num_threads(threads)
    sample_rows = M
    a = state["a"][:sample_rows].cpu()
    b = state["b"].cpu()
    numerics.gemm_fp32(a[:128], b)          # warm-up
    reps, spent = 0, 0.0
    while spent < 8.0 and reps < 40:
        t0 = time.perf_counter()
        numerics.gemm_fp32(a, b)
        spent += time.perf_counter() - t0
        reps += 1
    flop = 2.0 * sample_rows * N * K * reps
    return {
        "value": flop / spent / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "torch_num_threads": torch.get_num_threads(),
        "cpu_model": host["cpu_model"],
        "host_cores": host["host_cores"],
        "threads_note": host["threads_note"],
        "kind": "port",
        "sample": f"{reps} x torch CPU fp32 matmul of A[:{sample_rows}] (bf16 values) with all of B, "
                  f"{spent:.1f} s",
    }


def cpu_baselines_other():
    """The other workloads on the host's cores, bounded samples, one to three repetitions each:
    the reference's CPU case (mesh 4: plan -> signals -> lowered schedules -> op lists, then the
    fp16 matmul of the gathered A), the chunked reduce, and both attention shapes through
    torch's CPU attention over the gathered operands."""
    import numpy as np

    from oracle import numerics
    from syncopate_amd.communication.code_gen import CommGenerator
    from syncopate_amd.communication.common_descriptors import build_all_gather_plan_1d_swizzle
    from syncopate_amd.interface import lower_comm_plan_to_raw_schedules

    host = _host_cpu()
    threads = host["threads"]
    torch.set_num_threads(threads)
    result = {"cores": threads, "cpu_model": host["cpu_model"], "host_cores": host["host_cores"]}

    def compile_c1():
        plans = {r: build_all_gather_plan_1d_swizzle((4096, 512), torch.float16, 0, 4, r, "a", "pull") for r in range(4)}
        gen = CommGenerator(plans)
        gen.plan_signals()
        schedules = lower_comm_plan_to_raw_schedules(gen)
        gen.generate_code_for_plan()
        return [schedules[r]["a"].gen_block_offset_lists() for r in range(4)]
    compile_c1()
    t0 = time.perf_counter()
    for _ in range(5):
        compile_c1()
    result["c1_compile_us"] = (time.perf_counter() - t0) / 5 * 1e6
    torch.manual_seed(0)
    a = torch.cat([torch.randn(1024, 512).half() for _ in range(4)])
    b = torch.randn(512, 1024).half()
    a @ b
    t0 = time.perf_counter()
    for _ in range(3):
        a @ b
    result["c1_fp16_matmul_ms"] = (time.perf_counter() - t0) / 3 * 1e3
    t0 = time.perf_counter()
    a.float() @ b.float()
    result["c1_fp32_matmul_ms"] = (time.perf_counter() - t0) * 1e3

    rng = np.random.default_rng(1)
    recv = rng.standard_normal((8, 1024, 8192), dtype=np.float32)
    local = rng.standard_normal((8192, 8192), dtype=np.float32)
    t0 = time.perf_counter()
    numerics.ring_reduce(recv, local, 0, dtype="bf16")
    spent = time.perf_counter() - t0
    result["c3_reduce_ms"] = spent * 1e3
    result["c3_reduce_GBps"] = 9 * 1024 * 8192 * 2 / spent / 1e9
    result["c3_reduce_sample"] = "1 x numpy ring reduce of 8 x (1024, 8192), one bf16 rounding per add"

    torch.manual_seed(2)
    for name, (H, Sq, Skv, causal, heads) in {"c5_attention": (32, 4096, 32768, False, 8),
                                              "c4_attention_causal": (4, 16384, 16384, True, 2)}.items():
        q = torch.randn(1, heads, Sq, 128)
        k = torch.randn(1, heads, Skv, 128)
        v = torch.randn(1, heads, Skv, 128)
        t0 = time.perf_counter()
        numerics.sdpa_fp32(q, k, v, 128 ** -0.5, causal=causal)
        spent = time.perf_counter() - t0
        flop = 4.0 * heads * Sq * Skv * 128 * (0.5 if causal else 1.0)
        result[name + "_tflops"] = flop / spent / 1e12
        result[name + "_sample"] = (f"1 x torch CPU fp32 attention of {heads} of the {H} heads "
                                    f"({Sq} q rows x {Skv} kv rows), {spent:.1f} s")
    return result


def _traffic():
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def main():
    global BM, BN, NUM_SMS, LEAD_OPS, XCD_REMAP, LEAD_ON_COMPUTE_STREAM
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step is ~0.45 ms: the defaults time a few hundred of them (the whole run still takes well under a minute)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", default="", help="comma-separated subset of: " + ", ".join(SECTIONS) +
                    " (ag_gemm always runs; for profiler runs that want one kernel)")
    ap.add_argument("--no-graph", action="store_true", help="launch every step's operations from the host "
                    "instead of replaying them as one HIP graph")
    ap.add_argument("--resident-only", action="store_true",
                    help="skip every flag-gated run (for hardware-counter runs, which serialise kernels: "
                         "a gated consumer would wait for copies that can only start after it)")
    ap.add_argument("--copy-blocks", type=int, default=0,
                    help="0: the producer's chunk copies are hipMemcpyAsync (default); N > 0: the library's "
                         "streaming copy kernel with N workgroups")
    ap.add_argument("--tile", default=f"{BM}x{BN}", help="output tile of the consumer, e.g. 256x256 or 256x224")
    ap.add_argument("--programs", type=int, default=NUM_SMS, help="persistent programs of the consumer")
    ap.add_argument("--xcd-remap", action="store_true",
                    help="each XCD works on a contiguous range of tile ids (one chunk's tiles at a time)")
    ap.add_argument("--fuse-flags", action="store_true",
                    help="with --copy-blocks N: one kernel per chunk that copies and then sets the flag")
    ap.add_argument("--split-device", type=int, default=0, metavar="N",
                    help="give N compute units (a multiple of 8) to the producer's stream and the rest to the "
                         "consumer's, by compute-unit masks")
    ap.add_argument("--lead-copy-blocks", type=int, default=LEAD_COPY_BLOCKS,
                    help="N > 0: a leading chunk copy and its flag write are one kernel of N workgroups")
    ap.add_argument("--list-blocks", type=int, default=LIST_BLOCKS,
                    help="N > 0: the producer is ONE kernel of N workgroups that walks the list of chunk copies and raises "
                         "each chunk's flag (two kernels with --lead-ops: the leading chunks, then the rest)")
    ap.add_argument("--wave0-flag", type=int, default=-1,
                    help="N >= 0 (with --lead-ops 0): the consumer is launched together with the first copy and its "
                         "wave 0 - the rank's own, resident chunk - waits for flag N, so that the kernel's launch "
                         "and the cross-queue event leave the path while it spins until chunk N + 1 has landed")
    ap.add_argument("--flag-write-values", action="store_true",
                    help="with --no-graph: flag writes are stream memory operations instead of one-wavefront kernels")
    ap.add_argument("--lead-on-compute-stream", action="store_true",
                    help="the leading ops run on the compute stream itself, in front of the kernel")
    ap.add_argument("--lead-ops", type=int, default=LEAD_OPS,
                    help="the consumer launch waits for this many leading ops of the side stream (0: none)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one rank's share on ONE GPU: the other ranks of the mesh are "
                 "simulated by a side-stream producer; run it with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X (no GPU visible)")
    from syncopate_amd import _lib

    _lib.load()      # fail loudly if the HIP library has not been built
    BM, BN = (int(x) for x in args.tile.lower().split("x"))
    NUM_SMS = args.programs
    LEAD_OPS = args.lead_ops
    XCD_REMAP = args.xcd_remap
    LEAD_ON_COMPUTE_STREAM = args.lead_on_compute_stream
    only = set(x for x in args.only.split(",") if x) or set(SECTIONS)
    unknown = only - set(SECTIONS)
    if unknown:
        sys.exit(f"--only: unknown section(s) {sorted(unknown)}")
    if args.no_cpu_baseline:
        only.discard("cpu")
    gated = not args.resident_only
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    if args.split_device and (args.copy_blocks == 0 or not args.no_graph):
        sys.exit("--split-device splits the compute units between two streams: it needs the copy kernel "
                 "(--copy-blocks N) and launches from the host (--no-graph; a graph's kernel nodes carry no mask)")
    state = build_ag_gemm(device, args.copy_blocks, args.split_device, args.fuse_flags,
                          lead_copy_blocks=args.lead_copy_blocks, flag_write_values=args.flag_write_values,
                          list_blocks=args.list_blocks)
    if args.wave0_flag >= 0:
        state["tables"]["signal_offsets"][0] = args.wave0_flag
    with torch.cuda.stream(state["ctx"].compute_stream):
        wall_ms, gated_ms, no_lead_ms, resident_ms = run_ag_gemm(state, args.steps, args.warmup, args.resident_only,
                                                                 not args.no_graph)
        torch.cuda.synchronize()
        traffic_calibration(device)
        err, gathered = check_ag_gemm(state)
        ceiling = run_mfma_ceiling(device, state) if "mfma_ceiling" in only else None
    torch.cuda.synchronize()

    flop = 2.0 * M * N * K
    value = flop / (wall_ms * 1e-3) / 1e12
    kernel_tflops = flop / (gated_ms * 1e-3) / 1e12
    kernel_name = (f"gemm_wave_kernel<bf16, {'EarlyPipe16' if (BM, BN) in ((256, 256), (256, 224)) else 'SlabPipe<3 stages>'}, "
                   f"{BM}x{BN}, {8 if EIGHT_WAVES else 4} wavefronts, consumer>")
    traffic = _traffic().get("gemm_consumer_256x256_224_programs", {}) if (BM, BN, NUM_SMS) == (256, 256, 224) else {}
    line = {
        "metric": "AG-GEMM TFLOP/s",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_steps": SETTLE_STEPS,
        "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "resident_only": bool(args.resident_only),
        "config": {
            "workload": "AG-GEMM one rank's share, simulated mesh=8: A (8192,8192) bf16 arriving as 8 chunks "
                        "of 1024 rows in swizzled order behind flags, B (8192,3584) bf16 stored [N,K], "
                        "fp32 accumulate",
            "tile": [BM, BN, BK],
            "programs": NUM_SMS,
            "lead_ops": LEAD_OPS,
            "lead_copy_blocks": args.lead_copy_blocks,
            "producer": "side stream: " + (
                f"one kernel of {args.copy_blocks} workgroups per chunk that copies, then sets the flag"
                if args.fuse_flags else
                ("hipMemcpyAsync" if args.copy_blocks == 0 else f"copy kernel of {args.copy_blocks} workgroups")
                + " + flag-set kernel per chunk"),
            "launch": "eager" if args.no_graph else "a hip graph of two steps, replayed steps/2 times",
            "split_device": state["ctx"].cu_split,
        },
        "pct_bf16_mfma_peak": 100.0 * value / MFMA_BF16_PEAK_TFLOPS,
        # gated step against the same kernel with every chunk resident: the whole iteration, lead-in copies,
        # flag reset and stream joins included
        "flag_wait_overhead_pct": 100.0 * (wall_ms - resident_ms) / resident_ms,
        # the kernel alone, in the launch shape of the timed steps (behind the leading chunks)
        "kernel_only_gated_over_resident_pct": 100.0 * (gated_ms - resident_ms) / resident_ms,
        "kernel_launches_timed": args.steps,
        "kernel_ms_gated": gated_ms,
        "kernel_ms_gated_launched_with_first_copy": no_lead_ms,
        "kernel_ms_resident": resident_ms,
        "resident_tflops": flop / (resident_ms * 1e-3) / 1e12,
        "host_compile_ms": state["compile_ms"],
        "max_rel_err_vs_fp32": err,
        "gathered_a_matches": gathered,
        "roofline": {
            "kernel": kernel_name,
            "bound": "mfma",
            "achieved": kernel_tflops,
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": kernel_tflops / MFMA_BF16_PEAK_TFLOPS,
            "traffic": traffic.get("bytes_per_launch"),
            "traffic_source": traffic.get("source"),
        },
    }
    if ceiling is not None:
        line["mfma_ceiling"] = ceiling
        random_ceiling = ceiling.get("random_operands_256_workgroups_tflops")
        if random_ceiling:
            line["roofline"]["frac_of_random_operand_mfma_ceiling"] = kernel_tflops / random_ceiling
    if "library" in only:
        line["library_baselines"] = run_library_baselines(device, state)
    steps_small = max(20, min(args.steps, 60))
    if "throttled" in only and gated:
        line["throttled_producer"] = run_throttled(device, 20)
    if "reduce" in only:
        reduce_ms, reduce_bytes, reduce_padded_ms = run_reduce(device, max(args.steps, 30), args.warmup)
        line.update({
            "rs_reduce_launches": max(args.steps, 30),
            "rs_reduce_GBps": reduce_bytes / (reduce_ms * 1e-3) / 1e9,
            "rs_reduce_us": reduce_ms * 1e3,
            "rs_reduce_pct_hbm_peak": 100.0 * reduce_bytes / (reduce_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "rs_reduce_received_blocks_4KiB_further_apart_GBps": reduce_bytes / (reduce_padded_ms * 1e-3) / 1e9,
        })
        ceiling_reads = run_hbm_read_ceiling(device)
        line["hbm_read_ceiling"] = ceiling_reads
        # the reduce moves its bytes (8/9 of them reads at that placement, 1/9 writes) at this fraction of the
        # rate at which the same reads alone can be had
        line["rs_reduce_over_eight_stream_read_ceiling"] = line["rs_reduce_GBps"] / ceiling_reads["eight_streams_16MiB_apart_skewed_walk_GBps"]
    if "box_copies" in only:
        boxes = run_box_copies(device, steps_small, args.warmup)
        line["box_copy_launches"] = steps_small
        line["box_copy_GBps"] = {name: traffic_ / (ms * 1e-3) / 1e9 for name, (ms, traffic_) in boxes.items()}
        line["box_copy_us"] = {name: ms * 1e3 for name, (ms, _) in boxes.items()}
    if "gemm_rs" in only:
        rs = run_gemm_rs(device, steps_small, args.warmup, gated)
        line["gemm_rs"] = {
            "launches": rs["launches"],
            "producer_tflops": rs["flop"] / (rs["producer_ms"] * 1e-3) / 1e12,
            "producer_pct_bf16_mfma_peak": 100.0 * rs["flop"] / (rs["producer_ms"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "producer_ms": rs["producer_ms"],
            "producer_form": "256 programs, xcd_remap",
            "producer_ms_without_xcd_remap": rs["producer_ms_without_xcd_remap"],
        }
        if gated:
            line["gemm_rs"].update({
                "fused_step_ms": rs["fused_step_ms"],
                "fused_step_ms_by_programs": rs["fused_step_ms_by_programs"],
                "fused_step_tflops": rs["flop"] / (rs["fused_step_ms"] * 1e-3) / 1e12,
                "fused_step_over_producer_pct": 100.0 * (rs["fused_step_ms"] - rs["producer_ms"]) / rs["producer_ms"],
                "direct_reduce_form_ms": rs["direct_reduce_form_ms"],
                "direct_reduce_form_tflops": rs["flop"] / (rs["direct_reduce_form_ms"] * 1e-3) / 1e12,
                "direct_reduce_form_matches": rs["direct_reduce_form_matches"],
                "remote_store_form_ms": rs["remote_store_form_ms"],
                "remote_store_form_gemm_ms": rs["remote_store_form_gemm_ms"],
                "remote_store_form_tflops": rs["flop"] / (rs["remote_store_form_ms"] * 1e-3) / 1e12,
                "remote_store_form_over_producer_pct": 100.0 * (rs["remote_store_form_ms"] - rs["producer_ms"]) / rs["producer_ms"],
                "remote_store_form_matches": rs["remote_store_form_matches"],
                "reduce_matches": rs["reduce_matches"],
                "pushed_chunks_match": rs["pushed_chunks_match"],
            })
    if "attn_ag" in only:
        ag = run_attention_ag(device, gated=gated)
        line["attn_allgather"] = dict(ag, tflops=ag["flop"] / (ag["ms"] * 1e-3) / 1e12,
                                      pct_bf16_mfma_peak=100.0 * ag["flop"] / (ag["ms"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS)
    if "attn_a2a" in only:
        line["attn_all2all"] = run_attention_a2a(device, gated=gated)
    if "attn_slot" in only:
        line["attn_slot_probe"] = run_attention_slot(device)
        slot = line["attn_slot_probe"]["narrow_products_from_lds_beside_softmax_with_fills_random"]["products_tflops"]
        # the kernels' rates against the bare slot loop's (same MFMAs, LDS reads, softmax and fills on random operands,
        # nothing else): what is left is the kernels' own doing, the rest is the board's power limit
        if "attn_allgather" in line:
            line["attn_allgather"]["frac_of_slot_loop_on_random_operands"] = line["attn_allgather"]["tflops"] / slot
        if "attn_all2all" in line:
            line["attn_all2all"]["non_causal_frac_of_slot_loop_on_random_operands"] = line["attn_all2all"]["non_causal_tflops"] / slot
    if "cpu" in only:
        line["cpu_baseline"] = cpu_baseline(state)
        line["cpu_baselines_other"] = cpu_baselines_other()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
