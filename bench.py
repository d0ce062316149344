"""Benchmark of the chunk-scheduled AG+GEMM on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one fused all-gather+GEMM iteration of rank 0 of a simulated mesh of 8
(M, K, N = 8192, 8192, 3584): flags reset, the 7 peer chunks of A (1024 x 8192 bf16 each)
copied into the symmetric buffer on a side stream in the order the lowered schedule
prescribes (copy, then flag), the consumer GEMM (8192 x 8192 x 3584) on the compute stream
waiting on each chunk's flag.  All operands are resident in HBM before the timed region.
The W warm-up steps follow SETTLE_STEPS further untimed steps (an idle device's clocks settle
over the first ~10 ms of work); the timed region is exactly K steps.  Prints ONE JSON line.
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
# Bytes one launch of the 256x256 consumer kernel moves between L2 and the fabric: FETCH_SIZE and
# WRITE_SIZE of two counter runs of `bench.py --resident-only`, scaled by the readings of the
# library's copy kernel (profiles/bench_kernels_hbm_traffic.txt).  Counter runs
# serialise kernels, so this cannot be sampled while the benchmark itself runs.
GEMM_TRAFFIC_BYTES_PER_LAUNCH = 823.1e6

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


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def build_ag_gemm(device, copy_blocks=0, split_units=0, fuse_flags=False):
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
    ctx = CommContext(RANK, info, device=device, copy_blocks=copy_blocks, flag_sets=2, fuse_flags=fuse_flags)
    rows = M // WORLD
    for r in range(WORLD):     # every rank's symmetric buffer holds its own shard
        ctx.comm_buffers["a"][r][r * rows:(r + 1) * rows].copy_(a[r * rows:(r + 1) * rows])
    dev_tables = dict(
        cur_wave_sizes=torch.tensor(tables.block_shapes, dtype=torch.int32, device=device),
        wave_offsets=torch.tensor(tables.block_offsets, dtype=torch.int32, device=device),
        signal_offsets=torch.tensor(tables.signal_offsets, dtype=torch.int32, device=device),
        cum_tiles=tables.cum_tiles,
    )
    c = torch.empty(M, N, dtype=torch.bfloat16, device=device)
    return dict(a=a, b=b, c=c, ctx=ctx, tables=dev_tables, compile_ms=compile_ms)


def run_ag_gemm(state, steps, warmup, resident_only=False, use_graph=True):
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.gemm import gemm

    ctx, b, c, tables = state["ctx"], state["b"], state["c"], state["tables"]
    symm = ctx.comm_buffers["a"][RANK]
    stream = torch.cuda.current_stream()

    def consumer(flag_words):
        gemm(symm, b, c, WORLD, NUM_SMS, BM, BN, BK, GROUP_M, signal_ptr=flag_words, xcd_remap=XCD_REMAP,
             eight_waves=EIGHT_WAVES, **tables)

    def fused_step():
        cur = torch.cuda.current_stream()
        ctx.reset_signals()               # switches to the zeroed flag set
        ctx.start_after(cur)
        ctx.execute(lead_ops=LEAD_OPS)
        ctx.wait_lead(cur)                # the kernel starts behind the first two chunk copies (3x faster before it does)
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
                ctx.execute(lead_ops=lead)
                if lead:
                    ctx.wait_lead(stream)
                begin[i].record(stream)
                consumer(ctx.recv_signal_bufs[RANK])
                end[i].record(stream)
                ctx.end_before(stream)
            torch.cuda.synchronize()
            return sum(s.elapsed_time(e) for s, e in zip(begin, end)) / count
        gated_kernel_ms = kernel_ms(steps, LEAD_OPS)
        no_lead_kernel_ms = kernel_ms(min(steps, 20), 0) if LEAD_OPS else gated_kernel_ms
    check_status()
    ctx.check_status()

    # ---- same kernel, every chunk resident and every flag already set ----
    resident_flags = torch.ones_like(ctx.recv_signal_bufs[RANK])
    for _ in range(warmup):
        consumer(resident_flags)
    torch.cuda.synchronize()
    begin, end = _events(steps), _events(steps)
    for i in range(steps):
        begin[i].record(stream)
        consumer(resident_flags)
        end[i].record(stream)
    torch.cuda.synchronize()
    resident_kernel_ms = sum(s.elapsed_time(e) for s, e in zip(begin, end)) / steps
    check_status()
    if resident_only:
        wall_ms = gated_kernel_ms = no_lead_kernel_ms = resident_kernel_ms
    return wall_ms, gated_kernel_ms, no_lead_kernel_ms, resident_kernel_ms


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


def run_reduce(device, steps, warmup):
    """GEMM+RS chunked reduce of the headline GEMM+RS configuration: 8 x (1024, 8192) bf16 -> (1024, 8192).
    Launches rotate over three sets of operands (3 x 151 MB, more than the 256 MB of memory-side
    cache) so that every launch streams from HBM; the batch is timed as a whole."""
    from syncopate_amd.computation.reduce import ring_reduce

    world, rows, n, sets = 8, 1024, 8192, 3
    torch.manual_seed(1)
    recv = [torch.randn(world, rows, n, device=device).bfloat16() for _ in range(sets)]
    local = [torch.randn(world * rows, n, device=device).bfloat16() for _ in range(sets)]
    out = [torch.empty(rows, n, dtype=torch.bfloat16, device=device) for _ in range(sets)]
    stream = torch.cuda.current_stream()
    for i in range(max(warmup, sets)):
        ring_reduce(recv[i % sets], out[i % sets], local[i % sets], RANK)
    torch.cuda.synchronize()
    begin, end = _events(1)[0], _events(1)[0]
    begin.record(stream)
    for i in range(steps):
        ring_reduce(recv[i % sets], out[i % sets], local[i % sets], RANK)
    end.record(stream)
    torch.cuda.synchronize()
    ms = begin.elapsed_time(end) / steps
    nbytes = (world + 1) * rows * n * 2          # 8 reads + 1 write of a (1024, 8192) bf16 block
    return ms, nbytes


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
    stream = torch.cuda.current_stream()
    nbytes = rows * n * 2
    forms = {"copy": (None, False, 2 * nbytes), "add_exclusive": (ReduceOp.SUM, True, 3 * nbytes),
             "add_atomic": (ReduceOp.SUM, False, 3 * nbytes)}
    result = {}
    for name, (op, exclusive, traffic) in forms.items():
        for i in range(max(warmup, sets)):
            persistent_copy_last_contig(src[i % sets], dst[i % sets], num_sms=blocks, reduce_op=op, exclusive=exclusive)
        torch.cuda.synchronize()
        begin, end = _events(1)[0], _events(1)[0]
        begin.record(stream)
        for i in range(steps):
            persistent_copy_last_contig(src[i % sets], dst[i % sets], num_sms=blocks, reduce_op=op, exclusive=exclusive)
        end.record(stream)
        torch.cuda.synchronize()
        result[name] = (begin.elapsed_time(end) / steps, traffic)
    return result


def run_attention(device, steps, warmup):
    """All-gather attention at the headline ring / all-gather configuration: 4096 local q rows, 32 heads, against 32768
    kv rows as 8 chunks of 4096 in double-ring arrival order (every chunk resident), head dim 128; two q
    blocks per workgroup in opposite phases (pair_q_blocks)."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    B, H, Sq, Skv, D, chunks = 1, 32, 4096, 32768, 128, 8
    torch.manual_seed(2)
    q = torch.randn(B, H, Sq, D, device=device).bfloat16()
    k = torch.randn(B, H, Skv, D, device=device).bfloat16()
    v = torch.randn(B, H, Skv, D, device=device).bfloat16()
    chunk = Skv // chunks
    as_table = lambda rows: torch.tensor(rows, dtype=torch.int32, device=device)
    cums = [(i + 1) * B * H * Sq for i in range(chunks)]
    tables = dict(wave_offsets=as_table([[0, 0, 0, o * chunk] for o in (0, 1, 7, 6, 4, 5, 3, 2)]),
                  wave_sizes=as_table([[B, H, Sq, chunk]] * chunks), cum_wave_sizes=as_table(cums),
                  signal_offsets=as_table([-1, 0, 4, 1, 5, 2, 6, 3]), cum_tiles=cums[-1],
                  signal_ptr=torch.ones(chunks, dtype=torch.int64, device=device))
    out = torch.empty_like(q)
    for _ in range(warmup):
        attention_forward(q, k, v, D ** -0.5, out=out, pair_q_blocks=True, **tables)
    torch.cuda.synchronize()
    begin, end = _events(1)[0], _events(1)[0]
    begin.record()
    for _ in range(steps):
        attention_forward(q, k, v, D ** -0.5, out=out, pair_q_blocks=True, **tables)
    end.record()
    torch.cuda.synchronize()
    check_status()
    s = (q[0, 7].float() @ k[0, 7].float().t()) * D ** -0.5
    ref = torch.softmax(s, dim=-1) @ v[0, 7].float()
    err = ((out[0, 7].float() - ref).abs().max() / ref.abs().max()).item()
    return begin.elapsed_time(end) / steps, 4.0 * B * H * Sq * Skv * D, err


def run_producer(device, steps, warmup):
    """GEMM+RS producer of the headline GEMM+RS configuration: partial C (8192, 8192) = A (8192, 3584) B^T in
    wave order 1..7, 0 with per-wave counters and flags."""
    from syncopate_amd.computation.gemm import gemm_producer

    m, k, n, world = 8192, 3584, 8192, 8
    torch.manual_seed(3)
    a = (0.02 * torch.randn(m, k, device=device)).bfloat16()
    b = (0.02 * torch.randn(n, k, device=device)).bfloat16()
    c = torch.empty(m, n, dtype=torch.bfloat16, device=device)
    rows = m // world
    as_table = lambda rows_: torch.tensor(rows_, dtype=torch.int32, device=device)
    sizes = as_table([[rows, n]] * world)
    offsets = as_table([[((RANK + i + 1) % world) * rows, 0] for i in range(world)])
    signals = as_table(list(range(world)))
    flags = torch.zeros(world, dtype=torch.int64, device=device)
    counters = torch.zeros(world, dtype=torch.int32, device=device)

    def launch():
        counters.zero_()
        # 1024 tiles of 256 x 256: four full rounds of 256 programs
        gemm_producer(a, b, c, flags, sizes, offsets, signals, 256, 256, 256, BK, GROUP_M, cum_tiles=m * n,
                      counter_buffer=counters, xcd_remap=False, eight_waves=EIGHT_WAVES)

    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    begin, end = _events(1)[0], _events(1)[0]
    begin.record()
    for _ in range(steps):
        launch()
    end.record()
    torch.cuda.synchronize()
    assert flags.tolist() == [1] * world
    return begin.elapsed_time(end) / steps, 2.0 * m * n * k


def cpu_baseline(state):
    """torch CPU matmul over the gathered operands (fp32 values of the same bf16 inputs):
    a bounded sample of the same GEMM — a band of rows of A against all of B."""
    from oracle import numerics

    threads = min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    sample_rows = M
    a = state["a"][:sample_rows].cpu()
    b = state["b"].cpu()
    numerics.gemm_fp32(a[:128], b)          # warm-up
    reps, spent = 0, 0.0
    while spent < 10.0 and reps < 40:
        t0 = time.perf_counter()
        numerics.gemm_fp32(a, b)
        spent += time.perf_counter() - t0
        reps += 1
    flop = 2.0 * sample_rows * N * K * reps
    return {
        "value": flop / spent / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{reps} x torch CPU fp32 matmul of A[:{sample_rows}] (bf16 values) with all of B, "
                  f"{spent:.1f} s",
    }


def main():
    global BM, BN, NUM_SMS, LEAD_OPS, XCD_REMAP
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step is ~0.45 ms: the defaults time a few hundred of them (the whole run still takes well under a minute)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch every step's operations from the host "
                    "instead of replaying them as one HIP graph")
    ap.add_argument("--resident-only", action="store_true",
                    help="skip the flag-gated steps (for hardware-counter runs, which serialise kernels: "
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
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    if args.split_device and (args.copy_blocks == 0 or not args.no_graph):
        sys.exit("--split-device splits the compute units between two streams: it needs the copy kernel "
                 "(--copy-blocks N) and launches from the host (--no-graph; a graph's kernel nodes carry no mask)")
    state = build_ag_gemm(device, args.copy_blocks, args.split_device, args.fuse_flags)
    with torch.cuda.stream(state["ctx"].compute_stream):
        wall_ms, gated_ms, no_lead_ms, resident_ms = run_ag_gemm(state, args.steps, args.warmup, args.resident_only,
                                                     not args.no_graph)
    torch.cuda.synchronize()
    traffic_calibration(device)
    err, gathered = check_ag_gemm(state)
    reduce_ms, reduce_bytes = run_reduce(device, max(args.steps, 30), args.warmup)
    boxes = run_box_copies(device, max(args.steps, 20), args.warmup)
    attn_ms, attn_flop, attn_err = run_attention(device, 5, 2)
    prod_ms, prod_flop = run_producer(device, args.steps, args.warmup)

    flop = 2.0 * M * N * K
    value = flop / (wall_ms * 1e-3) / 1e12
    kernel_tflops = flop / (gated_ms * 1e-3) / 1e12
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
            "producer": "side stream: " + (
                f"one kernel of {args.copy_blocks} workgroups per chunk that copies, then sets the flag"
                if args.fuse_flags else
                ("hipMemcpyAsync" if args.copy_blocks == 0 else f"copy kernel of {args.copy_blocks} workgroups")
                + " + flag-set kernel per chunk"),
            "launch": "eager" if args.no_graph else "a hip graph of two steps, replayed steps/2 times",
            "split_device": state["ctx"].cu_split,
        },
        "pct_bf16_mfma_peak": 100.0 * value / MFMA_BF16_PEAK_TFLOPS,
        "flag_wait_overhead_pct": 100.0 * (gated_ms - resident_ms) / resident_ms,
        "step_over_resident_kernel_pct": 100.0 * (wall_ms - resident_ms) / resident_ms,
        "kernel_ms_gated": gated_ms,
        "kernel_ms_gated_launched_with_first_copy": no_lead_ms,
        "kernel_ms_resident": resident_ms,
        "resident_tflops": flop / (resident_ms * 1e-3) / 1e12,
        "rs_reduce_GBps": reduce_bytes / (reduce_ms * 1e-3) / 1e9,
        "rs_reduce_us": reduce_ms * 1e3,
        "rs_reduce_pct_hbm_peak": 100.0 * reduce_bytes / (reduce_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "box_copy_GBps": {name: traffic / (ms * 1e-3) / 1e9 for name, (ms, traffic) in boxes.items()},
        "box_copy_us": {name: ms * 1e3 for name, (ms, _) in boxes.items()},
        "rs_producer_tflops": prod_flop / (prod_ms * 1e-3) / 1e12,
        "rs_producer_pct_bf16_mfma_peak": 100.0 * prod_flop / (prod_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "attn_tflops": attn_flop / (attn_ms * 1e-3) / 1e12,
        "attn_pct_bf16_mfma_peak": 100.0 * attn_flop / (attn_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "attn_ms": attn_ms,
        "attn_max_rel_err_vs_fp32": attn_err,
        "host_compile_ms": state["compile_ms"],
        "max_rel_err_vs_fp32": err,
        "gathered_a_matches": gathered,
        "roofline": {
            "kernel": f"gemm_wave_kernel<bf16, {'EarlyPipe' if (BM, BN) in ((256, 256), (256, 224)) else 'SlabPipe<3 stages>'}, "
                      f"{BM}x{BN}, {8 if EIGHT_WAVES else 4} wavefronts, consumer>",
            "bound": "mfma",
            "achieved": kernel_tflops,
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": kernel_tflops / MFMA_BF16_PEAK_TFLOPS,
            "traffic": GEMM_TRAFFIC_BYTES_PER_LAUNCH,
        },
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(state)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
