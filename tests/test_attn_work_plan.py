"""Work plans of the paired attention kernel: host logic on the CPU, the kernel forms they drive on the GPU.

The table a plan is made for is the reference's: the all-to-all attention glue
(tests/test_all2all_attn_transform.py:58-117) expands W arrivals into W*W waves; the tile -> work mapping is
`oracle.visit_order.attn_tile_work` (syncopate/computation/attn/template.py:39-44, 80-121).  A plan only
chooses which program makes a visit and which visits of one program are a segment.
"""

import ctypes

import pytest
import torch

from oracle import numerics, visit_order
from syncopate_amd.computation.attn.work_plan import (WORK_CONTINUES, WORK_PAIR_MASK, WORK_SOLE_WRITER,
                                                      plan_attention_work, table_visits)

REL_TOL = 1e-2


def all2all_tables(world, heads, chunk, batch=1):
    """The W -> W*W wave expansion of the reference's all-to-all attention test, arrival order 0..W-1,
    flag w per arrival (element units)."""
    offsets, sizes, signals, cums, total = [], [], [], [], 0

    def emit(qc, kc, gate):
        nonlocal total
        offsets.append([0, 0, qc * chunk, kc * chunk])
        sizes.append([batch, heads, chunk, chunk])
        signals.append(gate)
        total += batch * heads * chunk
        cums.append(total)

    for w in range(world):
        emit(w, w, w)
        for p in range(w):
            emit(p, w, w)
            emit(w, p, w)
    return offsets, sizes, cums, signals, total


def allgather_tables(heads, sq, chunk, order, batch=1):
    offsets = [[0, 0, 0, c * chunk] for c in order]
    sizes = [[batch, heads, sq, chunk]] * len(order)
    cums = [(i + 1) * batch * heads * sq for i in range(len(order))]
    return offsets, sizes, cums, [-1] + list(range(len(order) - 1)), cums[-1]


def _host_check(hip, offsets, sizes, cums, causal, plan, require_masked=False):
    to = lambda rows: torch.tensor(rows, dtype=torch.int32).contiguous()
    o, s, c, w = to(offsets), to(sizes), to(cums), to(plan.words)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    return hip.syn_attn_check_work_list(p(o), p(s), p(c), len(cums), 128, 128, 1 if causal else 0, p(w), w.numel(),
                                        plan.num_programs, 1 if require_masked else 0)


# ------------------------------------------------------------------------------------------ host logic (CPU)

@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("max_visits", [None, 1, 2, 3])
@pytest.mark.parametrize("programs", [7, 64, 256])
def test_plan_lists_every_visit_once_and_passes_the_library_check(hip, causal, max_visits, programs):
    offsets, sizes, cums, signals, total = all2all_tables(4, 2, 1024)
    plan = plan_attention_work(offsets, sizes, cums, causal=causal, num_programs=programs, max_visits=max_visits,
                               list_masked_visits=True)
    visits = table_visits(offsets, sizes, cums, causal=causal)
    listed = sorted(word & WORK_PAIR_MASK for entries in plan.program_entries for word in entries)
    assert listed == [v.pair for v in visits] == list(range(total // 256))
    assert plan.words[:programs + 1] == [sum(len(e) for e in plan.program_entries[:p]) for p in range(programs + 1)]
    assert _host_check(hip, offsets, sizes, cums, causal, plan, require_masked=True) == 0
    # segments: consecutive entries on the same q blocks, no longer than asked, never across a masked visit
    by_pair = {v.pair: v for v in visits}
    segments_of = {}
    for entries in plan.program_entries:
        run = []
        for word in entries:
            run.append(by_pair[word & WORK_PAIR_MASK])
            if not word & WORK_CONTINUES:
                assert len({v.key for v in run}) == 1
                assert max_visits is None or len(run) <= max_visits
                assert all(v.kv_blocks > 0 for v in run) or len(run) == 1
                if run[0].kv_blocks:
                    segments_of.setdefault(run[0].key, []).append(run)
                run = []
        assert not run
    # "only writer" exactly where a pair of q blocks has one segment
    for entries in plan.program_entries:
        first = True
        for word in entries:
            v = by_pair[word & WORK_PAIR_MASK]
            if first and v.kv_blocks:
                assert bool(word & WORK_SOLE_WRITER) == (len(segments_of[v.key]) == 1)
            first = not word & WORK_CONTINUES
    # a program's segments follow the order of the waves
    for entries in plan.program_entries:
        starts = []
        first = True
        for word in entries:
            if first:
                starts.append(by_pair[word & WORK_PAIR_MASK].wave)
            first = not word & WORK_CONTINUES
        assert starts == sorted(starts)


def test_causal_costs_and_balance_of_the_16384_table():
    """The headline all-to-all configuration: 8 arrivals of 2048 rows, 4 heads -> 64 waves.  A visit of q chunk c
    against kv chunk p costs 16 kv blocks below the diagonal (p < c), 2 j + 2 on it (pair j of the chunk) and
    nothing above it: 16 640 kv blocks over 256 pairs of q blocks, 65 per program if perfectly dealt."""
    offsets, sizes, cums, signals, total = all2all_tables(8, 4, 2048)
    visits = table_visits(offsets, sizes, cums, causal=True)
    assert len(visits) == 64 * 32 and sum(v.kv_blocks for v in visits) == 16640
    assert sum(1 for v in visits if v.kv_blocks == 0) == 28 * 32
    diag = sorted(v.kv_blocks for v in visits if v.wave == 0)
    assert diag == sorted([2 * j + 2 for j in range(8)] * 4)
    for max_visits, slack in ((1, 1.15), (2, 1.15), (4, 1.3)):
        plan = plan_attention_work(offsets, sizes, cums, causal=True, num_programs=256, max_visits=max_visits)
        assert sum(plan.program_cost) == 16640
        assert max(plan.program_cost) <= slack * 65          # longer segments are coarser to deal
    # without a mask every pair of q blocks is one segment of eight visits and nothing is merged
    plan = plan_attention_work(offsets, sizes, cums, causal=False, num_programs=256)
    assert plan.segments == 256 and plan.merged_segments == 0 and set(plan.program_cost) == {128}


def test_library_check_rejects_broken_lists(hip):
    offsets, sizes, cums, signals, total = all2all_tables(3, 1, 512)
    good = plan_attention_work(offsets, sizes, cums, causal=True, num_programs=4, max_visits=2)
    assert _host_check(hip, offsets, sizes, cums, True, good) == 0
    assert _host_check(hip, offsets, sizes, cums, True, good, require_masked=True) != 0     # masked visits left out

    def broken(edit):
        words = list(good.words)
        edit(words)
        return good._replace(words=words)

    entries_at = good.num_programs + 1
    # a visit twice
    assert _host_check(hip, offsets, sizes, cums, True, broken(lambda w: w.__setitem__(entries_at + 1, w[entries_at]))) != 0
    # a pair index beyond the table
    assert _host_check(hip, offsets, sizes, cums, True, broken(lambda w: w.__setitem__(entries_at, 4000))) != 0
    # offsets that do not cover the entries
    assert _host_check(hip, offsets, sizes, cums, True, broken(lambda w: w.__setitem__(good.num_programs, w[good.num_programs] - 1))) != 0
    # "continues" on a program's last entry
    last = entries_at + good.words[1] - 1
    assert _host_check(hip, offsets, sizes, cums, True, broken(lambda w: w.__setitem__(last, w[last] | WORK_CONTINUES))) != 0
    # "only writer" on q blocks that two segments write
    one = plan_attention_work(offsets, sizes, cums, causal=True, num_programs=4, max_visits=1)
    idx = next(i for i, word in enumerate(one.words[5:], 5) if not word & WORK_SOLE_WRITER)
    assert _host_check(hip, offsets, sizes, cums, True, one) == 0
    bad = list(one.words)
    bad[idx] |= WORK_SOLE_WRITER
    assert _host_check(hip, offsets, sizes, cums, True, one._replace(words=bad)) != 0
    # tables the paired kernel does not take: an odd number of q blocks, a kv range from an odd block
    with pytest.raises(ValueError):
        plan_attention_work([[0, 0, 0, 0]], [[1, 1, 384, 256]], [384], causal=False, num_programs=2)
    with pytest.raises(ValueError):
        plan_attention_work([[0, 0, 0, 128]], [[1, 1, 256, 256]], [256], causal=True, num_programs=2)


# ------------------------------------------------------------------------------------------ the kernel (GPU)

def _qkv(Z, H, S, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return tuple(torch.randn(Z, H, S, 128, generator=g).to(dtype) for _ in range(3))


def _rel(out, ref):
    return ((out.float().cpu() - ref).abs().max() / ref.abs().max()).item()


def _assert_visit_log(log, offsets, sizes, cums, signals):
    for t, got in enumerate(log.cpu().tolist()):
        w = visit_order.attn_tile_work(t, offsets, sizes, cums, signals)
        assert got[:7] == [w["wave"], w["z"], w["h"], w["q_block"], w["kv_lo"], w["kv_hi"], w["signal"]], (t, got)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("max_visits,programs", [(None, 24), (1, 5), (2, 16), (3, 40)])
def test_planned_all2all_attention_matches_sdpa_and_visits_the_tables_tiles(hip, dtype, causal, max_visits, programs):
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    world, H, chunk = 3, 2, 512
    S = world * chunk
    offsets, sizes, cums, signals, total = all2all_tables(world, H, chunk)
    q, k, v = _qkv(1, H, S, dtype, seed=11)
    plan = plan_attention_work(offsets, sizes, cums, causal=causal, num_programs=programs, max_visits=max_visits,
                               list_masked_visits=True)
    flags = torch.ones(world, dtype=torch.int64, device="cuda")
    log = torch.full((total // 128, 8), -1, dtype=torch.int32, device="cuda")
    for remap in (False, True):
        log.fill_(-1)
        o, lse = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, wave_offsets=offsets, wave_sizes=sizes,
                                   cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals, cum_tiles=total,
                                   causal=causal, pair_q_blocks=True, xcd_remap=remap, work_plan=plan,
                                   return_lse=True, visit_log=log)
        check_status()
        ref = numerics.sdpa_fp32(q, k, v, 128 ** -0.5, causal=causal)
        assert _rel(o, ref) <= REL_TOL
        s = (q.float() @ k.float().transpose(-1, -2)) * 128 ** -0.5
        if causal:
            s = s.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), float("-inf"))
        assert (lse.cpu() - torch.logsumexp(s, dim=-1) / 0.6931471805599453).abs().max().item() <= 2e-2
        _assert_visit_log(log, offsets, sizes, cums, signals)
        # the program a tile ran on is the one its plan names
        ran_on = log.cpu()[:, 7].tolist()
        for p, entries in enumerate(plan.program_entries):
            for word in entries:
                pair = word & WORK_PAIR_MASK
                hw = ran_on[2 * pair]
                assert ran_on[2 * pair + 1] == hw
                if not remap:
                    assert hw == p


@pytest.mark.gpu
@pytest.mark.parametrize("programs", [0, 6])
def test_paired_kernel_takes_a_causal_mask_without_a_plan(hip, programs):
    """Two q blocks per workgroup under the mask: the lower q block sits the pair's last kv block out."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    Z, H, S = 2, 2, 1024
    q, k, v = _qkv(Z, H, S, torch.bfloat16, seed=5)
    # kv in three ragged chunks (even blocks), arrival order shuffled
    chunks = [(512, 1024), (0, 256), (256, 512)]
    offsets = [[0, 0, 0, lo] for lo, _ in chunks]
    sizes = [[Z, H, S, hi - lo] for lo, hi in chunks]
    cums = [(i + 1) * Z * H * S for i in range(3)]
    signals = [-1, 0, 1]
    flags = torch.ones(2, dtype=torch.int64, device="cuda")
    log = torch.full((cums[-1] // 128, 8), -1, dtype=torch.int32, device="cuda")
    for scale in (128 ** -0.5, 1.0):
        o = attention_forward(q.cuda(), k.cuda(), v.cuda(), scale, wave_offsets=offsets, wave_sizes=sizes,
                              cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals, cum_tiles=cums[-1],
                              causal=True, pair_q_blocks=True, num_programs=programs, visit_log=log)
        check_status()
        assert _rel(o, numerics.sdpa_fp32(q, k, v, scale, causal=True)) <= REL_TOL
    _assert_visit_log(log, offsets, sizes, cums, signals)


@pytest.mark.gpu
def test_plan_of_an_allgather_table_is_the_chained_form(hip):
    """Every wave lists the same q ranges: one segment per pair of q blocks, nothing merged - what
    chain_q_blocks does from the table alone; the two give the same bits."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    H, Sq, chunk, order = 3, 512, 256, [2, 0, 3, 1]
    offsets, sizes, cums, signals, total = allgather_tables(H, Sq, chunk, order)
    g = torch.Generator(device="cpu").manual_seed(3)
    q = torch.randn(1, H, Sq, 128, generator=g).bfloat16()
    k = torch.randn(1, H, 4 * chunk, 128, generator=g).bfloat16()
    v = torch.randn(1, H, 4 * chunk, 128, generator=g).bfloat16()
    pairs = H * Sq // 256
    plan = plan_attention_work(offsets, sizes, cums, causal=False, num_programs=pairs)
    assert plan.segments == pairs and plan.merged_segments == 0
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=total, pair_q_blocks=True)
    planned = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, work_plan=plan, **kw)
    chained = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, chain_q_blocks=True, **kw)
    check_status()
    assert torch.equal(planned, chained)
    assert _rel(planned, numerics.sdpa_fp32(q, k, v, 128 ** -0.5)) <= REL_TOL


@pytest.mark.gpu
def test_many_segments_contend_for_one_pair_of_q_blocks(hip):
    """Sixteen kv waves over ONE pair of q blocks per head, one visit per segment, far more programs than the
    device has compute units: every visit but the first of a head merges under the same two locks."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    H, Sq, chunk, waves = 2, 256, 256, 16
    offsets, sizes, cums, signals, total = allgather_tables(H, Sq, chunk, list(range(waves)))
    g = torch.Generator(device="cpu").manual_seed(9)
    q = torch.randn(1, H, Sq, 128, generator=g).half()
    k = torch.randn(1, H, waves * chunk, 128, generator=g).half()
    v = torch.randn(1, H, waves * chunk, 128, generator=g).half()
    flags = torch.ones(waves - 1, dtype=torch.int64, device="cuda")
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=total, pair_q_blocks=True)
    ref = numerics.sdpa_fp32(q, k, v, 128 ** -0.5)
    for programs in (32, 1024):
        plan = plan_attention_work(offsets, sizes, cums, causal=False, num_programs=programs, max_visits=1)
        assert plan.merged_segments == plan.segments == H * waves
        o = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, work_plan=plan, **kw)
        check_status()
        assert _rel(o, ref) <= REL_TOL
    # the single-tile kernel under the same contention
    o = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, num_programs=0,
                          **{key: val for key, val in kw.items() if key != "pair_q_blocks"})
    check_status()
    assert _rel(o, ref) <= REL_TOL


@pytest.mark.gpu
def test_kernel_reports_a_list_that_breaks_a_segment(hip):
    """A list that the host check would have rejected: an entry that claims to continue on other q blocks ends the
    launch with a status, not with wrong results or a fault."""
    from syncopate_amd import _lib
    from syncopate_amd.computation import _launch
    from syncopate_amd.computation.attn import attention_forward

    offsets, sizes, cums, signals, total = all2all_tables(2, 1, 512)
    plan = plan_attention_work(offsets, sizes, cums, causal=False, num_programs=2)
    # swap the continuation of program 0's first segment for a visit to the other pair of q blocks
    words = list(plan.words)
    start0, start1 = 3 + words[0], 3 + words[1]
    words[start0 + 1], words[start1 + 1] = (words[start1 + 1], words[start0 + 1])
    bad = plan._replace(words=words)
    q, k, v = _qkv(1, 1, 1024, torch.bfloat16, seed=1)
    flags = torch.ones(2, dtype=torch.int64, device="cuda")
    with pytest.raises(_lib.SyncopateHipError):
        attention_forward(q.cuda(), k.cuda(), v.cuda(), 1.0, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                          signal_ptr=flags, signal_offsets=signals, cum_tiles=total, pair_q_blocks=True, work_plan=bad)
    # past the host check (as a C caller who skips it would be): the kernel notices
    import syncopate_amd.computation.attn.template as template
    real = hip.syn_attn_check_work_list
    try:
        template._lib.load().syn_attn_check_work_list = lambda *a: 0
        attention_forward(q.cuda(), k.cuda(), v.cuda(), 1.0, wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums,
                          signal_ptr=flags, signal_offsets=signals, cum_tiles=total, pair_q_blocks=True, work_plan=bad)
    finally:
        template._lib.load().syn_attn_check_work_list = real
    with pytest.raises(RuntimeError, match="kernel status"):
        _launch.check_status()


@pytest.mark.gpu
@pytest.mark.parametrize("form", ["auto", "planned", "pairs", "tiles"])
def test_causal_attention_of_a_q_shard_that_does_not_start_at_zero(hip, form):
    """A rank's q rows [512, 1024) against kv gathered in four chunks (arrival order 1, 0, 3, 2) under a causal
    mask: q positions are the table's q offsets (syncopate/computation/attn/template.py:80-121 takes `offs_m` from
    the wave's q start, for the addresses and for the mask alike).  The chunk wholly above the shard's first q
    blocks is a visit that costs nothing; rows outside the shard are not written.  Every launch form gives the
    masked softmax of torch."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    H, S, lo, chunk, order = 2, 1024, 512, 256, [1, 0, 3, 2]
    q, k, v = _qkv(1, H, S, torch.bfloat16, seed=21)
    offsets = [[0, 0, lo, c * chunk] for c in order]
    sizes = [[1, H, S - lo, chunk]] * len(order)
    cums = [(i + 1) * H * (S - lo) for i in range(len(order))]
    signals = [-1, 0, 1, 2]
    flags = torch.ones(3, dtype=torch.int64, device="cuda")
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=cums[-1], causal=True)
    if form == "planned":
        plan = plan_attention_work(offsets, sizes, cums, causal=True, num_programs=3, max_visits=2)
        assert any(vis.kv_blocks == 0 for vis in table_visits(offsets, sizes, cums, causal=True))
        kw.update(pair_q_blocks=True, work_plan=plan)
    elif form == "pairs":
        kw.update(pair_q_blocks=True, num_programs=5)
    elif form == "auto":
        kw.update(form="auto")
    out = torch.full((1, H, S, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    o = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, out=out, **kw)
    check_status()
    ref = numerics.sdpa_fp32(q, k, v, 128 ** -0.5, causal=True)
    assert _rel(o[:, :, lo:], ref[:, :, lo:]) <= REL_TOL
    assert (o[:, :, :lo] == 7.0).all()


@pytest.mark.gpu
def test_tables_and_lists_longer_than_the_kernels_lds_copies(hip):
    """The paired kernel keeps the first 256 waves of the tables and the first 512 entries of a program's list in
    LDS and reads the rest from memory: 600 waves of one kv block over one pair of q blocks, as one program's list of
    600 single-visit segments, as one chained walk, and as tiles dealt to three programs."""
    from syncopate_amd.computation._launch import check_status
    from syncopate_amd.computation.attn import attention_forward

    H, Sq, chunk, waves = 1, 256, 128, 600
    order = [(7 * i) % waves for i in range(waves)]            # 7 and 600 are coprime: every chunk once
    offsets, sizes, cums, signals, total = allgather_tables(H, Sq, chunk, order)
    g = torch.Generator(device="cpu").manual_seed(31)
    q = torch.randn(1, H, Sq, 128, generator=g).bfloat16()
    k = torch.randn(1, H, waves * chunk, 128, generator=g).bfloat16()
    v = torch.randn(1, H, waves * chunk, 128, generator=g).bfloat16()
    flags = torch.ones(waves - 1, dtype=torch.int64, device="cuda")
    kw = dict(wave_offsets=offsets, wave_sizes=sizes, cum_wave_sizes=cums, signal_ptr=flags, signal_offsets=signals,
              cum_tiles=total, pair_q_blocks=True)
    ref = numerics.sdpa_fp32(q, k, v, 128 ** -0.5)
    # Every merge rounds the stored partial output to bf16, as in the reference (attn/template.py:307-361): 600
    # merges are a random walk of 600 steps of half a unit in the last place (2^-9 each), some 5 % - a property of
    # the merged form, not of how long its tables are.  The forms that keep their sums in registers stay within REL_TOL.
    merged_tol = 1e-1
    log = torch.full((total // 128, 8), -1, dtype=torch.int32, device="cuda")
    for max_visits, tol in ((None, REL_TOL), (1, merged_tol)):
        plan = plan_attention_work(offsets, sizes, cums, causal=False, num_programs=1, max_visits=max_visits)
        assert len(plan.program_entries[0]) == waves and plan.segments == (1 if max_visits is None else waves)
        log.fill_(-1)
        o = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, work_plan=plan, visit_log=log, **kw)
        check_status()
        assert _rel(o, ref) <= tol, max_visits
        _assert_visit_log(log, offsets, sizes, cums, signals)
    o = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, chain_q_blocks=True, **kw)
    check_status()
    assert _rel(o, ref) <= REL_TOL
    log.fill_(-1)
    o = attention_forward(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, num_programs=3, visit_log=log, **kw)
    check_status()
    assert _rel(o, ref) <= merged_tol
    _assert_visit_log(log, offsets, sizes, cums, signals)
