// Chunk-scheduled persistent GEMM for gfx950 (MI355X): C = A * B^T, fp32 accumulate.
//
// A workgroup owns a BM x BN tile of C and walks tile ids pid, pid + NUM_SMS, ... in the
// wave order of the schedule (syncopate/computation/gemm/template.py:69-136).  A and B are
// both K-contiguous, so a k-slab of either is a set of short rows.  Slabs go from HBM
// straight into an LDS ring with global_load_lds_dwordx4 (16 bytes per lane, no register
// staging); a wavefront-wide load fills 1 KB of consecutive LDS rows, and which 16-byte
// chunk of its row a lane fetches is XOR-swizzled with the row number so that the 128-bit
// fragment reads of v_mfma_f32_32x32x16 are bank-conflict free over the 64 LDS banks.
//
// Two pipelines over the same tile walk:
//   ring   4 stages of 32-deep slabs; the fill of slab s+3 is issued while slab s is being
//          multiplied, so three slabs are in flight and HBM/L2 latency is covered; one
//          barrier per slab, with MFMA work on both sides of it.  Needs K % 128 == 0.
//   pair   2 stages of 64-deep slabs (one in flight); any K % 64 == 0.
//
// Consumer form: before the first tile of a wave whose signal offset is >= 0 lane 0 spins on
// the flag word, then the whole workgroup takes an acquire fence (template.py:121-128).
// Producer form: after the C tile is stored the workgroup bumps counters[wave] and the last
// tile of the wave publishes the flag (template.py:343-348).
#include "common.h"

namespace syn {

struct GemmParams {
    const void* a;
    const void* b;
    void* c;
    uint64_t* flags;
    const int32_t* wave_sizes;
    const int32_t* wave_offsets;
    const int32_t* signal_offsets;
    int32_t* counters;
    int32_t* visit_log;
    int32_t* status;
    int64_t timeout_ticks;
    int32_t num_waves;
    int32_t M, N, K;
    int32_t group_m;
    int32_t num_sms;
    int32_t num_tiles;
    int32_t xcd_remap;
    int32_t k_stagger;
};

template <typename T>
struct Mfma32;

template <>
struct Mfma32<__bf16> {
    typedef bf16x8_t frag_t;
    static __device__ __forceinline__ f32x16_t run(frag_t a, frag_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

template <>
struct Mfma32<_Float16> {
    typedef f16x8_t frag_t;
    static __device__ __forceinline__ f32x16_t run(frag_t a, frag_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

template <typename T>
__device__ __forceinline__ uint2 pack4(float x0, float x1, float x2, float x3) {
    typedef T vec4 __attribute__((ext_vector_type(4)));
    vec4 v;
    v[0] = (T)x0;   // round to nearest even
    v[1] = (T)x1;
    v[2] = (T)x2;
    v[3] = (T)x3;
    return __builtin_bit_cast(uint2, v);
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;

// sched_group_barrier instruction classes
constexpr int kSgMfma = 0x008, kSgVmemRead = 0x020, kSgDsRead = 0x100;

// s_waitcnt immediate (gfx9 encoding) that waits until at most `vm` vector-memory operations
// of this wavefront are outstanding and, if lgkm_zero, until all LDS operations have returned.
constexpr int waitcnt_imm(int vm, bool lgkm_zero) {
    return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | ((lgkm_zero ? 0 : 0xF) << 8);
}

// HBM -> LDS without registers.  A slab of ROWS rows of ROW_BYTES bytes is cut into 1 KB
// blocks of consecutive rows; wavefront `wave` of NW fills blocks wave, wave + NW, ...; lane l
// lands at byte 16*l of its block.  `slab` is the wavefront-uniform address of the slab's first
// row at this k, `lane_off` this lane's byte offset inside block 0 (its row, and the swizzled
// 16-byte chunk it fetches).  Uniform base + 32-bit lane offset is the scalar-base addressing
// form: all loads of a step share one offset register.
template <int ROWS, int ROW_BYTES, int NW>
__device__ __forceinline__ void dma_slab(unsigned char* lds_slab, const unsigned char* slab,
                                         unsigned lane_off, size_t row_bytes, int wave) {
    constexpr int kRowsPerBlock = 1024 / ROW_BYTES;
#pragma unroll
    for (int i = 0; i < ROWS / (kRowsPerBlock * NW); ++i) {
        const int blk = i * NW + wave;
        __builtin_amdgcn_global_load_lds(
            (global_void_ptr)(slab + (size_t)(blk * kRowsPerBlock) * row_bytes + lane_off),
            (lds_void_ptr)(lds_slab + blk * 1024), 16, 0, 0);
    }
}

// 128-bit fragment reads of one k16 step: TM row tiles of A, TN row tiles of B.
template <typename T, int TM, int TN, int ROW_BYTES>
__device__ __forceinline__ void load_frags(typename Mfma32<T>::frag_t (&fa)[TM],
                                           typename Mfma32<T>::frag_t (&fb)[TN],
                                           const unsigned char* sbase, int a_rd, int b_rd, int chunk) {
    typedef typename Mfma32<T>::frag_t frag_t;
#pragma unroll
    for (int i = 0; i < TM; ++i)
        fa[i] = *reinterpret_cast<const frag_t*>(sbase + a_rd + i * 32 * ROW_BYTES + chunk);
#pragma unroll
    for (int j = 0; j < TN; ++j)
        fb[j] = *reinterpret_cast<const frag_t*>(sbase + b_rd + j * 32 * ROW_BYTES + chunk);
}

// TM x TN MFMAs of one k16 step.  B is the first operand, so each accumulator holds the
// transposed 32x32 tile D'[n][m].
template <typename T, int TM, int TN>
__device__ __forceinline__ void mma_step(f32x16_t (&acc)[TM][TN],
                                         const typename Mfma32<T>::frag_t (&fa)[TM],
                                         const typename Mfma32<T>::frag_t (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma32<T>::run(fb[j], fa[i], acc[i][j]);
}

// Scheduling pattern of one k16 step: the FILLS HBM->LDS loads go out first, then MFMAs of
// the current step alternate with the 128-bit LDS reads of the next step's fragments, so the
// reads' latency is covered by matrix work (MFMAs lead: they only need fragments read a step
// ago).
template <int R, int READS, int MFMAS>
__device__ __forceinline__ void interleave_reads() {
    if constexpr (R < READS) {
        constexpr int per_read = MFMAS / READS;
        constexpr int mfmas = R == 0 ? MFMAS - per_read * (READS - 1) : per_read;
        __builtin_amdgcn_sched_group_barrier(kSgMfma, mfmas, 0);
        __builtin_amdgcn_sched_group_barrier(kSgDsRead, 1, 0);
        interleave_reads<R + 1, READS, MFMAS>();
    }
}

template <int READS, int MFMAS, int FILLS>
__device__ __forceinline__ void interleave_hint() {
    if constexpr (FILLS > 0) __builtin_amdgcn_sched_group_barrier(kSgVmemRead, FILLS, 0);
    interleave_reads<0, READS, MFMAS>();
}

// ------------------------------------------------------------------ pipelines
//
// Both take the accumulators, the uniform addresses of the tile's A and B row panels and
// run the whole K loop.  On return every fill has landed and every wavefront has passed a
// barrier, so the stages may be refilled at once.

// pair: two stages of 64-deep slabs.  LDS row r (128 bytes) keeps logical chunk c at physical
// chunk c ^ ((r >> 1) & 7): a row covers half of the 64 banks (even rows the low half), a
// 128-bit read is served 16 consecutive rows per cycle, and (r >> 1) & 7 gives the 8 rows that
// share a half 8 distinct chunks.
template <typename T, int BM, int BN, int WGM, int WGN>
struct PairPipe {
    static constexpr int NW = WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int BK = 64, ROW = BK * 2;
    static constexpr int A_BYTES = BM * ROW, STAGE = (BM + BN) * ROW;
    static constexpr int FILLS = (BM + BN) / (8 * NW);
    static constexpr int K_ALIGN = 64;
    typedef typename Mfma32<T>::frag_t frag_t;

    static __device__ __forceinline__ void slab(f32x16_t (&acc)[TM][TN], const unsigned char* st,
                                                int a_rd, int b_rd, int half, int swz) {
        frag_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];
        load_frags<T, TM, TN, ROW>(fa0, fb0, st, a_rd, b_rd, ((0 + half) ^ swz) << 4);
        __builtin_amdgcn_sched_group_barrier(kSgDsRead, TM + TN, 0);
#pragma unroll
        for (int kk = 0; kk < 4; kk += 2) {
            load_frags<T, TM, TN, ROW>(fa1, fb1, st, a_rd, b_rd, (((kk + 1) * 2 + half) ^ swz) << 4);
            mma_step<T, TM, TN>(acc, fa0, fb0);
            if (kk == 0) interleave_hint<TM + TN, TM * TN, FILLS>();
            else interleave_hint<TM + TN, TM * TN, 0>();
            __builtin_amdgcn_sched_barrier(0);
            if (kk + 2 < 4) load_frags<T, TM, TN, ROW>(fa0, fb0, st, a_rd, b_rd, (((kk + 2) * 2 + half) ^ swz) << 4);
            mma_step<T, TM, TN>(acc, fa1, fb1);
            if (kk + 2 < 4) interleave_hint<TM + TN, TM * TN, 0>();
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    static __device__ __forceinline__ void run(f32x16_t (&acc)[TM][TN], const unsigned char* a_slab,
                                               const unsigned char* b_slab, size_t row_bytes, int K,
                                               int k_rot, int lane, int wave) {
        __shared__ __attribute__((aligned(1024))) unsigned char stage0[STAGE];
        __shared__ __attribute__((aligned(1024))) unsigned char stage1[STAGE];
        const int wm = wave / WGN, wn = wave % WGN;
        const int ld_row = lane >> 3;
        // blocks this wavefront fills are wave, wave + NW, ... (NW even): block parity = wave parity
        const int ld_chunk = (lane & 7) ^ ((((wave & 1) << 3 | ld_row) >> 1) & 7);
        const unsigned lane_off = (unsigned)(ld_row * row_bytes) + ld_chunk * 16;
        const int half = lane >> 5, swz = (lane >> 1) & 7;
        const int a_rd = (wm * WM + (lane & 31)) * ROW;
        const int b_rd = A_BYTES + (wn * WN + (lane & 31)) * ROW;
        const int k_steps = K / BK;
        const int rot = k_rot % k_steps;
        // slab i of this tile's walk is slab (i + rot) mod k_steps of K
        auto at = [&](int i) -> size_t { const int k = i + rot; return (size_t)(k >= k_steps ? k - k_steps : k) * ROW; };

        dma_slab<BM, ROW, NW>(stage0, a_slab + at(0), lane_off, row_bytes, wave);
        dma_slab<BN, ROW, NW>(stage0 + A_BYTES, b_slab + at(0), lane_off, row_bytes, wave);
        __syncthreads();                 // waits for the fills (vmcnt) and for every wavefront

        // two slabs per trip: fill the idle stage with slab ks+1 while slab ks is multiplied
        // out of the other; the barrier ending a slab also drains the fill.  The fill after the
        // last slab re-fetches that slab (no branch in the loop body; nothing reads it).
        const int pairs = k_steps >> 1;
        for (int pr = 0; pr < pairs; ++pr) {
            const size_t k_odd = at(2 * pr + 1);
            const size_t k_even = at(min(2 * pr + 2, k_steps - 1));
            dma_slab<BM, ROW, NW>(stage1, a_slab + k_odd, lane_off, row_bytes, wave);
            dma_slab<BN, ROW, NW>(stage1 + A_BYTES, b_slab + k_odd, lane_off, row_bytes, wave);
            slab(acc, stage0, a_rd, b_rd, half, swz);
            __syncthreads();
            dma_slab<BM, ROW, NW>(stage0, a_slab + k_even, lane_off, row_bytes, wave);
            dma_slab<BN, ROW, NW>(stage0 + A_BYTES, b_slab + k_even, lane_off, row_bytes, wave);
            slab(acc, stage1, a_rd, b_rd, half, swz);
            __syncthreads();
        }
        if (k_steps & 1) {
            slab(acc, stage0, a_rd, b_rd, half, swz);
            __syncthreads();
        }
    }
};

// ring: four stages of 32-deep slabs.  LDS row r (64 bytes) keeps logical chunk c at physical
// chunk c ^ ((r >> 2) & 3): 16 consecutive rows then hit 16 distinct 16-byte bank groups.
//
// Step s (slab s lives in stage s % 4):
//     issue the fill of slab s+3 into stage (s+3) % 4      (its last reader passed a barrier)
//     read the fragments of k16 step 1 of slab s            | MFMAs of k16 step 0 of slab s
//     wait: own part of slab s+1 landed, own LDS reads returned;  barrier
//     read the fragments of k16 step 0 of slab s+1          | MFMAs of k16 step 1 of slab s
// Fills past the last slab re-fetch it, so the count of outstanding fills is the same in
// every step and the wait is a constant "all but the newest two slabs".
template <typename T, int BM, int BN, int WGM, int WGN>
struct RingPipe {
    static constexpr int NW = WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int BK = 32, ROW = BK * 2;
    static constexpr int A_BYTES = BM * ROW, STAGE = (BM + BN) * ROW;
    static constexpr int FILLS = (BM + BN) / (16 * NW);     // fills per wavefront and slab
    static constexpr int K_ALIGN = 128;
    typedef typename Mfma32<T>::frag_t frag_t;

    struct Lane {
        unsigned lane_off;
        int a_rd, b_rd, chunk0, chunk1;
    };

    static __device__ __forceinline__ void fill(unsigned char* st, const unsigned char* a_slab,
                                                const unsigned char* b_slab, int slab_idx, const Lane& ln,
                                                size_t row_bytes, int wave) {
        const size_t k_off = (size_t)slab_idx * ROW;
        dma_slab<BM, ROW, NW>(st, a_slab + k_off, ln.lane_off, row_bytes, wave);
        dma_slab<BN, ROW, NW>(st + A_BYTES, b_slab + k_off, ln.lane_off, row_bytes, wave);
    }

    // one step; f0 holds the fragments of (cur, k16 step 0) on entry and of (nxt, step 0) on exit
    static __device__ __forceinline__ void step(f32x16_t (&acc)[TM][TN], frag_t (&fa0)[TM], frag_t (&fb0)[TN],
                                                const unsigned char* cur, const unsigned char* nxt,
                                                unsigned char* refill, const unsigned char* a_slab,
                                                const unsigned char* b_slab, int slab_idx, const Lane& ln,
                                                size_t row_bytes, int wave) {
        frag_t fa1[TM], fb1[TN];
        fill(refill, a_slab, b_slab, slab_idx, ln, row_bytes, wave);
        load_frags<T, TM, TN, ROW>(fa1, fb1, cur, ln.a_rd, ln.b_rd, ln.chunk1);
        mma_step<T, TM, TN>(acc, fa0, fb0);
        interleave_hint<TM + TN, TM * TN, FILLS>();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * FILLS, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        load_frags<T, TM, TN, ROW>(fa0, fb0, nxt, ln.a_rd, ln.b_rd, ln.chunk0);
        mma_step<T, TM, TN>(acc, fa1, fb1);
        interleave_hint<TM + TN, TM * TN, 0>();
        __builtin_amdgcn_sched_barrier(0);
    }

    static __device__ __forceinline__ void run(f32x16_t (&acc)[TM][TN], const unsigned char* a_slab,
                                               const unsigned char* b_slab, size_t row_bytes, int K,
                                               int k_rot, int lane, int wave) {
        __shared__ __attribute__((aligned(1024))) unsigned char st0[STAGE];
        __shared__ __attribute__((aligned(1024))) unsigned char st1[STAGE];
        __shared__ __attribute__((aligned(1024))) unsigned char st2[STAGE];
        __shared__ __attribute__((aligned(1024))) unsigned char st3[STAGE];
        const int wm = wave / WGN, wn = wave % WGN;
        Lane ln;
        // 16 rows of 64 bytes per 1 KB block: lane l fills row l / 4, physical chunk l % 4
        ln.lane_off = (unsigned)((lane >> 2) * row_bytes) + (((lane & 3) ^ ((lane >> 4) & 3)) << 4);
        ln.a_rd = (wm * WM + (lane & 31)) * ROW;
        ln.b_rd = A_BYTES + (wn * WN + (lane & 31)) * ROW;
        const int half = lane >> 5, swz = (lane >> 2) & 3;
        ln.chunk0 = ((0 + half) ^ swz) << 4;
        ln.chunk1 = ((2 + half) ^ swz) << 4;
        const int k_steps = K / BK, last = k_steps - 1;
        const int rot = k_rot % k_steps;
        // slab i of this tile's walk is slab (i + rot) mod k_steps of K
        auto at = [&](int i) -> int { const int k = min(i, last) + rot; return k >= k_steps ? k - k_steps : k; };

        fill(st0, a_slab, b_slab, at(0), ln, row_bytes, wave);
        fill(st1, a_slab, b_slab, at(1), ln, row_bytes, wave);
        fill(st2, a_slab, b_slab, at(2), ln, row_bytes, wave);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * FILLS, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        frag_t fa0[TM], fb0[TN];
        load_frags<T, TM, TN, ROW>(fa0, fb0, st0, ln.a_rd, ln.b_rd, ln.chunk0);

        for (int s = 0; s <= last; s += 4) {
            step(acc, fa0, fb0, st0, st1, st3, a_slab, b_slab, at(s + 3), ln, row_bytes, wave);
            step(acc, fa0, fb0, st1, st2, st0, a_slab, b_slab, at(s + 4), ln, row_bytes, wave);
            step(acc, fa0, fb0, st2, st3, st1, a_slab, b_slab, at(s + 5), ln, row_bytes, wave);
            step(acc, fa0, fb0, st3, st0, st2, a_slab, b_slab, at(s + 6), ln, row_bytes, wave);
        }
        // drain the re-fetches of the last slab before anything refills the stages
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
};

// ------------------------------------------------------------------ kernel

template <typename T, typename Pipe, int BM, int BN, int WGM, int WGN, bool PRODUCER>
__global__ void __launch_bounds__(64 * WGM * WGN) gemm_wave_kernel(const GemmParams p) {
    constexpr int WM = BM / WGM, WN = BN / WGN;   // wavefront tile
    constexpr int TM = WM / 32, TN = WN / 32;     // 32x32 MFMA tiles per wavefront

    __shared__ int s_abort;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;

    const int pid = logical_program_id((int)blockIdx.x, (int)gridDim.x, p.xcd_remap != 0);
    const int num_sms = p.num_sms;
    const int num_tiles = p.num_tiles;
    const int tiles_here = num_tiles / num_sms + (pid < num_tiles % num_sms ? 1 : 0);

    const int K = p.K, N = p.N;
    const size_t row_bytes = (size_t)K * sizeof(T);

    // --- wave walk state (uniform across the workgroup) ---
    int cur_wave = 0;
    int past_tiles = 0;
    int cur_m = p.wave_sizes[0] / BM;
    int cur_n = p.wave_sizes[1] / BN;
    int off_m = p.wave_offsets[0] / BM;
    int off_n = p.wave_offsets[1] / BN;
    int cur_tiles = cur_m * cur_n;
    int cur_sig = p.signal_offsets[0];

    if (tid == 0) s_abort = 0;
    __syncthreads();

    auto wait_flag = [&](int sig) -> bool {
        if (tid == 0) {
            const bool ok = spin_until_equal(p.flags + sig, 1ull, p.timeout_ticks);
            if (!ok) {
                report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, cur_wave, pid, sig);
                s_abort = 1;
            }
        }
        __syncthreads();
        acquire_fence_agent();
        return s_abort == 0;
    };

    if (!PRODUCER) {
        if (cur_sig >= 0) {
            if (!wait_flag(cur_sig)) return;
        }
    }

    const T* __restrict__ A = reinterpret_cast<const T*>(p.a);
    const T* __restrict__ B = reinterpret_cast<const T*>(p.b);
    T* __restrict__ C = reinterpret_cast<T*>(p.c);

    for (int it = 0; it < tiles_here; ++it) {
        const int tile_id = pid + it * num_sms;

        bool new_wave = false;
        while (tile_id >= past_tiles + cur_tiles) {
            past_tiles += cur_tiles;
            ++cur_wave;
            if (cur_wave >= p.num_waves) return;      // table shorter than the grid: host check failed
            cur_m = p.wave_sizes[cur_wave * 2] / BM;
            cur_n = p.wave_sizes[cur_wave * 2 + 1] / BN;
            off_m = p.wave_offsets[cur_wave * 2] / BM;
            off_n = p.wave_offsets[cur_wave * 2 + 1] / BN;
            cur_tiles = cur_m * cur_n;
            cur_sig = p.signal_offsets[cur_wave];
            new_wave = true;
        }
        if (!PRODUCER) {
            if (new_wave && cur_sig >= 0) {
                if (!wait_flag(cur_sig)) return;
            }
        }

        // get_pid_mn (template.py:10-18) on the wave-local tile id
        const int local = tile_id - past_tiles;
        const int in_group = p.group_m * cur_n;
        const int group_id = local / in_group;
        const int first_m = group_id * p.group_m;
        const int gsz = min(cur_m - first_m, p.group_m);
        const int pid_m = first_m + (local % gsz) + off_m;
        const int pid_n = (local % in_group) / gsz + off_n;

        if (p.visit_log != nullptr && tid == 0) {
            int4 rec = make_int4(pid, cur_wave, pid_m, pid_n);
            reinterpret_cast<int4*>(p.visit_log)[tile_id] = rec;
        }

        const size_t m0 = (size_t)pid_m * BM;
        const size_t n0 = (size_t)pid_n * BN;

        f32x16_t acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

        // Tiles walk K cyclically, neighbouring tiles starting 128 elements apart.  With a
        // power-of-two row pitch, programs that all sweep K from 0 in lockstep keep hitting the
        // same few memory channels; four phases spread them while tiles that share a panel of A
        // or B still stay within 512 elements of each other (L2 reuse).
        const int k_rot = p.k_stagger ? ((pid_m + pid_n) & 3) * (128 / Pipe::BK) : 0;
        Pipe::run(acc, reinterpret_cast<const unsigned char*>(A + m0 * (size_t)K),
                  reinterpret_cast<const unsigned char*>(B + n0 * (size_t)K), row_bytes, K, k_rot, lane, wave);

        // Epilogue.  With B as the first MFMA operand a lane holds, for column m = lane % 32 of
        // D', rows n = 8g + 4*(lane/32) + 0..3: four consecutive elements of one row of C -> one
        // 8-byte store.
        {
            T* c_row = C + (m0 + wm * WM + (lane & 31)) * (size_t)N + n0 + wn * WN + 4 * (lane >> 5);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const uint2 v = pack4<T>(acc[i][j][4 * g], acc[i][j][4 * g + 1],
                                                 acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                        *reinterpret_cast<uint2*>(c_row + (size_t)(32 * i) * N + 32 * j + 8 * g) = v;
                    }
        }

        if (PRODUCER) {
            if (cur_sig >= 0) {
                __threadfence();             // every lane's C stores are visible device-wide
                __syncthreads();
                if (tid == 0) {
                    const int done = __hip_atomic_fetch_add(p.counters + cur_wave, 1, __ATOMIC_RELEASE,
                                                            __HIP_MEMORY_SCOPE_AGENT);
                    if (done == cur_tiles - 1)
                        __hip_atomic_store(p.flags + cur_sig, 1ull, __ATOMIC_RELEASE,
                                           __HIP_MEMORY_SCOPE_SYSTEM);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- host side

static int64_t gemm_num_tiles(int64_t cum_tiles, int M, int N, int bm, int bn) {
    if (cum_tiles > 0) return (cum_tiles + (int64_t)bm * bn - 1) / ((int64_t)bm * bn);
    return (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
}

template <typename T, template <typename, int, int, int, int> class PipeT, int BM, int BN, int WGM, int WGN,
          bool PRODUCER>
static int launch_gemm(const GemmParams& p, int grid, hipStream_t stream) {
    typedef PipeT<T, BM, BN, WGM, WGN> Pipe;
    hipLaunchKernelGGL((gemm_wave_kernel<T, Pipe, BM, BN, WGM, WGN, PRODUCER>), dim3(grid),
                       dim3(64 * WGM * WGN), 0, stream, p);
    return (int)hipGetLastError();
}

// Workgroup shapes: 4 wavefronts (2x2, one per SIMD) or 8 (two per SIMD: one can issue MFMAs
// while the other waits for LDS or a barrier).
template <typename T, template <typename, int, int, int, int> class PipeT, bool PRODUCER>
static int dispatch_tile(const GemmParams& p, int bm, int bn, bool eight, int grid, hipStream_t stream) {
    if (eight) {
        if (bm == 256 && bn == 256) return launch_gemm<T, PipeT, 256, 256, 2, 4, PRODUCER>(p, grid, stream);
        if (bm == 128 && bn == 256) return launch_gemm<T, PipeT, 128, 256, 2, 4, PRODUCER>(p, grid, stream);
        if (bm == 256 && bn == 128) return launch_gemm<T, PipeT, 256, 128, 4, 2, PRODUCER>(p, grid, stream);
        return SYN_EINVAL;
    }
    if (bm == 256 && bn == 256) return launch_gemm<T, PipeT, 256, 256, 2, 2, PRODUCER>(p, grid, stream);
    if (bm == 128 && bn == 256) return launch_gemm<T, PipeT, 128, 256, 2, 2, PRODUCER>(p, grid, stream);
    if (bm == 256 && bn == 128) return launch_gemm<T, PipeT, 256, 128, 2, 2, PRODUCER>(p, grid, stream);
    if (bm == 128 && bn == 128) return launch_gemm<T, PipeT, 128, 128, 2, 2, PRODUCER>(p, grid, stream);
    return SYN_EINVAL;
}

template <typename T, bool PRODUCER>
static int dispatch_pipe(const GemmParams& p, int bm, int bn, bool eight, bool ring, int grid,
                         hipStream_t stream) {
    if (ring) return dispatch_tile<T, RingPipe, PRODUCER>(p, bm, bn, eight, grid, stream);
    return dispatch_tile<T, PairPipe, PRODUCER>(p, bm, bn, eight, grid, stream);
}

static int gemm_entry(const syn_gemm_desc* d, hipStream_t stream, bool producer) {
    if (d == nullptr) return SYN_EINVAL;
    if (!d->a || !d->b || !d->c || !d->wave_sizes || !d->wave_offsets || !d->signal_offsets)
        return SYN_EINVAL;
    if (d->num_waves <= 0 || d->M <= 0 || d->N <= 0 || d->K <= 0) return SYN_EINVAL;
    if (d->block_k != 64) return SYN_EINVAL;
    if (d->group_m <= 0 || d->num_sms <= 0) return SYN_EINVAL;
    if (d->dtype != SYN_DTYPE_BF16 && d->dtype != SYN_DTYPE_FP16) return SYN_EINVAL;
    if (d->M % d->block_m || d->N % d->block_n || d->K % 64) return SYN_EINVAL;
    if (!aligned16(d->a) || !aligned16(d->b) || !aligned16(d->c)) return SYN_EALIGN;
    if (producer && d->counters == nullptr) return SYN_EINVAL;
    if (d->flags == nullptr) return SYN_EINVAL;
    if (d->visit_log && !aligned16(d->visit_log)) return SYN_EALIGN;
    // the lane offset inside a block is 32 bits: 16 rows of K elements must fit
    if ((int64_t)d->K * 2 * 16 > (int64_t)UINT32_MAX) return SYN_EINVAL;

    const int64_t tiles = gemm_num_tiles(d->cum_tiles, d->M, d->N, d->block_m, d->block_n);
    if (tiles <= 0 || tiles > INT32_MAX) return SYN_EINVAL;
    if (d->cum_tiles > 0 && d->cum_tiles % ((int64_t)d->block_m * d->block_n)) return SYN_EINVAL;
    const int grid = (int)(tiles < d->num_sms ? tiles : d->num_sms);

    GemmParams p;
    p.a = d->a;
    p.b = d->b;
    p.c = d->c;
    p.flags = d->flags;
    p.wave_sizes = d->wave_sizes;
    p.wave_offsets = d->wave_offsets;
    p.signal_offsets = d->signal_offsets;
    p.counters = d->counters;
    p.visit_log = d->visit_log;
    p.status = d->status;
    p.timeout_ticks = timeout_ticks(d->spin_timeout_us);
    p.num_waves = d->num_waves;
    p.M = d->M;
    p.N = d->N;
    p.K = d->K;
    p.group_m = d->group_m;
    p.num_sms = d->num_sms;
    p.num_tiles = (int)tiles;
    p.xcd_remap = (d->options & SYN_GEMM_XCD_REMAP) ? 1 : 0;
    p.k_stagger = (d->options & SYN_GEMM_NO_K_STAGGER) ? 0 : 1;
    const bool eight = (d->options & SYN_GEMM_EIGHT_WAVES) != 0;
    // the ring needs whole groups of four 32-deep slabs
    const bool ring = !(d->options & SYN_GEMM_PAIR_PIPE) && d->K % 128 == 0;

    if (d->dtype == SYN_DTYPE_BF16) {
        return producer ? dispatch_pipe<__bf16, true>(p, d->block_m, d->block_n, eight, ring, grid, stream)
                        : dispatch_pipe<__bf16, false>(p, d->block_m, d->block_n, eight, ring, grid, stream);
    }
    return producer ? dispatch_pipe<_Float16, true>(p, d->block_m, d->block_n, eight, ring, grid, stream)
                    : dispatch_pipe<_Float16, false>(p, d->block_m, d->block_n, eight, ring, grid, stream);
}

}  // namespace syn

extern "C" {

int syn_gemm_consumer(const syn_gemm_desc* desc, syn_stream_t stream) {
    return syn::gemm_entry(desc, reinterpret_cast<hipStream_t>(stream), false);
}

int syn_gemm_producer(const syn_gemm_desc* desc, syn_stream_t stream) {
    return syn::gemm_entry(desc, reinterpret_cast<hipStream_t>(stream), true);
}

int syn_gemm_grid(int64_t cum_tiles, int32_t M, int32_t N, int32_t block_m, int32_t block_n,
                  int32_t num_sms) {
    if (block_m <= 0 || block_n <= 0 || num_sms <= 0) return SYN_EINVAL;
    const int64_t tiles = syn::gemm_num_tiles(cum_tiles, M, N, block_m, block_n);
    if (tiles <= 0 || tiles > INT32_MAX) return SYN_EINVAL;
    return (int)(tiles < num_sms ? tiles : num_sms);
}

int syn_gemm_check_waves(const int32_t* wave_sizes, const int32_t* wave_offsets,
                         const int32_t* signal_offsets, int32_t num_waves, int32_t M, int32_t N,
                         int32_t K, int32_t block_m, int32_t block_n, int32_t block_k,
                         int64_t cum_tiles, int64_t num_flags) {
    if (!wave_sizes || !wave_offsets || !signal_offsets) return SYN_EINVAL;
    if (num_waves <= 0 || M <= 0 || N <= 0 || K <= 0) return SYN_EINVAL;
    if (block_m <= 0 || block_n <= 0 || block_k <= 0) return SYN_EINVAL;
    if (M % block_m || N % block_n || K % block_k) return SYN_EINVAL;
    int64_t total = 0;
    for (int w = 0; w < num_waves; ++w) {
        const int64_t rows = wave_sizes[2 * w], cols = wave_sizes[2 * w + 1];
        const int64_t r0 = wave_offsets[2 * w], c0 = wave_offsets[2 * w + 1];
        if (rows <= 0 || cols <= 0 || r0 < 0 || c0 < 0) return SYN_EINVAL;
        if (rows % block_m || cols % block_n || r0 % block_m || c0 % block_n) return SYN_EINVAL;
        if (r0 + rows > M || c0 + cols > N) return SYN_ERANGE;
        const int64_t sig = signal_offsets[w];
        if (sig < -1) return SYN_EINVAL;
        if (sig >= 0 && num_flags >= 0 && sig >= num_flags) return SYN_ERANGE;
        total += rows * cols;
    }
    const int64_t expect = cum_tiles > 0 ? cum_tiles : (int64_t)M * N;
    if (total != expect) return SYN_EINVAL;
    return 0;
}

}  // extern "C"
