// Chunk-scheduled persistent GEMM for gfx950 (MI355X): C = A * B^T, fp32 accumulate.
//
// A workgroup owns a BM x BN tile of C and walks tile ids pid, pid + NUM_SMS, ... in the
// wave order of the schedule (syncopate/computation/gemm/template.py:69-136).  A and B are
// both K-contiguous, so a k-slab of either is a set of short rows.  Slabs go from HBM
// straight into LDS stages with global_load_lds_dwordx4 (16 bytes per lane, no register
// staging); a wavefront-wide load fills 1 KB of consecutive LDS rows, and which 16-byte
// chunk of its row a lane fetches is XOR-swizzled with the row number so that the 128-bit
// fragment reads of the MFMAs (16 rows x four chunks for v_mfma_f32_16x16x32, 32 rows x two for
// v_mfma_f32_32x32x16) are bank-conflict free over the 64 LDS banks.
//
// Pipelines over the same tile walk (the 64 fills of a 256x256 slab take the texture path of a
// compute unit about 1400 cycles, a k16 step of MFMAs 512: where the fills are issued matters):
//   early  2 stages of 64-deep slabs, the LDS reads of a slab bunched at its start so that its
//          stage is refilled during three quarters of the slab's MFMAs; the default for the tiles of
//          which only two stages fit the 160 KB of LDS (256x256, 256x224), on 16x16x32 MFMAs
//          (which cost less energy per product on a power-limited board; same bits) or, as an
//          option, on 32x32x16 ones.
//   slab   3 stages of 64-deep slabs, a slab's fills spread over the four k16 steps; the default
//          for the other tiles.  With 2 stages (an option) all fills go out in one step.
//          Rows are whole 128-byte cache lines; any K % 64 == 0.
//   ring   4 stages of 32-deep slabs, three in flight; rows are half cache lines, which costs
//          L1 fill bandwidth.  Needs K % 128 == 0.
// A tile's first fills are issued before the previous tile's C is stored; C leaves through a
// per-wavefront LDS strip as whole cache lines.
//
// Consumer form: before the first tile of a wave whose signal offset is >= 0 lane 0 spins on
// the flag word, then the whole workgroup takes an acquire fence (template.py:121-128).
// Producer form: after the C tile is stored the workgroup bumps counters[wave] and the last
// tile of the wave publishes the flag (template.py:343-348).
#include <mutex>

#include "common.h"

namespace syn {

struct GemmParams {
    const void* a;
    const void* b;
    void* c;
    uint64_t* flags;
    const uint64_t* wait_flags;          // producer that is a consumer as well: flags to wait for ...
    const int32_t* wait_offsets;         // ... and the index per wave (-1: none)
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
    int32_t acquire_always;      // SYN_GEMM_ACQUIRE_ALWAYS: fence behind every flag wait, not only behind a spin
    // remote bindings (kernel mode 2): per-wave peer tables for A and / or C
    const void* const* a_peers;
    const int32_t* a_target;
    void* const* c_peers;
    const int32_t* c_target;
    const int32_t* c_dst_offsets;
    int32_t c_ld;
    int32_t c_atomic;
    // per-wave K range {first k, count}: a wave contracts over part of K only (split-K waves,
    // whose partial products are added into C); null: every wave takes all of K
    const int32_t* wave_k;
};

// kernel modes
constexpr int kConsumer = 0, kProducer = 1, kRemote = 2, kRemoteAtomic = 3;   // kRemoteAtomic: kRemote whose C tiles are added

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

typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <typename T>
struct Mfma16;

template <>
struct Mfma16<__bf16> {
    // inline assembly: the accumulator is named as an AGPR tuple that is read and written in place (through the
    // builtin the register allocator moves accumulators between the two register files inside the K loop).
    // The compiler does not know that the statement is an MFMA and adds no wait states behind it, so the
    // hazards are covered by hand:
    //  - MFMA result -> MFMA accumulator input: the pipelines touch an accumulator once per quarter, at least
    //    eight MFMAs (128 cycles) apart, and always as the same whole tuple;
    //  - MFMA result -> vector ALU read or overwrite: a matrix op of N passes needs N + 3 wait states before a
    //    vector instruction may read or write its result registers (7 for the four passes of 16x16x32, 11 for
    //    eight, 19 for sixteen).  Every K loop ends in mfma_result_wait_states() below, which idles 24 - more
    //    than the longest form needs - before the epilogue reads the accumulators and before the next tile's
    //    zeros are written.
    static __device__ __forceinline__ void run(bf16x8_t a, bf16x8_t b, f32x4_t& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};

template <>
struct Mfma16<_Float16> {
    static __device__ __forceinline__ void run(f16x8_t a, f16x8_t b, f32x4_t& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};

// Wait states between the last assembly MFMA of a K loop and the first vector instruction that touches an
// accumulator (see Mfma16): 16 + 8 idle issue slots, once per tile.
__device__ __forceinline__ void mfma_result_wait_states() {
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
}

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

// The same with the fills spread out too: G groups of (MFMAs, fill, LDS read), every kind
// divided as evenly as integers allow.  A wavefront issues in order, so a burst of fills that
// outruns the vector-memory queue would hold its MFMAs back; one fill every few MFMAs never does.
template <int G, int GROUPS, int READS, int MFMAS, int FILLS>
__device__ __forceinline__ void spread_groups() {
    if constexpr (G < GROUPS) {
        constexpr int m = MFMAS * (G + 1) / GROUPS - MFMAS * G / GROUPS;
        constexpr int r = READS * (G + 1) / GROUPS - READS * G / GROUPS;
        constexpr int f = FILLS * (G + 1) / GROUPS - FILLS * G / GROUPS;
        if constexpr (m > 0) __builtin_amdgcn_sched_group_barrier(kSgMfma, m, 0);
        if constexpr (f > 0) __builtin_amdgcn_sched_group_barrier(kSgVmemRead, f, 0);
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(kSgDsRead, r, 0);
        spread_groups<G + 1, GROUPS, READS, MFMAS, FILLS>();
    }
}

template <int READS, int MFMAS, int FILLS>
__device__ __forceinline__ void spread_hint() {
    constexpr int want = READS > FILLS ? READS : FILLS;
    constexpr int groups = want < 1 ? 1 : (want > MFMAS ? MFMAS : want);
    spread_groups<0, groups, READS, MFMAS, FILLS>();
}

// Fills FIRST..LAST-1 of a stage of BM rows of A followed by BN rows of B, in the numbering
// of dma_slab (fill j of this wavefront is 1 KB block j * NW + wave of the stage).
template <int FIRST, int LAST, int BM, int ROW_BYTES, int NW>
__device__ __forceinline__ void dma_part(unsigned char* stage, const unsigned char* a_slab,
                                         const unsigned char* b_slab, unsigned lane_off,
                                         size_t row_bytes, int wave) {
    constexpr int kRowsPerBlock = 1024 / ROW_BYTES;
    constexpr int kABlocks = BM / kRowsPerBlock;
#pragma unroll
    for (int j = FIRST; j < LAST; ++j) {
        const int blk = j * NW + wave;                 // block of the stage: A blocks, then B blocks
        const unsigned char* src = blk < kABlocks
            ? a_slab + (size_t)(blk * kRowsPerBlock) * row_bytes
            : b_slab + (size_t)((blk - kABlocks) * kRowsPerBlock) * row_bytes;
        __builtin_amdgcn_global_load_lds((global_void_ptr)(src + lane_off),
                                         (lds_void_ptr)(stage + blk * 1024), 16, 0, 0);
    }
}


// The same for the slab pipelines, shaped so that a fill costs two instructions (M0, load): the
// wavefront's fill j is 1 KB block j * NW + wave of the stage; blocks of A come first and BM / 8
// is a multiple of NW, so whether fill j reads A or B is known at compile time.  `a_k` / `b_k`
// are the wavefront-uniform addresses of the panels at this slab's k, voff[i] the lane's byte
// offset for the i-th block of an operand (its row inside block i * NW + wave, and the swizzled
// 16-byte chunk): uniform base + 32-bit lane offset is the scalar-base addressing form.
template <int FIRST, int LAST, int BM, int NW, int NV>
__device__ __forceinline__ void dma_blocks(unsigned char* stage_wave, const unsigned char* a_k,
                                           const unsigned char* b_k, const unsigned (&voff)[NV]) {
    constexpr int kAFills = BM / (8 * NW);
#pragma unroll
    for (int j = FIRST; j < LAST; ++j) {
        const unsigned char* src = j < kAFills ? a_k + voff[j] : b_k + voff[j - kAFills];
        __builtin_amdgcn_global_load_lds((global_void_ptr)src, (lds_void_ptr)(stage_wave + j * NW * 1024), 16, 0, 0);
    }
}

// fill j of the wavefront alone
template <int BM, int NW, int NV>
__device__ __forceinline__ void dma_one(int j, unsigned char* stage_wave, const unsigned char* a_k,
                                        const unsigned char* b_k, const unsigned (&voff)[NV]) {
    constexpr int kAFills = BM / (8 * NW);
    const unsigned char* src = j < kAFills ? a_k + voff[j] : b_k + voff[j - kAFills];
    __builtin_amdgcn_global_load_lds((global_void_ptr)src, (lds_void_ptr)(stage_wave + j * NW * 1024), 16, 0, 0);
}

// ------------------------------------------------------------------ pipelines
//
// Both are split in two: prologue() issues the first fills of a tile from the uniform addresses
// of its A and B row panels; main() takes the accumulators and runs the whole K loop.  When
// main() returns every fill has landed and every wavefront has passed a barrier, so the stages
// may be refilled at once - the kernel issues the next tile's prologue before it stores C.

// slab: NST = two or three stages of 64-deep slabs (the description is for two; with three the
// refill is slab s+3 and a fill has two slab times to land).  LDS row r (128 bytes) keeps logical chunk c at physical
// chunk c ^ ((r >> 1) & 7): a row covers half of the 64 banks (even rows the low half), a
// 128-bit read is served 16 consecutive rows per cycle, and (r >> 1) & 7 gives the 8 rows that
// share a half 8 distinct chunks.  Rows are whole 128-byte cache lines.
//
// Slab s lives in stage s % 2 and is multiplied in four k16 steps:
//     steps 0-2: MFMAs of the step | read the fragments of the next step
//     wait: own fills of slab s+1 landed, own LDS reads returned;  barrier
//     step 3:    MFMAs             | read step 0 of slab s+1 | issue the fills of slab s+2
//                                    into the stage slab s has just been read out of
// so a barrier costs no LDS latency and a fill has one slab time to land.  Fills past the
// last slab re-fetch it (nothing reads them).
template <typename T, int BM, int BN, int WGM, int WGN, int NST>
struct SlabPipe {
    static constexpr int NW = WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int BK = 64, ROW = BK * 2;
    static constexpr int A_BYTES = BM * ROW, STAGE = (BM + BN) * ROW;
    static constexpr int LDS_BYTES = NST * STAGE;
    static constexpr int FILLS = (BM + BN) / (8 * NW);
    static constexpr int K_ALIGN = 64;
    static constexpr bool kMfma16 = false;
    typedef typename Mfma32<T>::frag_t frag_t;

    static constexpr int NV = (BM > BN ? BM : BN) / (8 * NW);    // fills per wavefront and operand
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "whole fills per wavefront and operand");
    struct Lane {
        unsigned voff[NV];
        int a_rd, b_rd, half, swz;
    };

    static __device__ __forceinline__ void fill(unsigned char* st, const unsigned char* a_slab,
                                                const unsigned char* b_slab, size_t k_off, const Lane& ln,
                                                size_t row_bytes, int wave) {
        dma_blocks<0, FILLS, BM, NW, NV>(st + wave * 1024, a_slab + k_off, b_slab + k_off, ln.voff);
    }

    // With three stages a slab's fills go out in four parts, one per k16 step, so that the
    // vector-memory queue never holds more than a few of them: part 0 of slab s+3 in step 3 of
    // slab s (into the stage slab s has left), parts 1-3 in steps 0-2 of slab s+1.
    static constexpr int SPREAD = NST == 3;
    static constexpr int part_begin(int q) { return SPREAD ? FILLS * q / 4 : (q == 0 ? 0 : FILLS); }
    template <int Q>
    static __device__ __forceinline__ void fill_part(unsigned char* st, const unsigned char* a_slab,
                                                     const unsigned char* b_slab, size_t k_off, const Lane& ln,
                                                     size_t row_bytes, int wave) {
        dma_blocks<part_begin(Q), part_begin(Q + 1), BM, NW, NV>(st + wave * 1024, a_slab + k_off, b_slab + k_off,
                                                                 ln.voff);
    }
    template <int Q>
    static constexpr int part_size() { return part_begin(Q + 1) - part_begin(Q); }

    // f0 holds the fragments of (cur, step 0) on entry and of (nxt, step 0) on exit.  `prv` is the
    // stage of slab s-1 (three stages only), which takes parts 1-3 of slab s+2 (at k_prev).
    static __device__ __forceinline__ void slab(f32x16_t (&acc)[TM][TN], frag_t (&fa0)[TM], frag_t (&fb0)[TN],
                                                unsigned char* cur, const unsigned char* nxt, unsigned char* prv,
                                                const unsigned char* a_slab, const unsigned char* b_slab,
                                                size_t k_refill, size_t k_prev, const Lane& ln, size_t row_bytes,
                                                int wave
                                                ) {
        frag_t fa1[TM], fb1[TN];
        if constexpr (SPREAD) fill_part<1>(prv, a_slab, b_slab, k_prev, ln, row_bytes, wave);
        load_frags<T, TM, TN, ROW>(fa1, fb1, cur, ln.a_rd, ln.b_rd, ((2 + ln.half) ^ ln.swz) << 4);
        mma_step<T, TM, TN>(acc, fa0, fb0);
        spread_hint<TM + TN, TM * TN, SPREAD ? part_size<1>() : 0>();
        __builtin_amdgcn_sched_barrier(0);

        if constexpr (SPREAD) fill_part<2>(prv, a_slab, b_slab, k_prev, ln, row_bytes, wave);
        load_frags<T, TM, TN, ROW>(fa0, fb0, cur, ln.a_rd, ln.b_rd, ((4 + ln.half) ^ ln.swz) << 4);
        mma_step<T, TM, TN>(acc, fa1, fb1);
        spread_hint<TM + TN, TM * TN, SPREAD ? part_size<2>() : 0>();
        __builtin_amdgcn_sched_barrier(0);

        if constexpr (SPREAD) fill_part<3>(prv, a_slab, b_slab, k_prev, ln, row_bytes, wave);
        load_frags<T, TM, TN, ROW>(fa1, fb1, cur, ln.a_rd, ln.b_rd, ((6 + ln.half) ^ ln.swz) << 4);
        mma_step<T, TM, TN>(acc, fa0, fb0);
        spread_hint<TM + TN, TM * TN, SPREAD ? part_size<3>() : 0>();
        __builtin_amdgcn_sched_barrier(0);

        // own fills of slab s+1 landed (those of slab s+2, all younger, may fly on)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((NST - 2) * FILLS, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        fill_part<0>(cur, a_slab, b_slab, k_refill, ln, row_bytes, wave);
        load_frags<T, TM, TN, ROW>(fa0, fb0, nxt, ln.a_rd, ln.b_rd, ((0 + ln.half) ^ ln.swz) << 4);
        mma_step<T, TM, TN>(acc, fa1, fb1);
        spread_hint<TM + TN, TM * TN, part_size<0>()>();
        __builtin_amdgcn_sched_barrier(0);
    }

    // the stages are distinct objects: LDS reads of one never wait for fills of the other
    template <int I>
    static __device__ __forceinline__ unsigned char* stage() {
        __shared__ __attribute__((aligned(1024))) unsigned char st[STAGE];
        return st;
    }

    static __device__ __forceinline__ Lane make_lane(size_t row_bytes, int lane, int wave) {
        const int wm = wave / WGN, wn = wave % WGN;
        Lane ln;
        const int ld_row = lane >> 3;
        // blocks this wavefront fills are wave, wave + NW, ... (NW even): block parity = wave parity
        const int ld_chunk = (lane & 7) ^ ((((wave & 1) << 3 | ld_row) >> 1) & 7);
#pragma unroll
        for (int i = 0; i < NV; ++i)
            ln.voff[i] = (unsigned)(((i * NW + wave) * 8 + ld_row) * row_bytes) + ld_chunk * 16;
        ln.half = lane >> 5;
        ln.swz = (lane >> 1) & 7;
        ln.a_rd = (wm * WM + (lane & 31)) * ROW;
        ln.b_rd = A_BYTES + (wn * WN + (lane & 31)) * ROW;
        return ln;
    }

    // byte offset inside a row of slab i of this tile's cyclic walk: slab (i + rot) mod k_steps of K
    static __device__ __forceinline__ size_t slab_off(int i, int rot, int k_steps) {
        const int k = min(i, k_steps - 1) + rot;
        return (size_t)(k >= k_steps ? k - k_steps : k) * ROW;
    }

    // Issue the fills of the tile's first two slabs.  Needs nothing but free stages, so the caller
    // runs it ahead of the previous tile's epilogue.
    static __device__ __forceinline__ void prologue(const unsigned char* a_slab, const unsigned char* b_slab,
                                                    size_t row_bytes, int K, int k_rot, int lane, int wave) {
        const Lane ln = make_lane(row_bytes, lane, wave);
        const int k_steps = K / BK, rot = k_rot % k_steps;
        fill(stage<0>(), a_slab, b_slab, slab_off(0, rot, k_steps), ln, row_bytes, wave);
        fill(stage<1>(), a_slab, b_slab, slab_off(1, rot, k_steps), ln, row_bytes, wave);
        if constexpr (NST == 3) fill_part<0>(stage<2>(), a_slab, b_slab, slab_off(2, rot, k_steps), ln, row_bytes, wave);
    }

    // The K loop of a tile whose prologue has been issued.  On return every fill has landed and
    // every wavefront has passed a barrier: the stages are free.
    static __device__ __forceinline__ void main(f32x16_t (&acc)[TM][TN], const unsigned char* a_slab,
                                                const unsigned char* b_slab, size_t row_bytes, int K,
                                                int k_rot, int lane, int wave) {
        unsigned char* const stage0 = stage<0>();
        unsigned char* const stage1 = stage<1>();
        const Lane ln = make_lane(row_bytes, lane, wave);
        const int k_steps = K / BK;
        const int rot = k_rot % k_steps;

        // slab 0 landed; slab 1 (and part 0 of slab 2) may fly on
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(FILLS + (NST == 3 ? part_size<0>() : 0), true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        frag_t fa0[TM], fb0[TN];
        load_frags<T, TM, TN, ROW>(fa0, fb0, stage0, ln.a_rd, ln.b_rd, ((0 + ln.half) ^ ln.swz) << 4);

        auto run = [&](unsigned char* cur, const unsigned char* nxt, unsigned char* prv, int s) {
            slab(acc, fa0, fb0, cur, nxt, prv, a_slab, b_slab, slab_off(s + NST, rot, k_steps),
                 slab_off(s + 2, rot, k_steps), ln, row_bytes, wave);
        };
        if constexpr (NST == 2) {
            const int pairs = k_steps >> 1;
            for (int pr = 0; pr < pairs; ++pr) {
                run(stage0, stage1, stage1, 2 * pr);
                run(stage1, stage0, stage0, 2 * pr + 1);
            }
            if (k_steps & 1) run(stage0, stage1, stage1, k_steps - 1);
        } else {
            unsigned char* const stage2 = stage<2>();
            const int triples = k_steps / 3, rest = k_steps - 3 * triples;
            for (int tr = 0; tr < triples; ++tr) {
                run(stage0, stage1, stage2, 3 * tr);
                run(stage1, stage2, stage0, 3 * tr + 1);
                run(stage2, stage0, stage1, 3 * tr + 2);
            }
            if (rest >= 1) run(stage0, stage1, stage2, 3 * triples);
            if (rest == 2) run(stage1, stage2, stage0, 3 * triples + 1);
        }
        // drain the re-fetches of the last slab before anything refills the stages
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
};

template <typename T, int BM, int BN, int WGM, int WGN>
using PairPipe = SlabPipe<T, BM, BN, WGM, WGN, 2>;
// early: two stages again, for the tile of which only two fit (256x256), with the LDS reads of a
// slab bunched at its start so that its stage can be refilled during three of the four k16 steps
// instead of one.  A wavefront keeps the fragments of all four steps in registers (128 VGPRs):
//     step 3 of slab s-1: MFMAs | read the fragments of steps 0, 1 of slab s
//     step 0: MFMAs | read the fragments of steps 2, 3;  wait for them;  barrier: the stage is free
//     step 1: MFMAs | first third of the fills of slab s+2 into that stage
//     step 2: MFMAs | second third;  wait: own fills of slab s+1 landed;  barrier
//     step 3: MFMAs | last third | read steps 0, 1 of slab s+1
// 64 fills of 1 KB take the texture path of a compute unit about 1400 cycles, a k16 step of MFMAs
// 512: issued in one step they hold the wavefronts (and their MFMAs) up, spread over three they
// do not.
template <typename T, int BM, int BN, int WGM, int WGN>
struct EarlyPipe : SlabPipe<T, BM, BN, WGM, WGN, 2> {
    typedef SlabPipe<T, BM, BN, WGM, WGN, 2> Base;
    using Base::TM;
    using Base::TN;
    using Base::ROW;
    using Base::FILLS;
    using Base::NW;
    using Base::NV;
    using Base::BK;
    typedef typename Base::frag_t frag_t;
    typedef typename Base::Lane Lane;
    static constexpr int PA = (FILLS + 2) / 3, PB = (FILLS - PA + 1) / 2, PC = FILLS - PA - PB;

    template <int STEP>
    static __device__ __forceinline__ void read_step(frag_t (&fa)[TM], frag_t (&fb)[TN], const unsigned char* st,
                                                     const Lane& ln) {
        load_frags<T, TM, TN, ROW>(fa, fb, st, ln.a_rd, ln.b_rd, ((2 * STEP + ln.half) ^ ln.swz) << 4);
    }

    // MFMAS MFMAs with READS LDS reads bunched two per MFMA at the front and FILLS fills spread out
    template <int G, int MFMAS, int READS, int NFILL>
    static __device__ __forceinline__ void hint_front() {
        if constexpr (G < MFMAS) {
            __builtin_amdgcn_sched_group_barrier(kSgMfma, 1, 0);
            constexpr int r = (2 * (G + 1) < READS ? 2 * (G + 1) : READS) - (2 * G < READS ? 2 * G : READS);
            constexpr int f = NFILL * (G + 1) / MFMAS - NFILL * G / MFMAS;
            if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(kSgDsRead, r, 0);
            if constexpr (f > 0) __builtin_amdgcn_sched_group_barrier(kSgVmemRead, f, 0);
            hint_front<G + 1, MFMAS, READS, NFILL>();
        }
    }


    static __device__ __forceinline__ void slab(f32x16_t (&acc)[TM][TN], frag_t (&fa)[4][TM], frag_t (&fb)[4][TN],
                                                unsigned char* cur, const unsigned char* nxt,
                                                const unsigned char* a_slab, const unsigned char* b_slab,
                                                size_t k_refill, const Lane& ln, int wave
                                                ) {
        const unsigned char* a_k = a_slab + k_refill;
        const unsigned char* b_k = b_slab + k_refill;
        unsigned char* const dst = cur + wave * 1024;

        read_step<2>(fa[2], fb[2], cur, ln);
        read_step<3>(fa[3], fb[3], cur, ln);
        mma_step<T, TM, TN>(acc, fa[0], fb[0]);
        hint_front<0, TM * TN, 2 * (TM + TN), 0>();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, true));     // own reads of this stage returned
        __builtin_amdgcn_s_barrier();                          // everyone's: the stage is free
        __builtin_amdgcn_sched_barrier(0);

        dma_blocks<0, PA, BM, NW, NV>(dst, a_k, b_k, ln.voff);
        mma_step<T, TM, TN>(acc, fa[1], fb[1]);
        spread_hint<0, TM * TN, PA>();
        __builtin_amdgcn_sched_barrier(0);

        dma_blocks<PA, PA + PB, BM, NW, NV>(dst, a_k, b_k, ln.voff);
        mma_step<T, TM, TN>(acc, fa[2], fb[2]);
        spread_hint<0, TM * TN, PB>();
        __builtin_amdgcn_sched_barrier(0);
        // own fills of slab s+1 landed (the two thirds of slab s+2 issued since may fly on)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(PA + PB, false));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        dma_blocks<PA + PB, FILLS, BM, NW, NV>(dst, a_k, b_k, ln.voff);
        read_step<0>(fa[0], fb[0], nxt, ln);
        read_step<1>(fa[1], fb[1], nxt, ln);
        mma_step<T, TM, TN>(acc, fa[3], fb[3]);
        hint_front<0, TM * TN, 2 * (TM + TN), PC>();
        __builtin_amdgcn_sched_barrier(0);
    }

    static __device__ __forceinline__ void main(f32x16_t (&acc)[TM][TN], const unsigned char* a_slab,
                                                const unsigned char* b_slab, size_t row_bytes, int K,
                                                int k_rot, int lane, int wave) {
        unsigned char* const stage0 = Base::template stage<0>();
        unsigned char* const stage1 = Base::template stage<1>();
        const Lane ln = Base::make_lane(row_bytes, lane, wave);
        const int k_steps = K / BK;
        const int rot = k_rot % k_steps;

        __builtin_amdgcn_s_waitcnt(waitcnt_imm(FILLS, true));       // slab 0 landed; slab 1 may fly on
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        frag_t fa[4][TM], fb[4][TN];
        read_step<0>(fa[0], fb[0], stage0, ln);
        read_step<1>(fa[1], fb[1], stage0, ln);

        const int pairs = k_steps >> 1;
        for (int pr = 0; pr < pairs; ++pr) {
            slab(acc, fa, fb, stage0, stage1, a_slab, b_slab, Base::slab_off(2 * pr + 2, rot, k_steps), ln, wave);
            slab(acc, fa, fb, stage1, stage0, a_slab, b_slab, Base::slab_off(2 * pr + 3, rot, k_steps), ln, wave);
        }
        if (k_steps & 1)
            slab(acc, fa, fb, stage0, stage1, a_slab, b_slab, Base::slab_off(k_steps + 1, rot, k_steps), ln, wave);
        // drain the re-fetches of the last slab before anything refills the stages
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
};

// early16: the early-read pipeline on 16x16x32 MFMAs.  A wavefront's 128 x 128 part of the tile is 8 x 8 accumulators
// of 16 x 16; a slab is two k32 steps of 64 MFMAs, run as four quarters of 32 (row blocks 0-3 or 4-7 of A against all
// eight column blocks).  A k32 step needs eight fragments of A and eight of B (one 128-bit LDS read each, lane l:
// row l % 16, 16-byte chunk l / 16 of the step's four), so the fragments of both steps are again 128 VGPRs:
//     quarter 3 of slab s-1: MFMAs | read the fragments of k32 step 0 of slab s
//     quarter 0: MFMAs | read the fragments of step 1;  wait for them;  barrier: the stage is free
//     quarter 1: MFMAs | first third of the fills of slab s+2 into that stage
//     quarter 2: MFMAs | second third;  wait: own fills of slab s+1 landed;  barrier
//     quarter 3: MFMAs | last third | read step 0 of slab s+1
template <typename T, int BM, int BN, int WGM, int WGN>
struct EarlyPipe16 : SlabPipe<T, BM, BN, WGM, WGN, 2> {
    typedef SlabPipe<T, BM, BN, WGM, WGN, 2> Base;
    using Base::TM;
    using Base::TN;
    using Base::ROW;
    using Base::FILLS;
    using Base::NW;
    using Base::NV;
    using Base::BK;
    using Base::WM;
    using Base::WN;
    using Base::A_BYTES;
    typedef typename Base::frag_t frag_t;
    typedef typename Base::Lane Lane;
    static constexpr bool kMfma16 = true;
    static constexpr int RM = 2 * TM, RN = 2 * TN;          // 16-row blocks of A and of B per wavefront
    static constexpr int PA = (FILLS + 2) / 3, PB = (FILLS - PA + 1) / 2, PC = FILLS - PA - PB;
    static_assert(RM % 2 == 0, "two quarters of row blocks");

    struct Lane16 {
        int a_rd, b_rd, quad, swz;
    };
    static __device__ __forceinline__ Lane16 make_lane16(int lane, int wave) {
        const int wm = wave / WGN, wn = wave % WGN;
        Lane16 l;
        l.a_rd = (wm * WM + (lane & 15)) * ROW;
        l.b_rd = A_BYTES + (wn * WN + (lane & 15)) * ROW;
        l.quad = lane >> 4;
        l.swz = (lane >> 1) & 7;
        return l;
    }

    // fragment g of a k32 step: 0 .. RM-1 the row blocks of A, then those of B
    template <int STEP>
    static __device__ __forceinline__ void read_frag(frag_t (&fa)[RM], frag_t (&fb)[RN], const unsigned char* st,
                                                     const Lane16& l, int g) {
        const int chunk = ((4 * STEP + l.quad) ^ l.swz) << 4;
        if (g < RM) fa[g] = *reinterpret_cast<const frag_t*>(st + l.a_rd + g * 16 * ROW + chunk);
        else fb[g - RM] = *reinterpret_cast<const frag_t*>(st + l.b_rd + (g - RM) * 16 * ROW + chunk);
    }
    template <int STEP>
    static __device__ __forceinline__ void read_step(frag_t (&fa)[RM], frag_t (&fb)[RN], const unsigned char* st,
                                                     const Lane16& l) {
#pragma unroll
        for (int g = 0; g < RM + RN; ++g) read_frag<STEP>(fa, fb, st, l, g);
    }

    // One quarter: row blocks HALF * RM/2 .. of A against all column blocks, `between(g)` after MFMA g.  The MFMAs
    // are volatile assembly, so the memory operations that `between` issues stay where the source puts them.
    // B is the first operand: acc[i][j] holds D'[n][m] of rows m = 16 i .. and columns n = 16 j .. of the wavefront's
    // part, lane l the four consecutive n = 4 (l / 16) + 0..3 of row m = l % 16
    template <int HALF, typename F>
    static __device__ __forceinline__ void quarter(f32x4_t (&acc)[RM][RN], const frag_t (&fa)[RM], const frag_t (&fb)[RN],
                                                   F&& between) {
#pragma unroll
        for (int i = 0; i < RM / 2; ++i)
#pragma unroll
            for (int j = 0; j < RN; ++j) {
                Mfma16<T>::run(fb[j], fa[HALF * (RM / 2) + i], acc[HALF * (RM / 2) + i][j]);
                between(i * RN + j);
            }
    }

    // fill f of `count` goes out after MFMA g of Q when f * Q / count == g
    template <int FIRST, int COUNT>
    static __device__ __forceinline__ void fill_slot(int g, int q, unsigned char* dst, const unsigned char* a_k,
                                                     const unsigned char* b_k, const Lane& ln) {
#pragma unroll
        for (int f = 0; f < COUNT; ++f)
            if (f * q / COUNT == g) dma_one<BM, NW, NV>(FIRST + f, dst, a_k, b_k, ln.voff);
    }

    static __device__ __forceinline__ void slab(f32x4_t (&acc)[RM][RN], frag_t (&fa)[2][RM], frag_t (&fb)[2][RN],
                                                unsigned char* cur, const unsigned char* nxt,
                                                const unsigned char* a_slab, const unsigned char* b_slab,
                                                size_t k_refill, const Lane& ln, const Lane16& l16, int wave) {
        constexpr int Q = RM * RN / 2;                         // MFMAs of a quarter
        static_assert(RM + RN <= Q, "a fragment read per MFMA");
        const unsigned char* a_k = a_slab + k_refill;
        const unsigned char* b_k = b_slab + k_refill;
        unsigned char* const dst = cur + wave * 1024;

        quarter<0>(acc, fa[0], fb[0], [&](int g) { if (g < RM + RN) read_frag<1>(fa[1], fb[1], cur, l16, g); });
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, true));     // own reads of this stage returned
        __builtin_amdgcn_s_barrier();                          // everyone's: the stage is free

        quarter<1>(acc, fa[0], fb[0], [&](int g) { fill_slot<0, PA>(g, Q, dst, a_k, b_k, ln); });
        quarter<0>(acc, fa[1], fb[1], [&](int g) { fill_slot<PA, PB>(g, Q, dst, a_k, b_k, ln); });
        // own fills of slab s+1 landed (the two thirds of slab s+2 issued since may fly on)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(PA + PB, false));
        __builtin_amdgcn_s_barrier();

        quarter<1>(acc, fa[1], fb[1], [&](int g) {
            if (g < RM + RN) read_frag<0>(fa[0], fb[0], nxt, l16, g);
            fill_slot<PA + PB, PC>(g, Q, dst, a_k, b_k, ln);
        });
    }

    static __device__ __forceinline__ void main(f32x4_t (&acc)[RM][RN], const unsigned char* a_slab,
                                                const unsigned char* b_slab, size_t row_bytes, int K,
                                                int k_rot, int lane, int wave) {
        unsigned char* const stage0 = Base::template stage<0>();
        unsigned char* const stage1 = Base::template stage<1>();
        const Lane ln = Base::make_lane(row_bytes, lane, wave);
        const Lane16 l16 = make_lane16(lane, wave);
        const int k_steps = K / BK;
        const int rot = k_rot % k_steps;

        __builtin_amdgcn_s_waitcnt(waitcnt_imm(FILLS, true));       // slab 0 landed; slab 1 may fly on
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        frag_t fa[2][RM], fb[2][RN];
        read_step<0>(fa[0], fb[0], stage0, l16);

        const int pairs = k_steps >> 1;
        for (int pr = 0; pr < pairs; ++pr) {
            slab(acc, fa, fb, stage0, stage1, a_slab, b_slab, Base::slab_off(2 * pr + 2, rot, k_steps), ln, l16, wave);
            slab(acc, fa, fb, stage1, stage0, a_slab, b_slab, Base::slab_off(2 * pr + 3, rot, k_steps), ln, l16, wave);
        }
        if (k_steps & 1)
            slab(acc, fa, fb, stage0, stage1, a_slab, b_slab, Base::slab_off(k_steps + 1, rot, k_steps), ln, l16, wave);
        // drain the re-fetches of the last slab before anything refills the stages
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
        __builtin_amdgcn_s_barrier();
        mfma_result_wait_states();      // the accumulators are read by vector instructions from here on
        __builtin_amdgcn_sched_barrier(0);
    }
};

// slab16: the three-stage pipeline on 16x16x32 MFMAs, for the tiles of which three stages fit.  The quarters and the
// fragment reads are those of early16; a slab's fills go out in four parts as in `slab`: part 0 of slab s+3 in quarter 3
// of slab s (into the stage slab s has left), parts 1-3 in quarters 0-2 of slab s+1; two slabs in flight.
//     quarter 0: MFMAs (k32 step 0) | read the fragments of step 1 | part 1 of slab s+2
//     quarter 1: MFMAs (step 0)     | part 2
//     quarter 2: MFMAs (step 1)     | part 3;  wait: own fills of slab s+1 landed, own reads returned;  barrier
//     quarter 3: MFMAs (step 1)     | read step 0 of slab s+1 | part 0 of slab s+3 into this slab's stage
template <typename T, int BM, int BN, int WGM, int WGN>
struct SlabPipe16 : SlabPipe<T, BM, BN, WGM, WGN, 3> {
    typedef SlabPipe<T, BM, BN, WGM, WGN, 3> Base;
    typedef EarlyPipe16<T, BM, BN, WGM, WGN> Ops;            // fragment reads and quarters
    using Base::TM;
    using Base::TN;
    using Base::FILLS;
    using Base::NW;
    using Base::NV;
    using Base::BK;
    typedef typename Base::frag_t frag_t;
    typedef typename Base::Lane Lane;
    typedef typename Ops::Lane16 Lane16;
    static constexpr bool kMfma16 = true;
    static constexpr int RM = 2 * TM, RN = 2 * TN;

    template <int PART>
    static __device__ __forceinline__ void fill_slot(int g, int q, unsigned char* stage_wave, const unsigned char* a_k,
                                                     const unsigned char* b_k, const Lane& ln) {
        constexpr int first = Base::part_begin(PART), count = Base::part_begin(PART + 1) - first;
#pragma unroll
        for (int f = 0; f < count; ++f)
            if (f * q / count == g) dma_one<BM, NW, NV>(first + f, stage_wave, a_k, b_k, ln.voff);
    }

    static __device__ __forceinline__ void slab(f32x4_t (&acc)[RM][RN], frag_t (&fa)[2][RM], frag_t (&fb)[2][RN],
                                                unsigned char* cur, const unsigned char* nxt, unsigned char* prv,
                                                const unsigned char* a_slab, const unsigned char* b_slab,
                                                size_t k_refill, size_t k_prev, const Lane& ln, const Lane16& l16,
                                                int wave) {
        constexpr int Q = RM * RN / 2;                         // MFMAs of a quarter
        static_assert(RM + RN <= Q, "a fragment read per MFMA");
        unsigned char* const prv_w = prv + wave * 1024;
        const unsigned char* a_p = a_slab + k_prev;
        const unsigned char* b_p = b_slab + k_prev;

        Ops::template quarter<0>(acc, fa[0], fb[0], [&](int g) {
            if (g < RM + RN) Ops::template read_frag<1>(fa[1], fb[1], cur, l16, g);
            fill_slot<1>(g, Q, prv_w, a_p, b_p, ln);
        });
        Ops::template quarter<1>(acc, fa[0], fb[0], [&](int g) { fill_slot<2>(g, Q, prv_w, a_p, b_p, ln); });
        Ops::template quarter<0>(acc, fa[1], fb[1], [&](int g) { fill_slot<3>(g, Q, prv_w, a_p, b_p, ln); });
        // own fills of slab s+1 landed (those of slab s+2, all younger, may fly on)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(FILLS, true));
        __builtin_amdgcn_s_barrier();

        Ops::template quarter<1>(acc, fa[1], fb[1], [&](int g) {
            if (g < RM + RN) Ops::template read_frag<0>(fa[0], fb[0], nxt, l16, g);
            fill_slot<0>(g, Q, cur + wave * 1024, a_slab + k_refill, b_slab + k_refill, ln);
        });
    }

    static __device__ __forceinline__ void main(f32x4_t (&acc)[RM][RN], const unsigned char* a_slab,
                                                const unsigned char* b_slab, size_t row_bytes, int K,
                                                int k_rot, int lane, int wave) {
        unsigned char* const stage0 = Base::template stage<0>();
        unsigned char* const stage1 = Base::template stage<1>();
        unsigned char* const stage2 = Base::template stage<2>();
        const Lane ln = Base::make_lane(row_bytes, lane, wave);
        const Lane16 l16 = Ops::make_lane16(lane, wave);
        const int k_steps = K / BK;
        const int rot = k_rot % k_steps;

        // slab 0 landed; slab 1 and part 0 of slab 2 may fly on
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(FILLS + Base::template part_size<0>(), true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        frag_t fa[2][RM], fb[2][RN];
        Ops::template read_step<0>(fa[0], fb[0], stage0, l16);

        auto run = [&](unsigned char* cur, const unsigned char* nxt, unsigned char* prv, int s) {
            slab(acc, fa, fb, cur, nxt, prv, a_slab, b_slab, Base::slab_off(s + 3, rot, k_steps),
                 Base::slab_off(s + 2, rot, k_steps), ln, l16, wave);
        };
        const int triples = k_steps / 3, rest = k_steps - 3 * triples;
        for (int tr = 0; tr < triples; ++tr) {
            run(stage0, stage1, stage2, 3 * tr);
            run(stage1, stage2, stage0, 3 * tr + 1);
            run(stage2, stage0, stage1, 3 * tr + 2);
        }
        if (rest >= 1) run(stage0, stage1, stage2, 3 * triples);
        if (rest == 2) run(stage1, stage2, stage0, 3 * triples + 1);
        // drain the re-fetches of the last slab before anything refills the stages
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
        __builtin_amdgcn_s_barrier();
        mfma_result_wait_states();      // the accumulators are read by vector instructions from here on
        __builtin_amdgcn_sched_barrier(0);
    }
};

// the deepest arrangement that fits next to the wave table: three stages, or the early-read form
// (the kernel's own LDS: up to 4 KB of wave table, 32 rows x 80 bytes of C staging per wavefront)
template <typename T, int BM, int BN, int WGM, int WGN,
          bool THREE = (3 * (BM + BN) * 128 + WGM * WGN * 32 * 80 + 4096 <= 160 * 1024)>
struct DeepPipeSel {
    // a wavefront part of 64 x 64 (the 128x128 tile) is 2 % faster on 32x32x16 MFMAs: eight MFMAs per quarter
    // leave no room beside the fragment reads
    typedef typename std::conditional<(BM / WGM) * (BN / WGN) <= 64 * 64, SlabPipe<T, BM, BN, WGM, WGN, 3>,
                                      SlabPipe16<T, BM, BN, WGM, WGN>>::type type;
};
template <typename T, int BM, int BN, int WGM, int WGN>
struct DeepPipeSel<T, BM, BN, WGM, WGN, false> {
    typedef EarlyPipe16<T, BM, BN, WGM, WGN> type;
};
template <typename T, int BM, int BN, int WGM, int WGN>
using DeepPipe = typename DeepPipeSel<T, BM, BN, WGM, WGN>::type;

// the same choice on 32x32x16 MFMAs (SYN_GEMM_MFMA_32X32)
template <typename T, int BM, int BN, int WGM, int WGN,
          bool THREE = (3 * (BM + BN) * 128 + WGM * WGN * 32 * 80 + 4096 <= 160 * 1024)>
struct DeepPipe32Sel {
    typedef SlabPipe<T, BM, BN, WGM, WGN, 3> type;
};
template <typename T, int BM, int BN, int WGM, int WGN>
struct DeepPipe32Sel<T, BM, BN, WGM, WGN, false> {
    typedef EarlyPipe<T, BM, BN, WGM, WGN> type;
};
template <typename T, int BM, int BN, int WGM, int WGN>
using DeepPipe32 = typename DeepPipe32Sel<T, BM, BN, WGM, WGN>::type;

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
    static constexpr bool kMfma16 = false;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int BK = 32, ROW = BK * 2;
    static constexpr int A_BYTES = BM * ROW, STAGE = (BM + BN) * ROW;
    static constexpr int LDS_BYTES = 4 * STAGE;
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

    template <int I>
    static __device__ __forceinline__ unsigned char* stage() {
        __shared__ __attribute__((aligned(1024))) unsigned char st[STAGE];
        return st;
    }

    static __device__ __forceinline__ Lane make_lane(size_t row_bytes, int lane, int wave) {
        const int wm = wave / WGN, wn = wave % WGN;
        Lane ln;
        // 16 rows of 64 bytes per 1 KB block: lane l fills row l / 4, physical chunk l % 4
        ln.lane_off = (unsigned)((lane >> 2) * row_bytes) + (((lane & 3) ^ ((lane >> 4) & 3)) << 4);
        ln.a_rd = (wm * WM + (lane & 31)) * ROW;
        ln.b_rd = A_BYTES + (wn * WN + (lane & 31)) * ROW;
        const int half = lane >> 5, swz = (lane >> 2) & 3;
        ln.chunk0 = ((0 + half) ^ swz) << 4;
        ln.chunk1 = ((2 + half) ^ swz) << 4;
        return ln;
    }

    // slab i of this tile's cyclic walk is slab (i + rot) mod k_steps of K
    static __device__ __forceinline__ int slab_at(int i, int rot, int k_steps) {
        const int k = min(i, k_steps - 1) + rot;
        return k >= k_steps ? k - k_steps : k;
    }

    static __device__ __forceinline__ void prologue(const unsigned char* a_slab, const unsigned char* b_slab,
                                                    size_t row_bytes, int K, int k_rot, int lane, int wave) {
        const Lane ln = make_lane(row_bytes, lane, wave);
        const int k_steps = K / BK, rot = k_rot % k_steps;
        fill(stage<0>(), a_slab, b_slab, slab_at(0, rot, k_steps), ln, row_bytes, wave);
        fill(stage<1>(), a_slab, b_slab, slab_at(1, rot, k_steps), ln, row_bytes, wave);
        fill(stage<2>(), a_slab, b_slab, slab_at(2, rot, k_steps), ln, row_bytes, wave);
    }

    static __device__ __forceinline__ void main(f32x16_t (&acc)[TM][TN], const unsigned char* a_slab,
                                                const unsigned char* b_slab, size_t row_bytes, int K,
                                                int k_rot, int lane, int wave) {
        unsigned char* const st0 = stage<0>();
        unsigned char* const st1 = stage<1>();
        unsigned char* const st2 = stage<2>();
        unsigned char* const st3 = stage<3>();
        const Lane ln = make_lane(row_bytes, lane, wave);
        const int k_steps = K / BK, last = k_steps - 1;
        const int rot = k_rot % k_steps;

        __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * FILLS, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        frag_t fa0[TM], fb0[TN];
        load_frags<T, TM, TN, ROW>(fa0, fb0, st0, ln.a_rd, ln.b_rd, ln.chunk0);

        for (int s = 0; s <= last; s += 4) {
            step(acc, fa0, fb0, st0, st1, st3, a_slab, b_slab, slab_at(s + 3, rot, k_steps), ln, row_bytes, wave);
            step(acc, fa0, fb0, st1, st2, st0, a_slab, b_slab, slab_at(s + 4, rot, k_steps), ln, row_bytes, wave);
            step(acc, fa0, fb0, st2, st3, st1, a_slab, b_slab, slab_at(s + 5, rot, k_steps), ln, row_bytes, wave);
            step(acc, fa0, fb0, st3, st0, st2, a_slab, b_slab, slab_at(s + 6, rot, k_steps), ln, row_bytes, wave);
        }
        // drain the re-fetches of the last slab before anything refills the stages
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
};

// ------------------------------------------------------------------ kernel

// C += v (two consecutive elements) with one packed 16-bit atomic add
template <typename T>
__device__ __forceinline__ void atomic_add2(T* dst, unsigned v);

template <>
__device__ __forceinline__ void atomic_add2<__bf16>(__bf16* dst, unsigned v) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2* gptr;
    __builtin_amdgcn_global_atomic_fadd_v2bf16((gptr)dst, __builtin_bit_cast(v2, v));
}

template <>
__device__ __forceinline__ void atomic_add2<_Float16>(_Float16* dst, unsigned v) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2* gptr;
    __builtin_amdgcn_global_atomic_fadd_v2f16((gptr)dst, __builtin_bit_cast(v2, v));
}

// 16 bytes stored through the XCD's L2 to memory (the agent-scope form of a store: what a relaxed
// atomic store at that scope compiles to, which exists for 8 bytes at most).  A vector store.
// A store of more than 8 bytes reads its data registers for two more issue slots; the compiler
// keeps vector instructions that write them away from its own stores but does not see this one,
// hence the s_nop.
__device__ __forceinline__ void store16_write_through(void* dst, uint4 v) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 data = {v.x, v.y, v.z, v.w};
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(dst), "v"(data) : "memory");
}

template <typename T, typename Pipe, int BM, int BN, int WGM, int WGN, int MODE>
__global__ void __launch_bounds__(64 * WGM * WGN) gemm_wave_kernel(const GemmParams p) {
    constexpr bool PRODUCER = MODE == kProducer;
    constexpr bool REMOTE = MODE == kRemote || MODE == kRemoteAtomic;
    // a kernel of its own for the adding form: with both epilogues in one kernel the compiler spills some 170 registers
    // in the per-tile code, and the storing form runs 10 % slower than the producer it otherwise equals
    constexpr bool ATOMIC = MODE == kRemoteAtomic;
    constexpr int WM = BM / WGM, WN = BN / WGN;   // wavefront tile
    constexpr int TM = WM / 32, TN = WN / 32;     // 32x32 MFMA tiles per wavefront

    __shared__ int s_abort;
    __shared__ int s_spun;
    // C staging of the epilogue: 32 rows x CS_COLS columns per wavefront, 64 columns where LDS allows
    constexpr int NWAVES = WGM * WGN;
    constexpr int CS_COLS = ((BN / WGN / 32) % 2 == 0 &&
                             Pipe::LDS_BYTES + NWAVES * 32 * (64 * 2 + 16) + 4096 <= 160 * 1024) ? 64 : 32;
    __shared__ __attribute__((aligned(16))) unsigned char s_cstage[NWAVES * 32 * (CS_COLS * 2 + 16)];

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

    // --- wave table: the first kLdsWaves rows live in LDS, the walk reads them from there ---
    constexpr int kLdsWaves = 128;
    __shared__ int s_waves[kLdsWaves][5];
    for (int w = tid; w < min(p.num_waves, kLdsWaves); w += 64 * WGM * WGN) {
        s_waves[w][0] = p.wave_sizes[2 * w] / BM;
        s_waves[w][1] = p.wave_sizes[2 * w + 1] / BN;
        s_waves[w][2] = p.wave_offsets[2 * w] / BM;
        s_waves[w][3] = p.wave_offsets[2 * w + 1] / BN;
        s_waves[w][4] = p.signal_offsets[w];
    }
    if (tid == 0) s_abort = 0;
    __syncthreads();

    // --- wave walk state (uniform across the workgroup) ---
    int cur_wave = -1, past_tiles = 0, cur_tiles = 0;
    int cur_m = 0, cur_n = 0, off_m = 0, off_n = 0, cur_sig = -1;
    int cur_wait = -1;            // flag index the wave waits for: its own signal (consumer), the second table's (producer)
    const T* a_base = nullptr;
    T* c_base = nullptr;
    int dst_m = 0, dst_n = 0;
    int cur_k0 = 0, cur_klen = p.K;
    auto enter_wave = [&](int w) {
        cur_wave = w;
        if (w < kLdsWaves) {
            cur_m = s_waves[w][0];
            cur_n = s_waves[w][1];
            off_m = s_waves[w][2];
            off_n = s_waves[w][3];
            cur_sig = s_waves[w][4];
        } else {
            cur_m = p.wave_sizes[w * 2] / BM;
            cur_n = p.wave_sizes[w * 2 + 1] / BN;
            off_m = p.wave_offsets[w * 2] / BM;
            off_n = p.wave_offsets[w * 2 + 1] / BN;
            cur_sig = p.signal_offsets[w];
        }
        cur_wait = PRODUCER ? (p.wait_offsets != nullptr ? p.wait_offsets[w] : -1) : cur_sig;
        cur_tiles = cur_m * cur_n;
        if (REMOTE) {
            // the wave's peer: A rows are read from its shard and / or C tiles go into its buffer,
            // both addressed by wave-local rows (template_ag.py:151-161, template_rs.py:140-166)
            a_base = p.a_peers ? reinterpret_cast<const T*>(p.a_peers[p.a_target[w]]) : nullptr;
            if (p.c_peers) {
                c_base = reinterpret_cast<T*>(p.c_peers[p.c_target[w]]);
                dst_m = p.c_dst_offsets[2 * w];
                dst_n = p.c_dst_offsets[2 * w + 1];
            }
            if (p.wave_k) {
                cur_k0 = p.wave_k[2 * w];
                cur_klen = p.wave_k[2 * w + 1];
            }
        }
    };
    enter_wave(0);

    auto wait_flag = [&](int sig) -> bool {
        if (tid == 0) {
            const uint64_t* flags = PRODUCER ? p.wait_flags : p.flags;
            s_spun = __hip_atomic_load(flags + sig, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 1ull;
            if (s_spun && !spin_until_equal(flags + sig, 1ull, p.timeout_ticks)) {
                report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, cur_wave, pid, sig);
                s_abort = 1;
            }
        }
        __syncthreads();
        // No program reads a chunk's rows before its flag is up, so the XCD's L2 (emptied when the kernel
        // began) cannot hold a stale line of it.  The acquire fence drops every clean line of that L2 -
        // the panels of A and B its 28 other programs are reusing - so only a program that really had
        // to wait takes it.  That rests on the caller: nothing on the device reads the gathered buffer
        // between the start of this kernel and a chunk's flag, and no flag is raised twice during the
        // launch.  SYN_GEMM_ACQUIRE_ALWAYS is for callers that cannot promise that.
        if (s_spun || p.acquire_always) acquire_fence_agent();
        return s_abort == 0;
    };

    // the reference's consumer waits for wave 0 before it looks at its first tile (template.py:92-97)
    if (cur_wait >= 0) {
        if (!wait_flag(cur_wait)) return;
    }

    const T* __restrict__ A = reinterpret_cast<const T*>(p.a);
    const T* __restrict__ B = reinterpret_cast<const T*>(p.b);
    T* __restrict__ C = reinterpret_cast<T*>(p.c);

    // Move the walk to `tile_id`; true if that entered a wave whose flag has to be waited for.
    // -1 wave index afterwards: the table is shorter than the grid (host check failed).
    auto advance = [&](int tile_id) -> bool {
        bool new_wave = false;
        while (tile_id >= past_tiles + cur_tiles) {
            past_tiles += cur_tiles;
            if (cur_wave + 1 >= p.num_waves) {
                cur_wave = -1;
                return false;
            }
            enter_wave(cur_wave + 1);
            new_wave = true;
        }
        return new_wave && cur_wait >= 0;
    };

    struct Tile {
        const unsigned char* a_panel;    // first row of the tile's 'BM' rows of A
        const unsigned char* b_panel;    // first row of the tile's 'BN' rows of B
        T* c_tile;                       // element (0, 0) of the tile in its C buffer
        size_t ldc;
        int k_rot, wave, sig, wave_tiles;
        int k_len;                       // elements of K the tile contracts over (the panels start at its first k)
    };
    // get_pid_mn (template.py:10-18) on the wave-local tile id, and the tile's K phase
    auto locate = [&](int tile_id) -> Tile {
        const int local = tile_id - past_tiles;
        const int in_group = p.group_m * cur_n;
        const int group_id = local / in_group;
        const int first_m = group_id * p.group_m;
        const int gsz = min(cur_m - first_m, p.group_m);
        const int pid_m_local = first_m + (local % gsz);
        const int pid_n_local = (local % in_group) / gsz;
        const int pid_m = pid_m_local + off_m;
        const int pid_n = pid_n_local + off_n;
        if (p.visit_log != nullptr && tid == 0) {
            int4 rec = make_int4(pid, cur_wave, pid_m, pid_n);
            reinterpret_cast<int4*>(p.visit_log)[tile_id] = rec;
        }
        Tile t;
        t.a_panel = reinterpret_cast<const unsigned char*>(A + (size_t)pid_m * BM * K);
        t.b_panel = reinterpret_cast<const unsigned char*>(B + (size_t)pid_n * BN * K);
        t.c_tile = C + (size_t)pid_m * BM * N + (size_t)pid_n * BN;
        t.ldc = (size_t)N;
        if (REMOTE) {
            if (a_base) t.a_panel = reinterpret_cast<const unsigned char*>(a_base + (size_t)pid_m_local * BM * K);
            if (c_base) {
                t.ldc = (size_t)p.c_ld;
                t.c_tile = c_base + ((size_t)dst_m + (size_t)pid_m_local * BM) * t.ldc + dst_n + (size_t)pid_n_local * BN;
            }
        }
        // Tiles walk K cyclically, neighbouring tiles starting 128 elements apart.  With a
        // power-of-two row pitch, programs that all sweep K from 0 in lockstep keep hitting the
        // same few memory channels; four phases spread them while tiles that share a panel of A
        // or B still stay within 512 elements of each other (L2 reuse).
        t.k_rot = p.k_stagger ? ((pid_m + pid_n) & 3) * (128 / Pipe::BK) : 0;
        t.k_len = K;
        if (REMOTE) {
            t.a_panel += (size_t)cur_k0 * sizeof(T);
            t.b_panel += (size_t)cur_k0 * sizeof(T);
            t.k_len = cur_klen;
        }
        t.wave = cur_wave;
        t.sig = cur_sig;
        t.wave_tiles = cur_tiles;
        return t;
    };
    auto panel_a = [&](const Tile& t) { return t.a_panel; };
    auto panel_b = [&](const Tile& t) { return t.b_panel; };

    if (tiles_here == 0) return;
    if (advance(pid)) {
        if (!wait_flag(cur_wait)) return;
    }
    if (cur_wave < 0) return;
    Tile tile = locate(pid);
    Pipe::prologue(panel_a(tile), panel_b(tile), row_bytes, tile.k_len, tile.k_rot, lane, wave);

    for (int it = 0; it < tiles_here; ++it) {
        constexpr bool M16 = Pipe::kMfma16;                   // 16x16x32 MFMAs: 2 TM x 2 TN accumulators of four floats
        constexpr int AR = M16 ? 2 * TM : TM, AC = M16 ? 2 * TN : TN, AE = M16 ? 4 : 16;
        typename std::conditional<M16, f32x4_t, f32x16_t>::type acc[AR][AC];
#pragma unroll
        for (int i = 0; i < AR; ++i)
#pragma unroll
            for (int j = 0; j < AC; ++j)
#pragma unroll
                for (int e = 0; e < AE; ++e) acc[i][j][e] = 0.f;

        Pipe::main(acc, panel_a(tile), panel_b(tile), row_bytes, tile.k_len, tile.k_rot, lane, wave);

        // The stages are free: start the next tile's fills before this tile's C is stored, unless
        // the next tile opens a wave whose flag is still to be waited for (nothing of a chunk may
        // be read before its flag).
        const bool has_next = it + 1 < tiles_here;
        const int next_id = pid + (it + 1) * num_sms;
        bool gated = false;
        Tile next = tile;
        if (has_next) {
            gated = advance(next_id);
            if (cur_wave < 0) return;
            if (!gated) {
                next = locate(next_id);
                Pipe::prologue(panel_a(next), panel_b(next), row_bytes, next.k_len, next.k_rot, lane, wave);
            }
        }

        // Epilogue.  With B as the first MFMA operand a lane holds, for column m = lane % 32 of
        // D', rows n = 8g + 4*(lane/32) + 0..3: four consecutive elements of one row of C.
        {
            // A store instruction of those groups would touch 32 rows with 16 bytes each, and the
            // texture path takes a cycle per cache line touched.  So a strip of 32 rows x CS_COLS
            // columns goes through a private piece of LDS (rows padded by 16 bytes) and leaves as
            // 16 bytes per lane, whole rows of the strip side by side: 8 or 16 lines per instruction.
            constexpr int CS_ROW = CS_COLS * 2 + 16;          // bytes per staged row
            constexpr int LPR = CS_COLS / 8;                  // lanes per row on the way out
            constexpr int RPI = 64 / LPR;                     // rows per store instruction
            unsigned char* const cs = s_cstage + wave * (32 * CS_ROW);
            unsigned char* const cs_wr = M16 ? cs + (lane & 15) * CS_ROW + 8 * (lane >> 4)
                                             : cs + (lane & 31) * CS_ROW + 8 * (lane >> 5);
            const unsigned char* const cs_rd = cs + (lane / LPR) * CS_ROW + (lane % LPR) * 16;
            T* const c_out = tile.c_tile + (size_t)(wm * WM + lane / LPR) * tile.ldc + wn * WN + (lane % LPR) * 8;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int js = 0; js < TN; js += CS_COLS / 32) {
                    if constexpr (M16) {
                        // the strip's 32 rows are two 16-row blocks, its columns CS_COLS / 16 blocks of 32 bytes
#pragma unroll
                        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                            for (int jb = 0; jb < CS_COLS / 16; ++jb)
                                *reinterpret_cast<uint2*>(cs_wr + rb * 16 * CS_ROW + jb * 32) =
                                    pack4<T>(acc[2 * i + rb][2 * js + jb][0], acc[2 * i + rb][2 * js + jb][1],
                                             acc[2 * i + rb][2 * js + jb][2], acc[2 * i + rb][2 * js + jb][3]);
                    } else {
#pragma unroll
                    for (int jj = 0; jj < CS_COLS / 32; ++jj)
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            *reinterpret_cast<uint2*>(cs_wr + jj * 64 + g * 16) =
                                pack4<T>(acc[i][js + jj][4 * g], acc[i][js + jj][4 * g + 1],
                                         acc[i][js + jj][4 * g + 2], acc[i][js + jj][4 * g + 3]);
                    }
                    if constexpr (ATOMIC) {
                        // one packed atomic per lane, the lanes of an instruction side by side in a row: every
                        // instruction adds into whole cache lines.  (Issued as 8 or 16 bytes per lane - four
                        // instructions that each touch a quarter of every line - the atomic form of the
                        // 8192 x 8192 x 3584 GEMM took 0.82-0.86 ms against 0.33 for the stores.)
                        constexpr int DPR = CS_COLS / 2;          // dwords of a staged row
                        constexpr int RPA = 64 / DPR;             // rows per atomic instruction
                        // (one carried address: written as a product per row, the unrolled loops keep dozens of 64-bit
                        // row addresses alive and the kernel spills them)
                        T* row_ptr = tile.c_tile + (size_t)(wm * WM + 32 * i + lane / DPR) * tile.ldc + wn * WN + 32 * js +
                                     (lane % DPR) * 2;
#pragma unroll
                        for (int t = 0; t < 32 / RPA; ++t) {
                            const int row = t * RPA + lane / DPR;
                            const unsigned v = *reinterpret_cast<const unsigned*>(cs + row * CS_ROW + (lane % DPR) * 4);
                            atomic_add2<T>(row_ptr, v);
                            row_ptr += (size_t)RPA * tile.ldc;
                            asm volatile("" : "+v"(row_ptr));
                        }
                        continue;
                    }
#pragma unroll
                    for (int t = 0; t < 32 / RPI; ++t) {
                        const uint4 v = *reinterpret_cast<const uint4*>(cs_rd + t * RPI * CS_ROW);
                        T* dst = c_out + (size_t)(32 * i + t * RPI) * tile.ldc + 32 * js;
                        if constexpr (REMOTE) {
                            // peer buffers need only be 8-byte aligned (two 8-byte stores per lane); where the
                            // tile's rows sit on 16-byte boundaries, one store.  (Tested here, on the address: as
                            // a field of the tile record the same fact moved the kernel's LDS layout, and the
                            // consumer and producer forms - which never look at it - fetched 30 % more from HBM.)
                            if (reinterpret_cast<uintptr_t>(dst) % 16 == 0) {
                                *reinterpret_cast<uint4*>(dst) = v;
                            } else {
                                const uint2 lo = {v.x, v.y}, hi = {v.z, v.w};
                                *reinterpret_cast<uint2*>(dst) = lo;
                                *reinterpret_cast<uint2*>(dst + 4) = hi;
                            }
                        } else if (PRODUCER) {
                            // written through the XCD's L2: the release below then has nothing
                            // of this tile left to write back
                            store16_write_through(dst, v);
                        } else {
                            *reinterpret_cast<uint4*>(dst) = v;
                        }
                    }
                }
        }

        if (PRODUCER) {
            if (tile.sig >= 0) {
                // Every lane's C stores were agent-scope write-through stores; the wait for their
                // acknowledgements in front of the barrier makes them visible device-wide before
                // thread 0 moves the count.  The count itself is a relaxed atomic: a release would
                // make the L2 look for dirty lines to write back once per tile, and there are none.
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
                __syncthreads();
                if (tid == 0) {
                    const int done = __hip_atomic_fetch_add(p.counters + tile.wave, 1, __ATOMIC_RELAXED,
                                                            __HIP_MEMORY_SCOPE_AGENT);
                    if (done == tile.wave_tiles - 1)
                        __hip_atomic_store(p.flags + tile.sig, 1ull, __ATOMIC_RELEASE,
                                           __HIP_MEMORY_SCOPE_SYSTEM);
                }
            }
        }

        if (has_next && gated) {
            if (!wait_flag(cur_wait)) return;
            next = locate(next_id);
            Pipe::prologue(panel_a(next), panel_b(next), row_bytes, next.k_len, next.k_rot, lane, wave);
        }
        tile = next;
    }
}

// ---------------------------------------------------------------- host side

static int64_t gemm_num_tiles(int64_t cum_tiles, int M, int N, int bm, int bn) {
    if (cum_tiles > 0) return (cum_tiles + (int64_t)bm * bn - 1) / ((int64_t)bm * bn);
    return (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
}

template <typename T, template <typename, int, int, int, int> class PipeT, int BM, int BN, int WGM, int WGN,
          int MODE>
static int launch_gemm(const GemmParams& p, int grid, hipStream_t stream) {
    typedef PipeT<T, BM, BN, WGM, WGN> Pipe;
    hipLaunchKernelGGL((gemm_wave_kernel<T, Pipe, BM, BN, WGM, WGN, MODE>), dim3(grid),
                       dim3(64 * WGM * WGN), 0, stream, p);
    return (int)hipGetLastError();
}

// Workgroup shapes: 4 wavefronts (2x2, one per SIMD) or 8 (two per SIMD: one can issue MFMAs
// while the other waits for LDS or a barrier).
template <typename T, template <typename, int, int, int, int> class PipeT, int MODE>
static int dispatch_tile(const GemmParams& p, int bm, int bn, bool eight, int grid, hipStream_t stream) {
    if (eight) {
        if (bm == 256 && bn == 256) return launch_gemm<T, PipeT, 256, 256, 2, 4, MODE>(p, grid, stream);
        if (bm == 128 && bn == 256) return launch_gemm<T, PipeT, 128, 256, 2, 4, MODE>(p, grid, stream);
        if (bm == 256 && bn == 128) return launch_gemm<T, PipeT, 256, 128, 4, 2, MODE>(p, grid, stream);
        return SYN_EINVAL;
    }
    if (bm == 256 && bn == 256) return launch_gemm<T, PipeT, 256, 256, 2, 2, MODE>(p, grid, stream);
    // 256x224: four wavefronts stacked in M, each 64 rows x 224 columns (2 x 7 MFMA tiles); N = 3584
    // is 16 of these, and 32 x 16 tiles are two full rounds of 256 programs
    if constexpr (PipeT<T, 256, 224, 4, 1>::K_ALIGN == 64)
        if (bm == 256 && bn == 224) return launch_gemm<T, PipeT, 256, 224, 4, 1, MODE>(p, grid, stream);
    if (bm == 128 && bn == 256) return launch_gemm<T, PipeT, 128, 256, 2, 2, MODE>(p, grid, stream);
    if (bm == 256 && bn == 128) return launch_gemm<T, PipeT, 256, 128, 2, 2, MODE>(p, grid, stream);
    if (bm == 128 && bn == 128) return launch_gemm<T, PipeT, 128, 128, 2, 2, MODE>(p, grid, stream);
    return SYN_EINVAL;
}

template <typename T, int MODE>
static int dispatch_pipe(const GemmParams& p, int bm, int bn, bool eight, bool ring, bool two_stage, bool mfma32,
                         int grid, hipStream_t stream) {
    // the remote-binding form exists for the default pipeline only
    if (MODE < kRemote) {
        if (ring) return dispatch_tile<T, RingPipe, MODE >= kRemote ? kConsumer : MODE>(p, bm, bn, eight, grid, stream);
        if (two_stage) return dispatch_tile<T, PairPipe, MODE >= kRemote ? kConsumer : MODE>(p, bm, bn, eight, grid, stream);
    }
    // tiles of which three stages do not fit have two forms of the early-read pipeline
    if (mfma32) return dispatch_tile<T, DeepPipe32, MODE>(p, bm, bn, eight, grid, stream);
    return dispatch_tile<T, DeepPipe, MODE>(p, bm, bn, eight, grid, stream);
}

__global__ void __launch_bounds__(256) clear_words_kernel(int32_t* words, int n);

// the tile shapes dispatch_tile has kernels for
static bool gemm_tile_shape_built(int bm, int bn, bool eight) {
    const bool common = (bm == 256 && bn == 256) || (bm == 128 && bn == 256) || (bm == 256 && bn == 128);
    return common || (!eight && ((bm == 256 && bn == 224) || (bm == 128 && bn == 128)));
}

// clear_counters > 0: the first that many words of `counters` are zeroed on the stream in front of the kernel,
// once every check has passed (a rejected call must not touch counters a running launch may own).
static int gemm_entry(const syn_gemm_desc* d, hipStream_t stream, int mode,
                      const syn_gemm_remote* remote = nullptr, const uint64_t* wait_flags = nullptr,
                      const int32_t* wait_signal_offsets = nullptr, int clear_counters = 0) {
    if (d == nullptr) return SYN_EINVAL;
    const bool producer = mode == kProducer;
    if ((wait_flags == nullptr) != (wait_signal_offsets == nullptr)) return SYN_EINVAL;
    if (wait_flags && !producer) return SYN_EINVAL;      // a consumer waits on `flags` itself
    const bool a_remote = remote && remote->a_peers, c_remote = remote && remote->c_peers;
    if (mode == kRemote) {
        if (!remote || (!a_remote && !c_remote)) return SYN_EINVAL;
        if (a_remote && !remote->a_target_rank) return SYN_EINVAL;
        if (c_remote && (!remote->c_target_rank || !remote->c_dst_offsets || remote->c_ld <= 0)) return SYN_EINVAL;
        if (c_remote && remote->c_ld % 4) return SYN_EALIGN;
        if (remote->c_atomic_add && !c_remote) return SYN_EINVAL;
        if (remote->k_ranges && !(c_remote && remote->c_atomic_add)) return SYN_EINVAL;   // partial products are added
    }
    if ((!d->a && !a_remote) || !d->b || (!d->c && !c_remote) || !d->wave_sizes || !d->wave_offsets ||
        !d->signal_offsets)
        return SYN_EINVAL;
    if (d->num_waves <= 0 || d->M <= 0 || d->N <= 0 || d->K <= 0) return SYN_EINVAL;
    if (d->block_k != 64) return SYN_EINVAL;
    if (d->group_m <= 0 || d->num_sms <= 0) return SYN_EINVAL;
    if (d->dtype != SYN_DTYPE_BF16 && d->dtype != SYN_DTYPE_FP16) return SYN_EINVAL;
    if (d->M % d->block_m || d->N % d->block_n || d->K % 64) return SYN_EINVAL;
    if ((d->a && !aligned16(d->a)) || !aligned16(d->b) || (d->c && !aligned16(d->c))) return SYN_EALIGN;
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
    p.wait_flags = wait_flags;
    p.wait_offsets = wait_signal_offsets;
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
    p.acquire_always = (d->options & SYN_GEMM_ACQUIRE_ALWAYS) ? 1 : 0;
    p.a_peers = a_remote ? remote->a_peers : nullptr;
    p.a_target = a_remote ? remote->a_target_rank : nullptr;
    p.c_peers = c_remote ? remote->c_peers : nullptr;
    p.c_target = c_remote ? remote->c_target_rank : nullptr;
    p.c_dst_offsets = c_remote ? remote->c_dst_offsets : nullptr;
    p.c_ld = c_remote ? remote->c_ld : 0;
    p.c_atomic = (remote && remote->c_atomic_add) ? 1 : 0;
    p.wave_k = remote ? remote->k_ranges : nullptr;
    const bool eight = (d->options & SYN_GEMM_EIGHT_WAVES) != 0;
    // the ring needs whole groups of four 32-deep slabs (and does not exist for 224-wide tiles)
    const bool ring = (d->options & SYN_GEMM_RING_PIPE) && d->K % 128 == 0 && d->block_n != 224;

    const int bm = d->block_m, bn = d->block_n;
    const bool two = (d->options & SYN_GEMM_TWO_STAGE) != 0;
    const bool m32 = (d->options & SYN_GEMM_MFMA_32X32) != 0;
    if (!gemm_tile_shape_built(bm, bn, eight)) return SYN_EINVAL;
    if (clear_counters > 0) {
        hipLaunchKernelGGL(clear_words_kernel, dim3((clear_counters + 255) / 256), dim3(256), 0, stream, d->counters,
                           clear_counters);
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) return (int)err;
    }
    if (d->dtype == SYN_DTYPE_BF16) {
        if (mode == kRemote)
            return p.c_atomic ? dispatch_pipe<__bf16, kRemoteAtomic>(p, bm, bn, eight, false, false, m32, grid, stream)
                              : dispatch_pipe<__bf16, kRemote>(p, bm, bn, eight, false, false, m32, grid, stream);
        return producer ? dispatch_pipe<__bf16, kProducer>(p, bm, bn, eight, ring, two, m32, grid, stream)
                        : dispatch_pipe<__bf16, kConsumer>(p, bm, bn, eight, ring, two, m32, grid, stream);
    }
    if (mode == kRemote)
        return p.c_atomic ? dispatch_pipe<_Float16, kRemoteAtomic>(p, bm, bn, eight, false, false, m32, grid, stream)
                          : dispatch_pipe<_Float16, kRemote>(p, bm, bn, eight, false, false, m32, grid, stream);
    return producer ? dispatch_pipe<_Float16, kProducer>(p, bm, bn, eight, ring, two, m32, grid, stream)
                    : dispatch_pipe<_Float16, kConsumer>(p, bm, bn, eight, ring, two, m32, grid, stream);
}

// ---- the producer entry point that allocates nothing ----
//
// Its per-wave tile counters live in a file-scope device array instead of caller memory.  Every
// device the library runs on holds its own copy of the array at its own address; the address is
// looked up once per device and used from then on wherever host code needs the array's memory.
constexpr int kStaticCounterWords = SYN_STATIC_MAX_WAVES;      // 16 KB per device
static __device__ __align__(256) int32_t scratch[kStaticCounterWords];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static int32_t* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device (0, a SYN_E* code or a hipError_t)
static int scratch_address(int32_t** out) {
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return (int)err;
    if (dev < 0 || dev >= kMaxDevices) return SYN_EINVAL;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return (int)err;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = reinterpret_cast<int32_t*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

// a fill kernel rather than a memset: a memset node in a captured graph is not reliable on replay
__global__ void __launch_bounds__(256) clear_words_kernel(int32_t* words, int n) {
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i < n) words[i] = 0;
}

}  // namespace syn

extern "C" {

int syn_gemm_producer_static(const syn_gemm_desc* desc, syn_stream_t stream) {
    using namespace syn;
    if (desc == nullptr) return SYN_EINVAL;
    if (desc->counters != nullptr) return SYN_EINVAL;        // the counters are the library's here
    if (desc->num_waves <= 0) return SYN_EINVAL;
    if (desc->num_waves > kStaticCounterWords) return SYN_E2BIG;
    int32_t* counters = nullptr;
    const int rc = scratch_address(&counters);
    if (rc != 0) return rc;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    syn_gemm_desc d = *desc;
    d.counters = counters;
    // the array keeps the last call's counts: the words this launch uses are zeroed in front of the kernel,
    // behind every check of the descriptor
    return gemm_entry(&d, s, kProducer, nullptr, nullptr, nullptr, desc->num_waves);
}

int syn_gemm_static_counters_peek(int32_t* host_out, int32_t count) {
    using namespace syn;
    if (host_out == nullptr || count <= 0 || count > kStaticCounterWords) return SYN_EINVAL;
    int32_t* counters = nullptr;
    const int rc = scratch_address(&counters);
    if (rc != 0) return rc;
    return (int)hipMemcpy(host_out, counters, sizeof(int32_t) * (size_t)count, hipMemcpyDeviceToHost);
}

int syn_gemm_consumer(const syn_gemm_desc* desc, syn_stream_t stream) {
    return syn::gemm_entry(desc, reinterpret_cast<hipStream_t>(stream), syn::kConsumer);
}

int syn_gemm_producer(const syn_gemm_desc* desc, syn_stream_t stream) {
    return syn::gemm_entry(desc, reinterpret_cast<hipStream_t>(stream), syn::kProducer);
}

int syn_gemm_consumer_producer(const syn_gemm_desc* desc, const uint64_t* wait_flags,
                               const int32_t* wait_signal_offsets, syn_stream_t stream) {
    if (wait_flags == nullptr || wait_signal_offsets == nullptr) return SYN_EINVAL;
    return syn::gemm_entry(desc, reinterpret_cast<hipStream_t>(stream), syn::kProducer, nullptr, wait_flags,
                           wait_signal_offsets);
}

int syn_gemm_remote_binding(const syn_gemm_desc* desc, const syn_gemm_remote* remote, syn_stream_t stream) {
    return syn::gemm_entry(desc, reinterpret_cast<hipStream_t>(stream), syn::kRemote, remote);
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
