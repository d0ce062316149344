// Chunked-KV flash attention forward for gfx950 (MI355X), head_dim 128.
//
// Work decomposition follows the reference kernel (syncopate/computation/attn/
// template.py:80-121, generated form transformer.py:555-660): tile id ->
// schedule wave -> (z, h, 128-row q block, kv block range); the program waits
// for the wave's flag, computes the partial attention of its q block over the
// kv range with a base-2 online softmax (template.py:173-300) and merges
// (O, lse2) into the output under a per-q-block lock (template.py:307-361).
// Programs are persistent: workgroup b runs tile ids b, b + grid, ... in
// increasing order, so an early (already arrived) wave is never queued behind a
// later one.
//
// Data path per 128-row kv block, 4 wavefronts x 32 q rows each:
//   S^T[kv, q] = K[kv, :] . Q[q, :]      K from LDS (A operand), Q fragments in registers
//   P^T        = exp2(S^T * scale - m)   per-q statistics are lane-local: lane % 32 == q
//   O^T[d, q] += V^T[d, kv] . P^T[kv, q] V row-major in LDS, read with transposing LDS loads
// Computing the transposed products keeps each q column in one lane pair, so
// the softmax needs one cross-lane exchange per block, and the accumulator
// layout of S^T is already the B-operand layout of the second product.
//
// K and V blocks go from HBM straight into LDS (global_load_lds_dwordx4, no register
// staging): the fills of V block n are issued between the MFMAs of S^T of block n, those of
// K block n+1 between the exponentials of block n, one at a time so that the in-order
// wavefront is never held at the vector-memory queue.
// The kernel stays under 256 registers and 80 KB of LDS, so two workgroups share a compute
// unit and one's exponentials overlap the other's matrix work.
#include <array>
#include <map>
#include <type_traits>
#include <vector>

#include "common.h"

namespace syn {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

struct AttnParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    float* lse;
    int32_t* lock;
    int32_t* first;
    uint64_t* flags;
    const int32_t* wave_offsets;
    const int32_t* wave_sizes;
    const int32_t* cum_wave_sizes;
    const int32_t* signal_offsets;
    int32_t* visit_log;
    int32_t* status;
    int32_t* counters;
    const uint64_t* wait_flags;          // producer form that is a consumer as well: flags to wait for ...
    const int32_t* wait_offsets;         // ... and the index per wave (-1: none)
    int64_t timeout_ticks;
    int32_t num_waves;
    int32_t Z, H, Sq, Skv;
    int32_t causal;
    int32_t num_tiles;
    int32_t xcd_remap;    // workgroups of one XCD take consecutive tiles (see logical_program_id)
    int32_t acquire_always;   // SYN_ATTN_ACQUIRE_ALWAYS: fence behind every flag wait, not only behind a spin
    const int32_t* work_list; // SYN_ATTN_WORK_LIST: [grid + 1] entry offsets, then the entries
    float qk_scale;       // sm_scale * 1.44269504 (template.py:178-179)
    // element strides {batch, head, row}
    int64_t q_st[3], k_st[3], v_st[3], o_st[3];
};

constexpr int kAttnThreads = 256;
constexpr int kHeadDim = 128;
constexpr int kBlockM = 128;
constexpr int kBlockN = 128;
constexpr int kRowBytes = kHeadDim * 2;             // 256: one row of K or V
constexpr int kBlockBytes = kBlockN * kRowBytes;    // 32768: one kv block of K or of V
constexpr int kFills = kBlockBytes / 1024 / 4;      // 8 fills of 1 KB per wavefront and block

template <typename T>
struct AttnMfma;

template <>
struct AttnMfma<__bf16> {
    typedef bf16x8_t frag_t;
    static __device__ __forceinline__ f32x16_t run(frag_t a, frag_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

template <>
struct AttnMfma<_Float16> {
    typedef f16x8_t frag_t;
    static __device__ __forceinline__ f32x16_t run(frag_t a, frag_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// The paired kernel's products: v_mfma_f32_16x16x32 (A: 16 rows x 32 k, lane l holds row l % 16, k 8 (l / 16) .. + 8;
// B: 32 k x 16 columns, lane l holds column l % 16, the same k; C: lane l holds column l % 16, rows 4 (l / 16) .. + 4).
// Same flop per cycle as the 32x32x16 form, and on random operands 11 % less energy per flop for the bare
// instruction (syn_probe_mfma_rate) - this kernel runs at the board's power limit, so that is speed.
template <typename T>
__device__ __forceinline__ f32x4_t mfma16(typename AttnMfma<T>::frag_t a, typename AttnMfma<T>::frag_t b, f32x4_t c);
template <>
__device__ __forceinline__ f32x4_t mfma16<__bf16>(bf16x8_t a, bf16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_t mfma16<_Float16>(f16x8_t a, f16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// The merged partial results (O, lse) of a q block pass from workgroup to workgroup, possibly on
// different XCDs, whose L2s are not coherent with each other.  A release / acquire fence pair
// would do it - but a release writes back every dirty line of the XCD's L2 and an acquire drops
// its clean lines, for all 32 compute units, once per tile: measured, the fences alone kept the
// kernel at two thirds of its time.  So these few words are stored THROUGH the L2 and loaded PAST
// it (the agent-scope forms of a store and a load), and the lock hand-over needs no fence: the
// stores have been acknowledged by memory before the lock word is written.
template <typename V>
__device__ __forceinline__ V load8_coherent(const void* ptr) {
    const uint64_t bits = __hip_atomic_load(reinterpret_cast<const uint64_t*>(ptr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(V, bits);
}
template <typename V>
__device__ __forceinline__ void store8_through(void* ptr, V value) {
    __hip_atomic_store(reinterpret_cast<uint64_t*>(ptr), __builtin_bit_cast(uint64_t, value), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_f32_coherent(const float* ptr) {
    return __builtin_bit_cast(float, __hip_atomic_load(reinterpret_cast<const uint32_t*>(ptr), __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ void store_f32_through(float* ptr, float value) {
    __hip_atomic_store(reinterpret_cast<uint32_t*>(ptr), __builtin_bit_cast(uint32_t, value), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// The hand-over of a q block's lock.  What orders it in hardware: every lane's stores of O and lse are
// write-through stores whose acknowledgement (s_waitcnt vmcnt(0)) means they have reached memory, the
// barrier collects all lanes, and thread 0's `first` store is acknowledged the same way before the lock word
// goes out; the next holder reads past its L2.  These two fences add nothing to that on this part (at
// workgroup scope they write back and invalidate nothing): they tell the COMPILER that the relaxed atomics
// around them may not change places.
__device__ __forceinline__ void lock_release_fence() { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup"); }
__device__ __forceinline__ void lock_taken_fence() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup"); }

// max(x of this lane, x of lane ^ 32) and the same for lane ^ 16, on the vector ALU: v_permlane32_swap exchanges
// lanes 32..63 of its first operand with lanes 0..31 of its second, v_permlane16_swap the odd rows of 16 lanes of the
// first with the even rows of the second - given two copies of x, every lane then holds its own value in one and
// its partner's in the other.  (__shfl_xor is an LDS instruction, ds_bpermute: in the paired kernel it would queue
// behind the LDS reads of the four wavefronts that are in their products, and the softmax waits for it twice.)
// Written as assembly because the compiler's own builtins for these two instructions fold max(first result, second
// result) into the first result; the s_nop before and after are the ones it places around them itself.
__device__ __forceinline__ float max_with_lane_xor32(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}
__device__ __forceinline__ float max_with_lane_xor16(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// The merge of a wavefront's 32 q rows into the output: O = O_stored * w_old + O_new * w_new, rounded to
// the output type (template.py:335-361), with lse beside it.  In the accumulator layout a lane owns
// scattered 8-byte pieces of one row (4 columns out of every 32, one row 256 bytes from the next): stored
// through the L2 like that, every piece travels to memory as a partial line, and the merge of one
// tile took 20 us - as much with the locks already held and the stored result read from the L2 as
// with the whole protocol, so it was the traffic and not the round trips.  Here the rows pass
// through a tile in LDS that belongs to the
// wavefront (the K and V blocks are free during the epilogue): memory is read and written in the
// layout "instruction k: rows 2k and 2k + 1, lane l the 8 bytes at 8 * (l % 32) of row 2k + l / 32",
// i.e. whole 256-byte rows, two full lines each.  Rows are 272 bytes apart in the tile so that the
// accumulator layout's accesses (32 rows at one column) spread over the banks.
constexpr int kStageRowBytes = 272;
constexpr int kStageBytes = 32 * kStageRowBytes;       // per wavefront

template <typename T>
__device__ __forceinline__ void merge_rows_through_lds(unsigned char* stage, T* o_rows, const int64_t o_pitch,
                                                       float* lse_rows, const f32x16_t (&o_acc)[4], const float inv_l,
                                                       const float lse2, const bool is_first, const int lane) {
    typedef T vec4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) vec4_t* lds_vec4_ptr;
    const int r = lane & 31, half = lane >> 5;
    const lds_vec4_ptr tile = (lds_vec4_ptr)(__attribute__((address_space(3))) void*)stage;
    // element offsets in units of 8 bytes
    auto by_row_pair = [&](const int k) { return ((2 * k + half) * kStageRowBytes >> 3) + r; };
    auto by_accumulator = [&](const int i, const int g) { return (r * kStageRowBytes >> 3) + 8 * i + 2 * g + half; };
    T* const mine = o_rows + (int64_t)half * o_pitch + 4 * r;      // instruction k: + 2 * k * o_pitch

    float w_old = 0.f, w_new = 1.f, lse_out = lse2;
    vec4_t old[4][4];
    if (!is_first) {
        vec4_t in[16];
        const float m_old = load_f32_coherent(lse_rows + r);
#pragma unroll
        for (int k = 0; k < 16; ++k) in[k] = load8_coherent<vec4_t>(mine + 2 * k * o_pitch);
#pragma unroll
        for (int k = 0; k < 16; ++k) tile[by_row_pair(k)] = in[k];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) old[i][g] = tile[by_accumulator(i, g)];
        const float delta = m_old - lse2;
        const float mmax = fmaxf(m_old, lse2);
        lse_out = mmax + fast_log2(1.0f + fast_exp2(-fabsf(delta)));
        w_old = fast_exp2(m_old - lse_out);
        w_new = fast_exp2(lse2 - lse_out);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float x[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) x[c] = o_acc[i][4 * g + c] * inv_l * w_new;
            if (!is_first) {
#pragma unroll
                for (int c = 0; c < 4; ++c) x[c] += (float)old[i][g][c] * w_old;
            }
            vec4_t out;
#pragma unroll
            for (int c = 0; c < 4; ++c) out[c] = (T)x[c];
            tile[by_accumulator(i, g)] = out;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int k = 0; k < 16; ++k) store8_through(mine + 2 * k * o_pitch, (vec4_t)tile[by_row_pair(k)]);
    if (half == 0) store_f32_through(lse_rows + r, lse_out);
}

// The same merge for the paired kernel, whose accumulators come from 16 x 16 products: a lane owns, of the q rows
// 16 b + l % 16 (b = 0, 1), the columns 16 t + 4 (l / 16) .. + 4 (t = 0..7) - again 8-byte pieces, which pass through
// the same tile in LDS to and from whole rows in memory.
template <typename T>
__device__ __forceinline__ void merge_rows16_through_lds(unsigned char* stage, T* o_rows, const int64_t o_pitch,
                                                         float* lse_rows, const f32x4_t (&o_acc)[8][2],
                                                         const float (&inv_l)[2], const float (&lse2)[2],
                                                         const bool is_first, const int lane) {
    typedef T vec4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) vec4_t* lds_vec4_ptr;
    const int r = lane & 31, half = lane >> 5, c16 = lane & 15, g = lane >> 4;
    const lds_vec4_ptr tile = (lds_vec4_ptr)(__attribute__((address_space(3))) void*)stage;
    // element offsets in units of 8 bytes
    auto by_row_pair = [&](const int k) { return ((2 * k + half) * kStageRowBytes >> 3) + r; };
    auto by_accumulator = [&](const int t, const int b) { return ((16 * b + c16) * kStageRowBytes >> 3) + 4 * t + g; };
    T* const mine = o_rows + (int64_t)half * o_pitch + 4 * r;      // instruction k: + 2 * k * o_pitch

    float w_old[2] = {0.f, 0.f}, w_new[2] = {1.f, 1.f}, lse_out[2] = {lse2[0], lse2[1]};
    vec4_t old[8][2];
    if (!is_first) {
        vec4_t in[16];
        float m_old[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) m_old[b] = load_f32_coherent(lse_rows + 16 * b + c16);
#pragma unroll
        for (int k = 0; k < 16; ++k) in[k] = load8_coherent<vec4_t>(mine + 2 * k * o_pitch);
#pragma unroll
        for (int k = 0; k < 16; ++k) tile[by_row_pair(k)] = in[k];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int b = 0; b < 2; ++b) old[t][b] = tile[by_accumulator(t, b)];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const float delta = m_old[b] - lse2[b];
            const float mmax = fmaxf(m_old[b], lse2[b]);
            lse_out[b] = mmax + fast_log2(1.0f + fast_exp2(-fabsf(delta)));
            w_old[b] = fast_exp2(m_old[b] - lse_out[b]);
            w_new[b] = fast_exp2(lse2[b] - lse_out[b]);
        }
    }
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            float x[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) x[c] = o_acc[t][b][c] * inv_l[b] * w_new[b];
            if (!is_first) {
#pragma unroll
                for (int c = 0; c < 4; ++c) x[c] += (float)old[t][b][c] * w_old[b];
            }
            vec4_t out;
#pragma unroll
            for (int c = 0; c < 4; ++c) out[c] = (T)x[c];
            tile[by_accumulator(t, b)] = out;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int k = 0; k < 16; ++k) store8_through(mine + 2 * k * o_pitch, (vec4_t)tile[by_row_pair(k)]);
    if (g == 0) {
#pragma unroll
        for (int b = 0; b < 2; ++b) store_f32_through(lse_rows + 16 * b + c16, lse_out[b]);
    }
}


typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;

// s_waitcnt immediate (gfx9 encoding): at most `vm` vector-memory operations outstanding
constexpr int attn_vmcnt(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

// The wave a tile id falls into: the first w with cum_wave_sizes[w] / block > tile_id (the reference walks
// the prefix sums one by one, template.py:39-44).  The prefix sums rise over the real waves and zero rows
// may pad the table's end, so that index is the number of real waves at or below the tile: sixty-four
// of them are looked at per load, one per lane, instead of one per trip to memory.  Wavefront-uniform;
// num_waves if the tile lies beyond the table.
__device__ __forceinline__ int find_wave(const int32_t* __restrict__ cum_wave_sizes, int num_waves, int block, int tile_id,
                                         int lane) {
    int w = 0;
    for (int base = 0; base < num_waves; base += 64) {
        const int idx = base + lane;
        const int cum = idx < num_waves ? cum_wave_sizes[idx] : 0;
        const unsigned long long below = __builtin_amdgcn_ballot_w64(cum != 0 && cum / block <= tile_id);
        w += __builtin_popcountll(below);
        if (below != ~0ull) break;
    }
    if (w < num_waves && cum_wave_sizes[w] == 0) w = num_waves;        // only padding is left
    return w;
}

// One kv block (128 rows of 256 bytes, `pitch` bytes apart in HBM) into LDS.  Wavefront `wave`
// issues 1 KB fills number wave, wave + 4, ... (4 rows each); lane l lands at byte 16*l of the
// fill, i.e. row l/16, physical 16-byte chunk l%16, and `lane_off` (row l/16 at the pitch, plus
// the logical chunk that lives there) makes it fetch the right 16 bytes.
__device__ __forceinline__ void dma_kv_block(unsigned char* lds, const unsigned char* src, size_t pitch,
                                             unsigned lane_off, int wave) {
#pragma unroll
    for (int i = 0; i < kFills; ++i) {
        const int blk = i * 4 + wave;
        __builtin_amdgcn_global_load_lds((global_void_ptr)(src + (size_t)(blk * 4) * pitch + lane_off),
                                         (lds_void_ptr)(lds + blk * 1024), 16, 0, 0);
    }
}

// LDS layouts (row = kv position in the block, 16 chunks of 16 bytes per row):
//   K: logical chunk c of row r at physical chunk c ^ (r & 15)        (128-bit row reads of
//      32 consecutive rows at one logical chunk hit 16 distinct chunks twice: conflict free)
//   V: logical chunk c of row r at physical chunk c ^ ((r & 3) << 2)  (a transposing read
//      touches 4 consecutive rows x 64 bytes: the 4 rows land in 4 distinct 64-byte granules)
//
// ds_read_b64_tr_b16: in every group of 16 lanes, lane i supplies the address of 4 consecutive
// 16-bit elements M[i][0..3] and receives M[4e + i/4][i%4] for e = 0..3.  With lane i pointing
// at V[kv + i/4][d0 + 4*(i%4) ...] it gets V[kv + 0..3][d0 + i]: four kv values of its own
// column - half of an MFMA A-operand fragment of V^T.

template <typename T>
__global__ void __launch_bounds__(kAttnThreads, 2) attn_fwd_kernel(const AttnParams p) {
    typedef typename AttnMfma<T>::frag_t frag_t;
    typedef T vec4_t __attribute__((ext_vector_type(4)));

    __shared__ __attribute__((aligned(1024))) unsigned char k_lds[kBlockBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char v_lds[kBlockBytes];
    __shared__ int s_abort;
    __shared__ int s_spun;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31;
    const int half = lane >> 5;

    if (tid == 0) s_abort = 0;
    __syncthreads();

    // fills: lane l covers row l/16 of its 4-row group; rows of fill `blk` are 4*blk + l/16 and
    // blk % 4 == wave, so (row & 15) == 4*wave + l/16 and (row & 3) == l/16
    const int f_row = lane >> 4, f_c = lane & 15;
    const size_t k_pitch = (size_t)p.k_st[2] * sizeof(T), v_pitch = (size_t)p.v_st[2] * sizeof(T);
    const unsigned k_fill_off = (unsigned)(f_row * k_pitch + ((f_c ^ (4 * wave + f_row)) << 4));
    const unsigned v_fill_off = (unsigned)(f_row * v_pitch + ((f_c ^ (f_row << 2)) << 4));
    // K fragment reads: row 32*j + r, logical chunk 2*ks + half
    const int k_rd = r * kRowBytes;
    // V^T fragment reads: 16-lane group g = lane/16: d0 = 16*(g & 1), kv offset 4*half (+8 for
    // the upper half of the fragment); lane i of the group: row +i/4, columns d0 + 4*(i%4)
    const int i16 = lane & 15;
    const int v_row = 4 * half + (i16 >> 2);                       // & 3 == i16 >> 2
    const int v_col_bytes = (16 * ((lane >> 4) & 1) + 4 * (i16 & 3)) * 2;    // 0..63
    // physical offset of (row v_row + 16*t2 [+8], d tile i): chunk (4*i + v_col_bytes/16) ^ ((row&3)<<2)
    const int v_swz = (i16 >> 2) << 2;
    int v_rd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        v_rd[i] = v_row * kRowBytes + ((((4 * i + (v_col_bytes >> 4)) ^ v_swz) << 4) | (v_col_bytes & 15));

    int k_chunk[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) k_chunk[ks] = ((2 * ks + half) ^ (r & 15)) << 4;

    const T* __restrict__ Q = reinterpret_cast<const T*>(p.q);
    const unsigned char* __restrict__ K = reinterpret_cast<const unsigned char*>(p.k);
    const unsigned char* __restrict__ V = reinterpret_cast<const unsigned char*>(p.v);
    T* __restrict__ O = reinterpret_cast<T*>(p.o);

    // Workgroups are dealt to the 8 XCDs in turn.  Consecutive tiles are the q blocks of one head and
    // read the same K and V: with the remap an XCD's workgroups take consecutive tiles, so a head's
    // K and V pass through one L2 instead of eight.
    const int first_tile = logical_program_id((int)blockIdx.x, (int)gridDim.x, p.xcd_remap != 0);
    for (int tile_id = first_tile; tile_id < p.num_tiles; tile_id += gridDim.x) {
        // ---- tile id -> wave -> (z, h, q block, kv range) ----
        const int w = find_wave(p.cum_wave_sizes, p.num_waves, kBlockM, tile_id, lane);
        if (w >= p.num_waves) return;
        const int prev = w == 0 ? 0 : p.cum_wave_sizes[w - 1] / kBlockM;
        const int t = tile_id - prev;
        const int size_h = p.wave_sizes[w * 4 + 1];
        const int nq = p.wave_sizes[w * 4 + 2] / kBlockM;
        const int nkv = p.wave_sizes[w * 4 + 3] / kBlockN;
        const int z = t / (nq * size_h) + p.wave_offsets[w * 4 + 0];
        const int h = (t / nq) % size_h + p.wave_offsets[w * 4 + 1];
        const int qb = t % nq + p.wave_offsets[w * 4 + 2] / kBlockM;
        const int kv_lo = p.wave_offsets[w * 4 + 3] / kBlockN;
        const int kv_hi = kv_lo + nkv;
        const int sig = p.signal_offsets[w];

        if (p.visit_log != nullptr && tid == 0) {
            int4* rec = reinterpret_cast<int4*>(p.visit_log) + 2 * (size_t)tile_id;
            rec[0] = make_int4(w, z, h, qb);
            rec[1] = make_int4(kv_lo, kv_hi, sig, (int)blockIdx.x);
        }

        // producer form (generated epilogue, transform/transformer.py:880-901): count the tile in
        // its wave; the tile that completes the wave (all z, h and q blocks of it: the kv range is
        // not counted) publishes the wave's flag.  Called by one thread, behind the tile's stores.
        auto count_tile = [&]() {
            if (p.counters != nullptr && sig >= 0) {
                const int wave_tiles = p.wave_sizes[w * 4 + 0] * size_h * nq;
                const int done = __hip_atomic_fetch_add(p.counters + w, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                if (done == wave_tiles - 1)
                    __hip_atomic_store(p.flags + sig, 1ull, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        };

        // causal: kv blocks strictly above the diagonal contribute nothing; a tile that lies wholly
        // above it has no output of its own but still counts towards its wave
        const int kv_end = p.causal ? min(kv_hi, qb + 1) : kv_hi;
        if (kv_lo >= kv_end) {
            if (tid == 0) count_tile();
            continue;
        }

        // producer form (counters given): the wave's flag is one this kernel SETS; it waits only if a
        // second flag array says what for (a kernel that consumes one exchange and feeds another)
        const int wait_sig = p.wait_offsets != nullptr ? p.wait_offsets[w] : (p.counters == nullptr ? sig : -1);
        if (wait_sig >= 0) {
            if (tid == 0) {
                const uint64_t* wait_flags = p.wait_flags != nullptr ? p.wait_flags : p.flags;
                s_spun = __hip_atomic_load(wait_flags + wait_sig, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 1ull;
                if (s_spun && !spin_until_equal(wait_flags + wait_sig, 1ull, p.timeout_ticks)) {
                    report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, w, (int)blockIdx.x, wait_sig);
                    s_abort = 1;
                }
            }
            __syncthreads();
            // Nothing reads a chunk's lines before its flag is up, so this XCD's L2 cannot hold a stale one
            // (it was emptied when the kernel began); the fence - it drops every clean line of the L2, the K
            // and V blocks other workgroups are about to reuse among them - is kept for the workgroup that
            // really had to wait.  (The caller's part: nothing on the device reads a chunk before its flag during
            // the launch and no flag is raised twice; SYN_ATTN_ACQUIRE_ALWAYS otherwise.)
            if (s_spun || p.acquire_always) acquire_fence_agent();
            if (s_abort) return;
        }

        const size_t head = (size_t)z * p.H + h;
        const int q_row = qb * kBlockM + wave * 32 + r;              // this lane's q position
        const T* q_src = Q + z * p.q_st[0] + h * p.q_st[1] + q_row * p.q_st[2] + 8 * half;
        const unsigned char* k_base = K + (z * p.k_st[0] + h * p.k_st[1]) * (int64_t)sizeof(T);
        const unsigned char* v_base = V + (z * p.v_st[0] + h * p.v_st[1]) * (int64_t)sizeof(T);

        // both stages are free here: every wavefront has passed the barrier that ends a tile
        dma_kv_block(k_lds, k_base + (size_t)kv_lo * kBlockN * k_pitch, k_pitch, k_fill_off, wave);

        frag_t qf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const frag_t*>(q_src + 16 * ks);

        f32x16_t o_acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.f;
        float m_i = -INFINITY;
        float l_i = 0.f;     // this lane's share of the row sum (its 64 of every 128 kv columns)
        // the Q loads must not be counted among the fills below
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::"v"(qf[0]), "v"(qf[1]), "v"(qf[2]), "v"(qf[3]), "v"(qf[4]), "v"(qf[5]), "v"(qf[6]), "v"(qf[7]));

        // one kv block; MASK: the causal diagonal block (kv positions beyond a q row are masked)
        auto kv_block = [&](const int n, auto mask_tag) {
            constexpr bool MASK = decltype(mask_tag)::value;
            // ---- K block n has landed (nothing newer is in flight: V block n is fetched below) ----
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);

            // ---- S^T = K . Q^T : 4 tiles of [32 kv, 32 q]; fragments of step ks+1 are read
            //      while step ks is multiplied ----
            // The fills of V block n are issued one per k16 step between the MFMAs: a wavefront issues in
            // order, and eight 1 KB fills in a row would hold it at the vector-memory queue.
            f32x16_t s[4];
            {
                dma_kv_block(v_lds, v_base + (size_t)n * kBlockN * v_pitch, v_pitch, v_fill_off, wave);
                const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                frag_t kf[2][4];
                const unsigned char* k_row = k_lds + k_rd;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    kf[0][j] = *reinterpret_cast<const frag_t*>(k_row + 32 * j * kRowBytes + k_chunk[0]);
                __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);     // the four reads of step 0 go first
#pragma unroll
                for (int ks = 0; ks < 8; ++ks) {
                    if (ks < 7) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            kf[(ks + 1) & 1][j] = *reinterpret_cast<const frag_t*>(
                                k_row + 32 * j * kRowBytes + k_chunk[ks + 1]);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        s[j] = AttnMfma<T>::run(kf[ks & 1][j], qf[ks], ks == 0 ? zero : s[j]);
                    if (ks < 7) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        }
                    } else {
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                }
            }

            // ---- every wavefront is done with K: the next K block is fetched inside the softmax ----
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): own LDS reads have returned
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);

            // ---- online softmax in base 2 ----
            if constexpr (MASK) {
                const int lim = q_row - n * kBlockN - 4 * half;     // mask where 32j + 8(e/4) + e%4 > lim
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        if (32 * j + 8 * (e >> 2) + (e & 3) > lim) s[j][e] = -INFINITY;
            }
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[j][e]);
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_i, mx * p.qk_scale);
            const float alpha = fast_exp2(m_i - m_new);
            // rescale O only when some row's maximum moved (wavefront-uniform test)
            if (__builtin_amdgcn_ballot_w64(m_new != m_i) != 0) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;
            }
            // the exponentials, with the eight fills of K block n+1 spread between them
            __builtin_amdgcn_sched_barrier(0);
            dma_kv_block(k_lds, k_base + (size_t)min(n + 1, kv_end - 1) * kBlockN * k_pitch, k_pitch, k_fill_off, wave);
            float row_sum = 0.f;
            frag_t pf[8];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float pe = fast_exp2(s[j][e] * p.qk_scale - m_new);
                    row_sum += pe;
                    // S^T rows 8g+4*half+0..3 (g = e/4): elements 8*(t%2)..+7 of tile t/2 are
                    // the kv indices 16t + 8*(i/4) + 4*half + i%4 that step t contracts over
                    pf[2 * j + (e >> 3)][e & 7] = (T)pe;
                }
#pragma unroll
            for (int f = 0; f < kFills; ++f) {
                __builtin_amdgcn_sched_group_barrier(0x400, 8, 0);      // 8 of the 64 exponentials
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            }
            l_i = l_i * alpha + row_sum;
            m_i = m_new;

            // ---- V block n has landed (only the next K block's fills are newer) ----
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(attn_vmcnt(kFills));
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);

            // ---- O^T += V^T . P^T; the fragments of step t2+1 are read while step t2 is multiplied ----
            {
                typedef short s16x8_t __attribute__((ext_vector_type(8)));
                s16x4_t vlo[2][4], vhi[2][4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    vlo[0][i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(v_lds + v_rd[i]));
                    vhi[0][i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(v_lds + v_rd[i] + 8 * kRowBytes));
                }
                __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);     // the eight reads of step 0 go first
#pragma unroll
                for (int t2 = 0; t2 < 8; ++t2) {
                    if (t2 < 7) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const unsigned char* src = v_lds + 16 * (t2 + 1) * kRowBytes + v_rd[i];
                            vlo[(t2 + 1) & 1][i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)src);
                            vhi[(t2 + 1) & 1][i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src + 8 * kRowBytes));
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const s16x4_t lo = vlo[t2 & 1][i], hi = vhi[t2 & 1][i];
                        const s16x8_t both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        o_acc[i] = AttnMfma<T>::run(__builtin_bit_cast(frag_t, both), pf[t2], o_acc[i]);
                    }
                    if (t2 < 7) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                        }
                    } else {
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                    }
                }
            }

            // ---- every wavefront is done with V: the next V block is fetched inside the next S^T ----
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };
        // under a causal mask the diagonal block, if this tile reaches it, is the last one
        const bool diagonal = p.causal && kv_end - 1 == qb;
        const int plain_end = diagonal ? kv_end - 1 : kv_end;
        for (int n = kv_lo; n < plain_end; ++n) kv_block(n, std::false_type{});
        if (diagonal) kv_block(qb, std::true_type{});
        // the re-fetches of the last block land before anything refills the stages or exits
        __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        // ---- epilogue: lse2 = m + log2(l), O = acc / l (template.py:307-309) ----
        const float l_tot = l_i + __shfl_xor(l_i, 32);
        const float lse2 = m_i + fast_log2(l_tot);
        const float inv_l = 1.0f / l_tot;

        const int lock_idx = (int)(head * (p.Sq / kBlockM)) + qb;
        if (tid == 0) {
            const uint64_t t0 = wall_clock64();
            bool ok = true;
            while (atomicCAS(p.lock + lock_idx, 0, 1) != 0) {
                __builtin_amdgcn_s_sleep(4);
                if ((int64_t)(wall_clock64() - t0) > p.timeout_ticks) { ok = false; break; }
            }
            if (!ok) {
                report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, w, (int)blockIdx.x, -2);
                s_abort = 1;
            }
            lock_taken_fence();
        }
        __syncthreads();
        if (s_abort) return;

        const bool is_first = __hip_atomic_load(p.first + lock_idx, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT) == 0;
        // (the K and V blocks are free: every wavefront is past its last block and the barrier above)
        merge_rows_through_lds<T>(wave < 3 ? k_lds + wave * kStageBytes : v_lds,
                                  O + z * p.o_st[0] + h * p.o_st[1] + (int64_t)(qb * kBlockM + wave * 32) * p.o_st[2], p.o_st[2],
                                  p.lse + head * p.Sq + qb * kBlockM + wave * 32, o_acc, inv_l, lse2, is_first, lane);

        // every lane's stores have been acknowledged by memory; then the barrier; then the hand-over
        __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));
        __syncthreads();
        if (tid == 0) {
            lock_release_fence();
            __hip_atomic_store(p.first + lock_idx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));
            lock_release_fence();
            __hip_atomic_store(p.lock + lock_idx, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            count_tile();
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Two q blocks per workgroup, in opposite phases.
//
// A kv block costs a wavefront about as many cycles on the vector ALU (the softmax: 64 scores per
// lane, one quarter-rate exponential each) as on the matrix pipe (128 MFMAs of 16 x 16 x 32), and two
// independent workgroups on a compute unit drift into step, so that both pipes idle half of the time.  Here
// one workgroup of eight wavefronts holds two q blocks that read the same kv range - group 0
// (wavefronts 0-3) tile 2i, group 1 (wavefronts 4-7) tile 2i + 1 - and runs them one slot apart:
//
//   slot         0      1      2          3          4          ...   2N         2N+1
//   group 0      S0     sm0    PV0,S1     sm1        PV1,S2           PV(N-1)    -
//   group 1      -      S0     sm0        PV0,S1     sm1              sm(N-1)    PV(N-1)
//
// so in every slot the two wavefronts of a SIMD use different pipes.  Both groups read K and V
// from the same LDS blocks (half the fills per q row); K and V are double buffered: K(n+1) is
// fetched in slot 2n and V(n) in slot 2n+1, each by the group that is in its softmax, into the buffers
// whose last readers (K(n-1), V(n-2)) finished in slot 2n-1, and have landed by the end of slot 2n+1.
// One barrier per slot, i.e. two per kv block and wavefront instead of four.
//
// The products are 16 x 16 x 32 MFMAs (a wavefront's 32 q rows as two halves of 16 that share every K and V
// fragment).  With 32 x 32 x 16 products - the same flop, the same LDS reads, a third fewer vector instructions
// around them - the board ran this kernel at its power limit, 1.75 to 2.2 GHz instead of 2.4; the narrower
// form draws less per flop, the clock stays at 2.4 GHz, and the launch is 2 to 6 % shorter although it takes
// more cycles.
// ---------------------------------------------------------------------------------------------
constexpr int kPairThreads = 512;
constexpr int kPairFills = kBlockBytes / 1024 / 8;      // 4 fills of 1 KB per wavefront and block

// A fill of the paired kernel: 16 bytes per lane from `src` to LDS at `lds` + 16 * lane, written as assembly so that
// the COMPILER DOES NOT KNOW OF IT.  Told of a load into LDS (the builtin), it makes every later LDS read wait for
// it, s_waitcnt vmcnt(0) - it cannot tell that the read is of another buffer - and the wavefronts whose products
// follow their fills stood still until their own fills had crossed the memory system: the slots with fills took
// 5400 cycles, the others 2800.  What has to wait for a fill does so in the kernel's own s_waitcnt vmcnt(0): before
// the barrier that ends an odd slot, and before the first products of a segment.  (Untold loads in flight make the
// compiler's own vmcnt counts for its loads and stores wait for more than they need, never for less: the counter
// retires in order.)
__device__ __forceinline__ void fill16_untold(const unsigned char* src, const unsigned char* lds) {
    const unsigned lds_addr = (unsigned)(uintptr_t)(lds_void_ptr)lds;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "m0");
}

__device__ __forceinline__ void dma_kv_block8(unsigned char* lds, const unsigned char* src, size_t pitch,
                                              unsigned lane_off, int wave8) {
#pragma unroll
    for (int i = 0; i < kPairFills; ++i) {
        const int blk = i * 8 + wave8;                  // blk % 4 == wave8 % 4: the swizzle of the 4-wave form holds
        fill16_untold(src + (size_t)(blk * 4) * pitch + lane_off, lds + blk * 1024);
    }
}

// The same block by four wavefronts (`wave` = 0..3): fills wave, wave + 4, ...
__device__ __forceinline__ void dma_kv_block4(unsigned char* lds, const unsigned char* src, size_t pitch,
                                              unsigned lane_off, int wave) {
#pragma unroll
    for (int i = 0; i < 2 * kPairFills; ++i) {
        const int blk = i * 4 + wave;
        fill16_untold(src + (size_t)(blk * 4) * pitch + lane_off, lds + blk * 1024);
    }
}

// A V block of the paired kernel in LDS: the fills (4 rows of 256 bytes each) with an even number lie one after the
// other, those with an odd number likewise, 16 KB + 128 bytes further on - so rows 4..7 of every eight sit half a row
// (32 banks) askew of rows 0..3, which an exclusive-or of the column could only do at the price of a per-lane address
// for every 16 columns (see the kernel's note on its layouts).
constexpr int kPairVOddFills = kBlockBytes / 2 + 128;
constexpr int kPairVBlockBytes = kBlockBytes + 1024;
__device__ __forceinline__ void dma_v_block4(unsigned char* lds, const unsigned char* src, size_t pitch,
                                             unsigned lane_off, int wave) {
#pragma unroll
    for (int i = 0; i < 2 * kPairFills; ++i) {
        const int blk = i * 4 + wave;
        fill16_untold(src + (size_t)(blk * 4) * pitch + lane_off, lds + (blk >> 1) * 1024 + (wave & 1) * kPairVOddFills);
    }
}

//
// The visits of a program come in SEGMENTS: one or more visits to the same pair of q blocks, walked as one run of
// kv blocks with the running maxima, sums and output in registers, and written (or merged) once, at the end.
//   kPairTiles       a segment is one visit; pair b, b + grid, ... of the table; merged under the q blocks' locks.
//   kPairChainWaves  (SYN_ATTN_CHAIN_Q_BLOCKS) every wave lists the same (z, h, q) ranges and there are as many
//                    programs as a wave has pairs: program b's segment is pair b of wave 0, of wave 1, ...; each
//                    wave's kv range behind that wave's flag; the q blocks are written once, without locks.
//   kPairWorkList    (SYN_ATTN_WORK_LIST) the caller's list says which visits a program makes, in which order, which
//                    of them continue a segment, and whether a segment is the only one that writes its q blocks.
// CAUSAL: kv blocks above a q block's diagonal contribute nothing - a visit ends at the diagonal of its higher q
// block, the lower q block sits the last block out, and each masks its own diagonal block.
constexpr int kPairTiles = 0, kPairChainWaves = 1, kPairWorkList = 2;
constexpr int32_t kWorkPairMask = SYN_ATTN_WORK_PAIR_MASK;
constexpr int kPairLdsWaves = 256, kPairLdsEntries = 512;

template <typename T, int MODE, bool CAUSAL>
__global__ void __launch_bounds__(kPairThreads, 1) attn_pair_kernel(const AttnParams p) {
    typedef typename AttnMfma<T>::frag_t frag_t;
    typedef T vec4_t __attribute__((ext_vector_type(4)));
    static_assert(!(CAUSAL && MODE == kPairChainWaves), "the waves of a causal table do not share their kv extent");

    __shared__ __attribute__((aligned(1024))) unsigned char k_lds[2 * kBlockBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char v_lds[2 * kPairVBlockBytes];
    __shared__ int s_abort;
    __shared__ int s_spun;
    // the head of the wave table and of this program's list, read once: what a visit is (a search over the prefix
    // sums, then a row of the table) is looked up at every change of visit, where all eight wavefronts wait for it -
    // from LDS that takes a tenth of a trip to memory
    __shared__ int s_cum[kPairLdsWaves];             // tiles up to and including the wave (0: padding)
    __shared__ int s_row[kPairLdsWaves][8];          // size_h, q blocks, first z, first h, first q block, kv_lo, kv blocks, signal
    __shared__ int s_entries[kPairLdsEntries];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave8 >> 2;          // which of the two q blocks
    const int wave = wave8 & 3;          // 32-row slice of the q block
    const int c16 = lane & 15;           // the lane's column of a 16 x 16 MFMA tile: q rows c16 and 16 + c16 of the slice
    const int g = lane >> 4;             // the lane's group of four rows of a tile / its eight k of an operand

    if (tid == 0) s_abort = 0;
    for (int w = tid; w < min(p.num_waves, kPairLdsWaves); w += kPairThreads) {
        s_cum[w] = p.cum_wave_sizes[w] / kBlockM;
        s_row[w][0] = p.wave_sizes[w * 4 + 1];
        s_row[w][1] = p.wave_sizes[w * 4 + 2] / kBlockM;
        s_row[w][2] = p.wave_offsets[w * 4 + 0];
        s_row[w][3] = p.wave_offsets[w * 4 + 1];
        s_row[w][4] = p.wave_offsets[w * 4 + 2] / kBlockM;
        s_row[w][5] = p.wave_offsets[w * 4 + 3] / kBlockN;
        s_row[w][6] = p.wave_sizes[w * 4 + 3] / kBlockN;
        s_row[w][7] = p.signal_offsets[w];
    }

    // LDS layouts of this kernel (row = kv position in the block, 16 chunks of 16 bytes per row):
    //   K: logical chunk c of row r at physical chunk c ^ (r & 15): a 16-byte read per lane of the rows 16 a + l % 16
    //      at the chunk 4 ks + l / 16 - an A operand of S^T = K . Q^T - finds 16 distinct chunks per 16 lanes.
    //   V: logical chunk c of row r at physical chunk c ^ ((r & 3) << 1), and the fills with an odd number (rows 4..7
    //      of every eight) half a row askew, see dma_v_block4.  A transposing read touches, per 32 lanes, 8 rows x 32
    //      bytes (rows 4 g + i / 4 for two values of g): rows 0..3 land in the four 32-byte granules of one half of
    //      the 64 banks, rows 4..7 in the other half.  The 16 columns a read is for enter the address as 32 t: the
    //      exclusive-or moves bits 5 and 6 only, so t / 4 is an offset in the instruction and a lane carries four
    //      addresses.  (With the exclusive-or over all three bits, c ^ ((r & 7) << 1), the layout needs no askew
    //      half - and eight addresses per lane, or two instructions per read to make them: both were measured,
    //      the one spills registers, the other costs 40 % more vector instructions than the whole softmax.)
    // A fill of 1 KB is 4 rows; wavefront wave8 issues fills wave8, wave8 + 8, ...: row = 4 blk + l / 16 with
    // blk % 4 == wave8 % 4, so both swizzles are per-wavefront constants on the fill side.
    const int f_row = lane >> 4, f_c = lane & 15;
    const size_t k_pitch = (size_t)p.k_st[2] * sizeof(T), v_pitch = (size_t)p.v_st[2] * sizeof(T);
    const unsigned k_fill_off = (unsigned)(f_row * k_pitch + ((f_c ^ (4 * wave + f_row)) << 4));
    const unsigned v_fill_off = (unsigned)(f_row * v_pitch + ((f_c ^ (f_row << 1)) << 4));
    // K fragment of kv tile a, k step ks: row 16 a + c16, logical chunk 4 ks + g = 4 ks ^ g, physical (4 ks) ^ (g ^ c16)
    const int k_rd = c16 * kRowBytes;
    const int k_swz = (g ^ c16) << 4;
    // V^T fragment of d tile t, kv step u: lane i of its 16 points at V[32 u + 4 g + i / 4][16 t + 4 (i % 4) ..] and
    // receives V[32 u + 4 g + 0..3][16 t + i]; a second read 16 rows further down gives the other four k of the
    // operand.  Row 32 u + 4 g + i / 4 is row i / 4 of fill 8 u + g: at 4096 u + 1024 (g / 2), askew if g is odd.
    // v_rd[t % 4] + 128 (t / 4) + 4096 u (+ 2048 for the second read) is the address in the block.
    int v_rd[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
        v_rd[t] = (g >> 1) * 1024 + (g & 1) * kPairVOddFills + (c16 >> 2) * kRowBytes +
                  (((2 * t + ((c16 & 3) >> 1)) ^ ((c16 >> 2) << 1)) << 4) + 8 * (c16 & 1);

    const T* __restrict__ Q = reinterpret_cast<const T*>(p.q);
    const unsigned char* __restrict__ K = reinterpret_cast<const unsigned char*>(p.k);
    const unsigned char* __restrict__ V = reinterpret_cast<const unsigned char*>(p.v);
    T* __restrict__ O = reinterpret_cast<T*>(p.o);

    const int pairs_per_wave = p.cum_wave_sizes[0] / kBlockM / 2;
    const int num_pairs = MODE == kPairChainWaves ? pairs_per_wave : p.num_tiles / 2;
    if (MODE == kPairChainWaves && (int)gridDim.x != pairs_per_wave) {
        if (tid == 0) report_status(p.status, SYN_STATUS_BAD_CHAIN, 0, (int)blockIdx.x, pairs_per_wave);
        return;
    }
    const int program = logical_program_id((int)blockIdx.x, (int)gridDim.x, p.xcd_remap != 0);

    // where the program stands: the next pair of the table (kPairTiles, kPairChainWaves) or the entry of its list
    int pair = program;
    int e = 0, e_end = 0, e_begin = 0;
    const int32_t* entries = nullptr;
    if constexpr (MODE == kPairWorkList) {
        e = e_begin = __builtin_amdgcn_readfirstlane(p.work_list[program]);
        e_end = __builtin_amdgcn_readfirstlane(p.work_list[program + 1]);
        entries = p.work_list + gridDim.x + 1;
        for (int i = tid; i < min(e_end - e_begin, kPairLdsEntries); i += kPairThreads) s_entries[i] = entries[e_begin + i];
    }
    __syncthreads();
    auto entry_at = [&](const int i) __attribute__((always_inline)) {
        return __builtin_amdgcn_readfirstlane(i - e_begin < kPairLdsEntries ? s_entries[i - e_begin] : entries[i]);
    };
    // what a tile id is: wave, (z, h, q block), kv range in blocks, flag (the lookup of find_wave, on the copy in LDS)
    struct Where {
        int w, z, h, qb, kv_lo, kv_len, sig;
        bool paired;        // an even number of q blocks in the wave, an even number of tiles in front of it
    };
    auto locate = [&](const int tile, Where& at) __attribute__((always_inline)) -> bool {
        int w = 0;
        for (int base = 0; base < p.num_waves; base += 64) {
            const int idx = base + lane;
            const int cum = idx >= p.num_waves ? 0 : (idx < kPairLdsWaves ? s_cum[idx] : p.cum_wave_sizes[idx] / kBlockM);
            const unsigned long long below = __builtin_amdgcn_ballot_w64(cum != 0 && cum <= tile);
            w += __builtin_popcountll(below);
            if (below != ~0ull) break;
        }
        if (w >= p.num_waves) return false;
        int row[8], prev;
        if (w < kPairLdsWaves) {
#pragma unroll
            for (int f = 0; f < 8; ++f) row[f] = __builtin_amdgcn_readfirstlane(s_row[w][f]);
            prev = w == 0 ? 0 : __builtin_amdgcn_readfirstlane(s_cum[w - 1]);
            if (__builtin_amdgcn_readfirstlane(s_cum[w]) == 0) return false;          // only padding is left
        } else {
            row[0] = p.wave_sizes[w * 4 + 1];
            row[1] = p.wave_sizes[w * 4 + 2] / kBlockM;
            row[2] = p.wave_offsets[w * 4 + 0];
            row[3] = p.wave_offsets[w * 4 + 1];
            row[4] = p.wave_offsets[w * 4 + 2] / kBlockM;
            row[5] = p.wave_offsets[w * 4 + 3] / kBlockN;
            row[6] = p.wave_sizes[w * 4 + 3] / kBlockN;
            row[7] = p.signal_offsets[w];
            prev = p.cum_wave_sizes[w - 1] / kBlockM;
            if (p.cum_wave_sizes[w] == 0) return false;
        }
        const int t = tile - prev;
        at.w = w;
        at.z = t / (row[1] * row[0]) + row[2];
        at.h = (t / row[1]) % row[0] + row[3];
        at.qb = t % row[1] + row[4];
        at.kv_lo = row[5];
        at.kv_len = row[6];
        at.sig = row[7];
        at.paired = !(row[1] & 1) && !(prev & 1);
        return true;
    };
    auto advance = [&]() __attribute__((always_inline)) {
        if constexpr (MODE == kPairWorkList) ++e;
        else pair += gridDim.x;
    };
    auto pending = [&]() __attribute__((always_inline)) { return MODE == kPairWorkList ? e < e_end : pair < num_pairs; };

    // wait for flag `sg` of the wave `wv` that is being entered; false when the wait gave up
    // A look ahead at the flag of the visit after the one being entered (thread 0): asked for here, read at the next
    // change of visit, a kv range later.  A flag goes up once per launch, so a 1 seen early still holds then; a 0
    // means nothing and the flag is read again.
    int peeked_sig = -1;
    unsigned long long peeked = 0;
    auto peek_flag = [&](const int sg) __attribute__((always_inline)) {
        peeked_sig = sg;
        if (tid == 0 && sg >= 0) peeked = __hip_atomic_load(p.flags + sg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    auto wait_for_flag = [&](const int sg, const int wv) __attribute__((always_inline)) -> bool {
        if (tid == 0) {
            const bool seen_up = peeked_sig == sg && peeked == 1ull;
            s_spun = !seen_up && __hip_atomic_load(p.flags + sg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 1ull;
            if (s_spun && !spin_until_equal(p.flags + sg, 1ull, p.timeout_ticks)) {
                report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, wv, (int)blockIdx.x, sg);
                s_abort = 1;
            }
        }
        __syncthreads();
        // (both words are the same for every lane: read as scalars, so that what depends on them - whether the
        // walk goes on - stays wavefront-uniform for the compiler too)
        if (__builtin_amdgcn_readfirstlane(s_spun) || p.acquire_always) acquire_fence_agent();       // see attn_fwd_kernel
        const bool ok = __builtin_amdgcn_readfirstlane(s_abort) == 0;
        __syncthreads();       // s_spun may be written again only when everyone has read it
        return ok;
    };

    for (; pending(); advance()) {
        // ---- the segment's first visit: tile id -> wave -> (z, h, q block, kv range); the two tiles of a pair
        //      differ in the q block only ----
        int entry = 0;
        if constexpr (MODE == kPairWorkList) entry = entry_at(e);
        const int pair_id = MODE == kPairWorkList ? (entry & kWorkPairMask) : pair;
        const bool sole_writer = MODE == kPairChainWaves || (MODE == kPairWorkList && (entry & SYN_ATTN_WORK_SOLE_WRITER));
        const int tile_id = 2 * pair_id + grp;
        Where first;
        if (!locate(tile_id, first)) return;
        const int w = first.w, z = first.z, h = first.h, qb = first.qb;
        const int kv_lo = first.kv_lo, kv_len = first.kv_len, sig = first.sig;
        // the caller promised an even number of q blocks per wave (and, under a causal mask, q ranges and kv
        // ranges that begin at even blocks: the lower q block of a pair then never finds its whole visit masked
        // while the higher one has work); leave a note instead of wrong results
        if (!first.paired || (CAUSAL && ((kv_lo | (qb - grp)) & 1))) {
            if (lane == 0 && wave8 == 0) report_status(p.status, SYN_STATUS_BAD_PAIRING, w, (int)blockIdx.x, kv_lo);
            return;
        }

        if (p.visit_log != nullptr && lane == 0 && wave == 0) {
            int4* rec = reinterpret_cast<int4*>(p.visit_log) + 2 * (size_t)tile_id;
            rec[0] = make_int4(w, z, h, qb);
            rec[1] = make_int4(kv_lo, kv_lo + kv_len, sig, (int)blockIdx.x);
        }

        // kv blocks the pair walks in this visit: under a causal mask, up to the diagonal of its higher q block
        const int diag_hi = qb | 1;                     // the higher q block of the pair
        const int nkv = CAUSAL ? min(kv_len, diag_hi + 1 - kv_lo) : kv_len;
        if (CAUSAL && nkv <= 0) continue;               // wholly above the diagonal: visited, nothing to add

        if (sig >= 0 && !wait_for_flag(sig, w)) return;

        const size_t head = (size_t)z * p.H + h;
        const int q_row = qb * kBlockM + wave * 32 + c16;          // and q_row + 16
        const T* q_src = Q + z * p.q_st[0] + h * p.q_st[1] + q_row * p.q_st[2] + 8 * g;
        const unsigned char* const k_head = K + (z * p.k_st[0] + h * p.k_st[1]) * (int64_t)sizeof(T);
        const unsigned char* const v_head = V + (z * p.v_st[0] + h * p.v_st[1]) * (int64_t)sizeof(T);

        // With the XCD remap the workgroups of an XCD work on the q blocks of one or two heads at the
        // same time and read the same K and V: each pair starts its walk over a visit's kv blocks
        // one block after its neighbour's and wraps around, so that they ask the L2 for different
        // lines at any moment while staying within a window of blocks that the L2 holds (the sum
        // over kv blocks is order-free up to rounding).  A visit that reaches a diagonal is walked from its
        // first block: every row's first block then has an unmasked position, and the masked blocks come last.
        auto rotation = [&](const int lo, const int len, const int walked) __attribute__((always_inline)) {
            if (!p.xcd_remap || (CAUSAL && lo + len > (qb & ~1))) return 0;
            return (int)((unsigned)pair_id % (unsigned)walked);
        };
        // what a kv block is to THIS group's q block: how far it lies beyond the block before the diagonal - 0 or less
        // below the diagonal (nothing masked), 1 the diagonal block, 2 the block after it (everything masked)
        auto beyond = [&](const int kv_block) __attribute__((always_inline)) { return kv_block - qb + 1; };

        // ---- the walk: the K fills run one block ahead of the V fills; both step through the visit's blocks
        //      (rotated) and the K walk enters the segment's next visit when its own is used up ----
        int k_lo = kv_lo, k_nkv = nkv, k_next = 1, k_rot = rotation(kv_lo, kv_len, nkv);
        int v_nkv = nkv, v_next = 0, v_rot = k_rot;
        const unsigned char* k_walk = k_head + (size_t)kv_lo * kBlockN * k_pitch;
        const unsigned char* v_walk = v_head + (size_t)kv_lo * kBlockN * v_pitch;
        int k_wave = w;                                  // kPairChainWaves: the wave the K walk is in
        // `beyond` of the blocks whose softmax is still to come: block n (the next one), n + 1 and n + 2
        int m0 = CAUSAL ? beyond(kv_lo + k_rot) : 0, m1 = 0, m2 = 0;
        // (The chained forms without a causal mask keep the masking block of `softmax`, which they never enter, and
        // get their zeros here from behind an opaque statement: with the block in place the register allocator finds
        // the assignment it finds for the causal forms - 237 registers, nothing spilled; without it, 256 and 53
        // registers spilled inside the loop over kv blocks.)
        if constexpr (!CAUSAL && MODE != kPairTiles) {
            asm volatile("s_mov_b32 %0, 0" : "=s"(m0));
            m2 = m0;
        }

        // the flag of the visit that follows the one the K walk has just entered, if the segment goes on
        auto look_ahead = [&]() __attribute__((always_inline)) {
            int next_tile;
            if constexpr (MODE == kPairTiles) {
                return;
            } else if constexpr (MODE == kPairChainWaves) {
                if (k_wave + 1 >= p.num_waves) return;
                next_tile = tile_id + 2 * (k_wave + 1) * pairs_per_wave;
            } else {
                if (!(entry & SYN_ATTN_WORK_CONTINUES) || e + 1 >= e_end) return;
                next_tile = 2 * (entry_at(e + 1) & kWorkPairMask) + grp;
            }
            Where at;
            if (locate(next_tile, at)) peek_flag(at.sig);
        };

        // the K walk enters the segment's next visit: 1 entered, 0 the segment ends here, -1 give up
        auto enter_next_visit = [&]() __attribute__((always_inline)) -> int {
            int next_tile;
            if constexpr (MODE == kPairTiles) {
                return 0;
            } else if constexpr (MODE == kPairChainWaves) {
                if (k_wave + 1 >= p.num_waves || p.cum_wave_sizes[k_wave + 1] == 0) return 0;
                ++k_wave;
                next_tile = tile_id + 2 * k_wave * pairs_per_wave;
            } else {
                if (!(entry & SYN_ATTN_WORK_CONTINUES) || e + 1 >= e_end) return 0;
                ++e;
                entry = entry_at(e);
                next_tile = 2 * (entry & kWorkPairMask) + grp;
            }
            Where at;
            const bool found = locate(next_tile, at);
            const int walked = CAUSAL ? min(at.kv_len, diag_hi + 1 - at.kv_lo) : at.kv_len;
            // the visit has to be to this segment's q blocks (for kPairChainWaves: every wave lists the ranges of
            // wave 0), and under a causal mask a visit with nothing below the diagonal cannot continue a segment
            if (!found || !at.paired || at.z != z || at.h != h || at.qb != qb || (MODE == kPairChainWaves && at.w != k_wave) ||
                (CAUSAL && (walked <= 0 || (at.kv_lo & 1)))) {
                if (tid == 0) report_status(p.status, SYN_STATUS_BAD_CHAIN, found ? at.w : -1, (int)blockIdx.x, next_tile);
                return -1;
            }
            if (p.visit_log != nullptr && lane == 0 && wave == 0) {
                int4* rec = reinterpret_cast<int4*>(p.visit_log) + 2 * (size_t)next_tile;
                rec[0] = make_int4(at.w, z, h, qb);
                rec[1] = make_int4(at.kv_lo, at.kv_lo + at.kv_len, at.sig, (int)blockIdx.x);
            }
            if (at.sig >= 0 && !wait_for_flag(at.sig, at.w)) return -1;
            look_ahead();
            k_lo = at.kv_lo;
            k_nkv = walked;
            k_rot = rotation(at.kv_lo, at.kv_len, walked);
            k_next = 0;
            k_walk = k_head + (size_t)at.kv_lo * kBlockN * k_pitch;
            return 1;
        };
        look_ahead();
        // every wavefront has passed the barrier that ended the previous segment: all four buffers are free
        dma_kv_block8(k_lds, k_walk + (size_t)k_rot * kBlockN * k_pitch, k_pitch, k_fill_off, wave8);

        // Q^T operands of the two 16-row halves of the slice: [b][ks] = Q[q_row + 16 b][32 ks + 8 g .. + 8]
        frag_t qf[2][4];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qf[b][ks] = *reinterpret_cast<const frag_t*>(q_src + 16 * b * p.q_st[2] + 32 * ks);
        // O^T: [t][b] = columns 16 t + 4 g + 0..3 of q row 16 b + c16
        f32x4_t o_acc[8][2];
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int b = 0; b < 2; ++b) o_acc[t][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        float m_i[2] = {-INFINITY, -INFINITY};
        float l_i[2] = {0.f, 0.f};
        // S^T: [a][b] = kv positions 16 a + 4 g + 0..3 of the block against q row 16 b + c16
        f32x4_t s[8][2];
        // P^T operands: [b][u] holds, as k 8 g + x, the kv position 16 (2 u + x / 4) + 4 g + x % 4 - the lane's own
        // probabilities of the tiles 2 u and 2 u + 1; the V^T operand reads its rows in the same order
        frag_t pf[2][4];

        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));       // K block 0 (and Q) have landed
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        // V(m) and K(m+1) are fetched in slots 2m and 2m + 1 and are first read in slot 2m + 2; their buffers were last
        // read in slot 2m - 1.  A wavefront stands still for some 350 cycles at every fill it issues, wherever the fill
        // is placed, so the fills are left to the group that is in its softmax, which has a thousand cycles to spare
        // beside the other group's products: group 1 asks for K(m+1) at the start of slot 2m (in `fetch`), group 0 for
        // V(m) at the start of slot 2m + 1 (`fill_v`), four wavefronts a block.  Every wavefront waits for its own fills
        // before the barrier that ends slot 2m + 1.  (Measured against every wavefront issuing an eighth of both blocks
        // at the start of slot 2m: 1 to 3 % faster.  The softmax before the fills, or the fills spread among the
        // products, or the next blocks touched ahead so that the fills hit in the L2: the same or slower.)
        // `fetch` returns 1 when K(m+1) was asked for, 0 when block m is the segment's last, -1 to give up (a flag did
        // not come within the time limit, or the next visit is not one of this segment's: every wavefront is
        // told so at the same fetch, and the program ends).
        const unsigned char* v_src_pending = nullptr;
        int v_buf_pending = 0;
        auto fill_v = [&]() __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
            dma_v_block4(v_lds + v_buf_pending * kPairVBlockBytes, v_src_pending, v_pitch, v_fill_off, wave);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto fetch = [&](const int m) __attribute__((always_inline)) -> int {
            __builtin_amdgcn_sched_barrier(0);
            // block m is the first of a new visit exactly when the V walk has used its visit up; the K walk
            // entered that visit when it fetched K(m) and has not moved since
            if (v_next == v_nkv) {
                v_nkv = k_nkv;
                v_rot = k_rot;
                v_walk = v_head + (size_t)k_lo * kBlockN * v_pitch;
                v_next = 0;
            }
            int b = v_next + v_rot;
            b = b >= v_nkv ? b - v_nkv : b;
            v_src_pending = v_walk + (size_t)b * kBlockN * v_pitch;       // for group 0's fill_v, one slot on
            v_buf_pending = m & 1;
            ++v_next;
            int more = 1;
            if (k_next == k_nkv) more = enter_next_visit();
            if (more > 0) {
                b = k_next + k_rot;
                b = b >= k_nkv ? b - k_nkv : b;
                if (grp == 1)
                    dma_kv_block4(k_lds + ((m + 1) & 1) * kBlockBytes, k_walk + (size_t)b * kBlockN * k_pitch, k_pitch, k_fill_off, wave);
                ++k_next;
                if constexpr (CAUSAL) m2 = beyond(k_lo + b);
            }
            __builtin_amdgcn_sched_barrier(0);
            return __builtin_amdgcn_readfirstlane(more);       // the same in every lane: a scalar for the compiler too
        };

        constexpr int kG = 4, kPer = 8 / kG, kGroups = 4 * kPer;          // V^T fragments per group of products, groups per step
        constexpr int kGS = 2, kPerS = 8 / kGS, kGroupsS = 4 * kPerS;     // the same for the K fragments of the scores,
        constexpr int kDS = 4;                                            // of which this many groups are in registers
        // S^T = K(n) . Q^T: 8 kv tiles x 4 k steps, each K fragment against the two halves of the q slice.
        // Group u = k step u / kPerS, kv tiles kGS (u % kPerS) .. + kGS.  The fragments of group u and of the
        // next three are in registers; the register a pair of products has just consumed is refilled with the fragment
        // of group u + 4, so a read has almost four groups (256 MFMA cycles) to come back - two groups ahead measured 2
        // to 3 % slower, groups of four tiles two ahead the same as this.  (Asking for the first groups' fragments
        // sixteen products before the end of weighted_values, into registers of used-up probabilities, measured the same.)
        auto scores = [&](const int n) __attribute__((always_inline)) {
            const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
            __builtin_amdgcn_s_setprio(3);       // (the first products of a segment have no weighted_values before them)
            frag_t kf[kDS][kGS];
            const unsigned char* k_row = k_lds + (n & 1) * kBlockBytes + k_rd;
            // (opaque to the compiler, which would otherwise carry the four chunk offsets in registers around the loop
            // over kv blocks - registers this kernel does not have)
            int swz = k_swz;
            asm volatile("" : "+v"(swz));
            auto k_at = [&](const int u, const int j) __attribute__((always_inline)) {
                return k_row + 16 * (kGS * (u % kPerS) + j) * kRowBytes + (swz ^ (64 * (u / kPerS)));
            };
#pragma unroll
            for (int u = 0; u < kDS; ++u)
#pragma unroll
                for (int j = 0; j < kGS; ++j) kf[u][j] = *reinterpret_cast<const frag_t*>(k_at(u, j));
            __builtin_amdgcn_sched_group_barrier(0x100, kDS * kGS, 0);
#pragma unroll
            for (int u = 0; u < kGroupsS; ++u) {
                const int ks = u / kPerS;
#pragma unroll
                for (int j = 0; j < kGS; ++j) {
                    const int a = kGS * (u % kPerS) + j;
#pragma unroll
                    for (int b = 0; b < 2; ++b) s[a][b] = mfma16<T>(kf[u % kDS][j], qf[b][ks], ks == 0 ? zero : s[a][b]);
                    if (u + kDS < kGroupsS) kf[u % kDS][j] = *reinterpret_cast<const frag_t*>(k_at(u + kDS, j));
                }
                if (u + kDS < kGroupsS) {
#pragma unroll
                    for (int j = 0; j < kGS; ++j) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    }
                } else {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2 * kGS, 0);
                }
            }
        };

        // online softmax in base 2 over the scores in s; leaves P^T in pf.  `past` > 0 (CAUSAL): the block reaches
        // the q block's diagonal (1) or lies wholly behind it (2) - positions beyond a row's own are masked.  A row
        // has seen an unmasked position by then (a visit that reaches the diagonal is walked from its first block,
        // which is at or below the lower q block), so its running maximum is finite and a wholly masked block adds
        // exact zeros.
        auto softmax = [&](const int past) __attribute__((always_inline)) {
            __builtin_amdgcn_s_setprio(0);
            if ((CAUSAL || MODE != kPairTiles) && past > 0) {
                // q row wave * 32 + 16 b + c16 against kv position 16 a + 4 g + i of the block
                const int lim = wave * 32 + c16 - 4 * g - (past - 1) * kBlockN;     // mask where 16 a + i > lim + 16 b
#pragma unroll
                for (int a = 0; a < 8; ++a)
#pragma unroll
                    for (int b = 0; b < 2; ++b)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (16 * a + i - 16 * b > lim) s[a][b][i] = -INFINITY;
            }
            float mx[2] = {-INFINITY, -INFINITY};
#pragma unroll
            for (int a = 0; a < 8; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i) mx[b] = fmaxf(mx[b], s[a][b][i]);
            float m_new[2], alpha[2];
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                mx[b] = max_with_lane_xor32(max_with_lane_xor16(mx[b]));
                m_new[b] = fmaxf(m_i[b], mx[b] * p.qk_scale);
                alpha[b] = fast_exp2(m_i[b] - m_new[b]);
            }
            if (__builtin_amdgcn_ballot_w64(m_new[0] != m_i[0] || m_new[1] != m_i[1]) != 0) {
#pragma unroll
                for (int t = 0; t < 8; ++t)
#pragma unroll
                    for (int b = 0; b < 2; ++b)
#pragma unroll
                        for (int i = 0; i < 4; ++i) o_acc[t][b][i] *= alpha[b];
            }
            float row_sum[2] = {0.f, 0.f};
#pragma unroll
            for (int a = 0; a < 8; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float pe = fast_exp2(s[a][b][i] * p.qk_scale - m_new[b]);
                        row_sum[b] += pe;
                        pf[b][a >> 1][4 * (a & 1) + i] = (T)pe;
                    }
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                l_i[b] = l_i[b] * alpha[b] + row_sum[b];
                m_i[b] = m_new[b];
            }
        };

        // O^T += V(n)^T . P^T: 8 d tiles x 4 kv steps of 32, each V^T fragment against the two halves of the q slice
        // A wavefront in its products asks to be issued before the other wavefront of its SIMD, which is in its softmax
        // (s_setprio 3 here and in `scores`, 0 in `softmax`): the matrix pipe is the one that must not wait.  1.5 to
        // 3 % on the all-to-all tables, which run at the full clock; nothing on the all-gather table, which the board's
        // power limit bounds.
        auto weighted_values = [&](const int n) __attribute__((always_inline)) {
            typedef short s16x8_t __attribute__((ext_vector_type(8)));
            __builtin_amdgcn_s_setprio(3);
            const unsigned char* v_blk = v_lds + (n & 1) * kPairVBlockBytes;
            // group w = kv step w / kPer, d tiles kG (w % kPer) .. + kG
            auto v_at = [&](const int w, const int j) __attribute__((always_inline)) {
                const int t = kG * (w % kPer) + j;
                return v_blk + 4096 * (w / kPer) + 128 * (t >> 2) + v_rd[t & 3];
            };
            s16x4_t vlo[2][kG], vhi[2][kG];
#pragma unroll
            for (int w = 0; w < 2; ++w)
#pragma unroll
                for (int j = 0; j < kG; ++j) {
                    const unsigned char* src = v_at(w, j);
                    vlo[w][j] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)src);
                    vhi[w][j] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src + 2048));
                }
            __builtin_amdgcn_sched_group_barrier(0x100, 4 * kG, 0);
#pragma unroll
            for (int w = 0; w < kGroups; ++w) {
                const int u = w / kPer;
#pragma unroll
                for (int j = 0; j < kG; ++j) {
                    const int t = kG * (w % kPer) + j;
                    const s16x4_t lo = vlo[w & 1][j], hi = vhi[w & 1][j];
                    const s16x8_t both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
                    for (int b = 0; b < 2; ++b)
                        o_acc[t][b] = mfma16<T>(__builtin_bit_cast(frag_t, both), pf[b][u], o_acc[t][b]);
                    if (w + 2 < kGroups) {
                        const unsigned char* src = v_at(w + 2, j);
                        vlo[w & 1][j] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)src);
                        vhi[w & 1][j] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(src + 2048));
                    }
                }
                if (w + 2 < kGroups) {
#pragma unroll
                    for (int j = 0; j < kG; ++j) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    }
                } else {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2 * kG, 0);
                }
            }
        };

        // a slot ends when every wavefront's LDS reads have returned; at the end of an odd slot the
        // blocks fetched one slot earlier have landed as well
        auto end_even = [&]() __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xc07f);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };
        auto end_odd = [&]() __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0x0070);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };

        // the two groups run the same phases one slot apart; written out per group so that the scores
        // (group 0) or the probabilities (group 1) are the only block-sized values that live across
        // an iteration.  `more`: block n + 1 exists and its K block has been asked for.
        int n = 0;
        int more = fetch(0);                             // slot 0; m2 = mode of block 1
        if (more < 0) return;
        m1 = m2;
        if (grp == 0) {
            scores(0);
            end_even();
            while (more > 0) {
                fill_v();                             // slot 2n + 1: V(n)
                softmax(m0);
                end_odd();
                more = fetch(n + 1);                     // slot 2n + 2
                if (more < 0) return;
                weighted_values(n);
                scores(n + 1);
                end_even();
                ++n;
                m0 = m1;
                m1 = m2;
            }
            fill_v();                                 // slot 2N - 1
            softmax(m0);
            end_odd();
            weighted_values(n);                   // slot 2N
            end_even();
            end_odd();                                   // slot 2N + 1: group 1 finishes
        } else {
            end_even();                                  // slot 0: group 0 starts
            scores(0);                            // slot 1
            end_odd();
            while (more > 0) {
                more = fetch(n + 1);                     // slot 2n + 2
                if (more < 0) return;
                softmax(m0);
                end_even();
                weighted_values(n);               // slot 2n + 3
                scores(n + 1);
                end_odd();
                ++n;
                m0 = m1;
                m1 = m2;
            }
            softmax(m0);                              // slot 2N
            end_even();
            weighted_values(n);                   // slot 2N + 1
            end_odd();
        }

        // ---- epilogue: lse2 = m + log2(l), O = acc / l, merged into the output under the q blocks' locks ----
        float lse2[2], inv_l[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            float l_tot = l_i[b] + __shfl_xor(l_i[b], 16);
            l_tot += __shfl_xor(l_tot, 32);
            lse2[b] = m_i[b] + fast_log2(l_tot);
            inv_l[b] = 1.0f / l_tot;
        }
        const int lock_idx = (int)(head * (p.Sq / kBlockM)) + qb;
        if (sole_writer) {
            // the only segment that writes these q blocks: nothing to merge with and nobody to exclude
            merge_rows16_through_lds<T>(wave8 < 4 ? k_lds + wave8 * kStageBytes : v_lds + (wave8 - 4) * kStageBytes,
                                      O + z * p.o_st[0] + h * p.o_st[1] + (int64_t)(qb * kBlockM + wave * 32) * p.o_st[2], p.o_st[2],
                                      p.lse + head * p.Sq + qb * kBlockM + wave * 32, o_acc, inv_l, lse2, true, lane);
            __syncthreads();       // the tiles in LDS are free for the next segment's fills
            if (tid == 0) {
                __hip_atomic_store(p.first + lock_idx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.first + lock_idx + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            continue;
        }
        // One lock word per PAIR of q blocks (the lower block's; every program of a launch of this kernel pairs the same
        // blocks), and it carries whether the pair has been written: bit 0 held, bit 1 written.  Taking it is one
        // atomic OR whose result says both whether it was free and whether somebody was first - one trip to memory
        // where a compare-and-swap per block followed by a load of `first` were three - and the hand-over is one store.
        if (tid == 0) {
            const uint64_t t0 = wall_clock64();
            int seen;
            for (;;) {
                seen = __hip_atomic_fetch_or(p.lock + lock_idx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (!(seen & 1)) break;
                __builtin_amdgcn_s_sleep(4);
                if ((int64_t)(wall_clock64() - t0) > p.timeout_ticks) {
                    report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, w, (int)blockIdx.x, -2);
                    s_abort = 1;
                    break;
                }
            }
            s_spun = (seen & 2) == 0;            // (the word is free between flag waits) nobody has written the pair yet
            lock_taken_fence();
        }
        __syncthreads();
        if (__builtin_amdgcn_readfirstlane(s_abort)) return;
        const bool is_first = __builtin_amdgcn_readfirstlane(s_spun) != 0;
        // (the K and V blocks are free: every wavefront has passed the last slot's barrier)
        merge_rows16_through_lds<T>(wave8 < 4 ? k_lds + wave8 * kStageBytes : v_lds + (wave8 - 4) * kStageBytes,
                                  O + z * p.o_st[0] + h * p.o_st[1] + (int64_t)(qb * kBlockM + wave * 32) * p.o_st[2], p.o_st[2],
                                  p.lse + head * p.Sq + qb * kBlockM + wave * 32, o_acc, inv_l, lse2, is_first, lane);

        // every lane's stores have been acknowledged by memory; then the barrier; then the hand-over
        __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));
        __syncthreads();
        if (tid == 0) {
            // tid 0 is in group 0: its lock_idx is the lower q block of the pair
            lock_release_fence();
            __hip_atomic_store(p.lock + lock_idx, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.first + lock_idx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.first + lock_idx + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <typename T>
static int launch_attn_pairs(const AttnParams& p, int grid, int mode, bool causal, hipStream_t stream) {
    const dim3 g(grid), b(kPairThreads);
    if (mode == kPairChainWaves)
        hipLaunchKernelGGL((attn_pair_kernel<T, kPairChainWaves, false>), g, b, 0, stream, p);
    else if (mode == kPairWorkList && causal)
        hipLaunchKernelGGL((attn_pair_kernel<T, kPairWorkList, true>), g, b, 0, stream, p);
    else if (mode == kPairWorkList)
        hipLaunchKernelGGL((attn_pair_kernel<T, kPairWorkList, false>), g, b, 0, stream, p);
    else if (causal)
        hipLaunchKernelGGL((attn_pair_kernel<T, kPairTiles, true>), g, b, 0, stream, p);
    else
        hipLaunchKernelGGL((attn_pair_kernel<T, kPairTiles, false>), g, b, 0, stream, p);
    return (int)hipGetLastError();
}

template <typename T>
static int launch_attn(const AttnParams& p, int grid, hipStream_t stream) {
    hipLaunchKernelGGL((attn_fwd_kernel<T>), dim3(grid), dim3(kAttnThreads), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace syn

extern "C" {

int syn_attn_check_waves(const int32_t* wave_offsets, const int32_t* wave_sizes,
                         const int32_t* cum_wave_sizes, const int32_t* signal_offsets,
                         int32_t num_waves, int32_t Z, int32_t H, int32_t Sq, int32_t Skv,
                         int32_t block_m, int32_t block_n, int64_t cum_tiles, int64_t num_flags) {
    if (!wave_offsets || !wave_sizes || !cum_wave_sizes || !signal_offsets) return SYN_EINVAL;
    if (num_waves <= 0 || Z <= 0 || H <= 0 || Sq <= 0 || Skv <= 0) return SYN_EINVAL;
    if (block_m <= 0 || block_n <= 0 || Sq % block_m || Skv % block_n) return SYN_EINVAL;
    int64_t running = 0;
    bool tail = false;   // zero-filled padding rows may follow the real waves (template.py:613-619)
    for (int w = 0; w < num_waves; ++w) {
        const int32_t* sz = wave_sizes + 4 * w;
        const int32_t* of = wave_offsets + 4 * w;
        if (cum_wave_sizes[w] == 0 && sz[0] == 0 && sz[1] == 0 && sz[2] == 0 && sz[3] == 0) {
            tail = true;
            continue;
        }
        if (tail) return SYN_EINVAL;     // a real wave after padding would never be selected
        for (int a = 0; a < 4; ++a)
            if (sz[a] <= 0 || of[a] < 0) return SYN_EINVAL;
        if (sz[2] % block_m || of[2] % block_m || sz[3] % block_n || of[3] % block_n) return SYN_EINVAL;
        if ((int64_t)of[0] + sz[0] > Z || (int64_t)of[1] + sz[1] > H) return SYN_ERANGE;
        if ((int64_t)of[2] + sz[2] > Sq || (int64_t)of[3] + sz[3] > Skv) return SYN_ERANGE;
        running += (int64_t)sz[0] * sz[1] * sz[2];
        if (cum_wave_sizes[w] != running) return SYN_EINVAL;
        const int64_t sig = signal_offsets[w];
        if (sig < -1) return SYN_EINVAL;
        if (sig >= 0 && num_flags >= 0 && sig >= num_flags) return SYN_ERANGE;
    }
    if (running <= 0 || running != cum_tiles) return SYN_EINVAL;
    return 0;
}

int syn_attn_check_work_list(const int32_t* wave_offsets, const int32_t* wave_sizes, const int32_t* cum_wave_sizes,
                             int32_t num_waves, int32_t block_m, int32_t block_n, int32_t causal,
                             const int32_t* work_list, int64_t work_list_words, int32_t num_programs,
                             int32_t require_masked_visits) {
    if (!wave_offsets || !wave_sizes || !cum_wave_sizes || !work_list) return SYN_EINVAL;
    if (num_waves <= 0 || block_m <= 0 || block_n <= 0 || num_programs <= 0) return SYN_EINVAL;
    if (work_list_words < (int64_t)num_programs + 1) return SYN_EINVAL;
    const int32_t* entries = work_list + num_programs + 1;
    const int64_t num_entries = work_list_words - num_programs - 1;
    if (work_list[0] != 0 || work_list[num_programs] != num_entries) return SYN_EINVAL;
    for (int b = 0; b < num_programs; ++b)
        if (work_list[b + 1] < work_list[b]) return SYN_EINVAL;
    int real_waves = 0;
    while (real_waves < num_waves && cum_wave_sizes[real_waves] != 0) ++real_waves;
    if (real_waves == 0 || cum_wave_sizes[real_waves - 1] % (2 * block_m)) return SYN_EINVAL;
    const int64_t pairs = cum_wave_sizes[real_waves - 1] / block_m / 2;

    struct Visit { int z, h, qb, walked; };
    auto visit_of = [&](int64_t pair, Visit* v) -> bool {
        int w = 0;
        while (w < real_waves && cum_wave_sizes[w] / block_m <= 2 * pair) ++w;
        if (w >= real_waves) return false;
        const int prev = w == 0 ? 0 : cum_wave_sizes[w - 1] / block_m;
        const int t = (int)(2 * pair) - prev;
        const int sh = wave_sizes[4 * w + 1], nq = wave_sizes[4 * w + 2] / block_m;
        if (sh <= 0 || nq <= 0 || (nq & 1) || (prev & 1)) return false;
        v->z = t / (nq * sh) + wave_offsets[4 * w];
        v->h = (t / nq) % sh + wave_offsets[4 * w + 1];
        v->qb = t % nq + wave_offsets[4 * w + 2] / block_m;
        const int lo = wave_offsets[4 * w + 3] / block_n, len = wave_sizes[4 * w + 3] / block_n;
        v->walked = len;
        if (causal) {
            if ((lo & 1) || (v->qb & 1)) return false;
            v->walked = len < v->qb + 2 - lo ? len : v->qb + 2 - lo;
        }
        return true;
    };

    std::vector<unsigned char> seen((size_t)pairs, 0);
    // per pair of q blocks: segments that write it, and whether one of them claims to be the only one
    std::map<std::array<int, 3>, std::pair<int, int>> writers;
    for (int b = 0; b < num_programs; ++b) {
        bool continued = false;
        Visit first{};
        for (int64_t i = work_list[b]; i < work_list[b + 1]; ++i) {
            const int32_t entry = entries[i];
            if (entry & ~(SYN_ATTN_WORK_PAIR_MASK | SYN_ATTN_WORK_CONTINUES | SYN_ATTN_WORK_SOLE_WRITER)) return SYN_EINVAL;
            const int64_t pair = entry & SYN_ATTN_WORK_PAIR_MASK;
            if (pair >= pairs || seen[(size_t)pair]) return SYN_EINVAL;       // every visit at most once
            seen[(size_t)pair] = 1;
            Visit v;
            if (!visit_of(pair, &v)) return SYN_EINVAL;
            const bool continues = (entry & SYN_ATTN_WORK_CONTINUES) != 0;
            if (v.walked <= 0) {
                // wholly above the diagonal: logged, nothing else; never part of a segment
                if (continued || continues) return SYN_EINVAL;
                continue;
            }
            if (continued) {
                if (v.z != first.z || v.h != first.h || v.qb != first.qb) return SYN_EINVAL;
            } else {
                first = v;
                auto& wr = writers[{v.z, v.h, v.qb}];
                wr.first += 1;
                wr.second += (entry & SYN_ATTN_WORK_SOLE_WRITER) ? 1 : 0;
            }
            if (continues && i + 1 >= work_list[b + 1]) return SYN_EINVAL;    // nothing to continue with
            continued = continues;
        }
    }
    for (const auto& kv : writers)
        if (kv.second.second && kv.second.first != 1) return SYN_EINVAL;      // "only writer" beside another segment
    for (int64_t pair = 0; pair < pairs; ++pair) {
        if (seen[(size_t)pair]) continue;
        Visit v;
        if (!visit_of(pair, &v)) return SYN_EINVAL;
        if (v.walked > 0 || require_masked_visits) return SYN_EINVAL;         // a visit with work is missing
    }
    return 0;
}

int syn_attn_fwd(const syn_attn_desc* d, syn_stream_t stream) {
    using namespace syn;
    if (d == nullptr) return SYN_EINVAL;
    if (!d->q || !d->k || !d->v || !d->o || !d->lse || !d->lock || !d->first) return SYN_EINVAL;
    if (!d->wave_offsets || !d->wave_sizes || !d->cum_wave_sizes || !d->signal_offsets || !d->flags)
        return SYN_EINVAL;
    if (d->num_waves <= 0 || d->Z <= 0 || d->H <= 0 || d->Sq <= 0 || d->Skv <= 0) return SYN_EINVAL;
    if (d->D != kHeadDim || d->block_m != kBlockM || d->block_n != kBlockN) return SYN_EINVAL;
    if (d->Sq % kBlockM || d->Skv % kBlockN) return SYN_EINVAL;
    if (d->dtype != SYN_DTYPE_BF16 && d->dtype != SYN_DTYPE_FP16) return SYN_EINVAL;
    if (d->causal && d->Sq != d->Skv) return SYN_EINVAL;
    if (d->cum_tiles <= 0 || d->cum_tiles % kBlockM) return SYN_EINVAL;
    if ((d->wait_flags == nullptr) != (d->wait_signal_offsets == nullptr)) return SYN_EINVAL;
    if (d->wait_flags && !d->counters) return SYN_EINVAL;     // without counters `flags` is what is waited for
    if (!(d->sm_scale > 0.f)) return SYN_EINVAL;
    if (!aligned16(d->q) || !aligned16(d->k) || !aligned16(d->v) || !aligned16(d->o)) return SYN_EALIGN;
    if (d->visit_log && !aligned16(d->visit_log)) return SYN_EALIGN;
    const int64_t tiles = d->cum_tiles / kBlockM;
    if (tiles > INT32_MAX) return SYN_EINVAL;

    AttnParams p;
    p.q = d->q;
    p.k = d->k;
    p.v = d->v;
    p.o = d->o;
    p.lse = d->lse;
    p.lock = d->lock;
    p.first = d->first;
    p.flags = d->flags;
    p.wave_offsets = d->wave_offsets;
    p.wave_sizes = d->wave_sizes;
    p.cum_wave_sizes = d->cum_wave_sizes;
    p.signal_offsets = d->signal_offsets;
    p.visit_log = d->visit_log;
    p.status = d->status;
    p.counters = d->counters;
    p.wait_flags = d->wait_flags;
    p.wait_offsets = d->wait_signal_offsets;
    p.timeout_ticks = timeout_ticks(d->spin_timeout_us);
    p.num_waves = d->num_waves;
    p.Z = d->Z;
    p.H = d->H;
    p.Sq = d->Sq;
    p.Skv = d->Skv;
    p.causal = d->causal ? 1 : 0;
    p.num_tiles = (int)tiles;
    p.xcd_remap = (d->options & SYN_ATTN_XCD_REMAP) ? 1 : 0;
    p.acquire_always = (d->options & SYN_ATTN_ACQUIRE_ALWAYS) ? 1 : 0;
    p.work_list = d->work_list;
    p.qk_scale = d->sm_scale * 1.44269504f;
    {
        // all-zero strides: contiguous [Z, H, S, D]
        const int64_t dq[3] = {(int64_t)d->H * d->Sq * kHeadDim, (int64_t)d->Sq * kHeadDim, kHeadDim};
        const int64_t dk[3] = {(int64_t)d->H * d->Skv * kHeadDim, (int64_t)d->Skv * kHeadDim, kHeadDim};
        struct { const int64_t* in; const int64_t* dflt; int64_t* out; } sets[4] = {
            {d->q_strides, dq, p.q_st}, {d->k_strides, dk, p.k_st}, {d->v_strides, dk, p.v_st}, {d->o_strides, dq, p.o_st}};
        for (auto& s : sets) {
            const bool unset = s.in[0] == 0 && s.in[1] == 0 && s.in[2] == 0;
            for (int i = 0; i < 3; ++i) {
                s.out[i] = unset ? s.dflt[i] : s.in[i];
                if (s.out[i] < 0 || s.out[i] % 8) return SYN_EALIGN;     // 16-byte rows
            }
            if (s.out[2] < kHeadDim) return SYN_EINVAL;
            // the lane offset of a fill is 32 bits: 4 rows at the pitch must fit
            if (s.out[2] * 2 * 4 > (int64_t)UINT32_MAX) return SYN_EINVAL;
        }
    }

    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (d->options & SYN_ATTN_PAIR_Q_BLOCKS) {
        // two q blocks per workgroup: the caller vouches for an even number of q blocks in every wave
        if (d->counters || d->wait_flags || d->wait_signal_offsets || tiles % 2) return SYN_EINVAL;
        const bool chain = (d->options & SYN_ATTN_CHAIN_Q_BLOCKS) != 0;
        const bool list = (d->options & SYN_ATTN_WORK_LIST) != 0;
        if (chain && (list || d->causal)) return SYN_EINVAL;
        if ((chain || list) && d->num_programs <= 0) return SYN_EINVAL;
        if (list != (d->work_list != nullptr)) return SYN_EINVAL;
        int grid = d->num_programs > 0 ? d->num_programs : (int)(tiles / 2);
        if (!list && grid > tiles / 2) grid = (int)(tiles / 2);      // a list names its programs' visits itself
        const int mode = chain ? kPairChainWaves : (list ? kPairWorkList : kPairTiles);
        return d->dtype == SYN_DTYPE_BF16 ? launch_attn_pairs<__bf16>(p, grid, mode, d->causal != 0, s)
                                          : launch_attn_pairs<_Float16>(p, grid, mode, d->causal != 0, s);
    }
    if (d->options & (SYN_ATTN_CHAIN_Q_BLOCKS | SYN_ATTN_WORK_LIST)) return SYN_EINVAL;
    if (d->work_list != nullptr) return SYN_EINVAL;
    int grid = d->num_programs > 0 ? d->num_programs : (int)tiles;
    if (grid > tiles) grid = (int)tiles;
    return d->dtype == SYN_DTYPE_BF16 ? launch_attn<__bf16>(p, grid, s)
                                      : launch_attn<_Float16>(p, grid, s);
}

}  // extern "C"
