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
// Data path per 128-wide kv block, 4 wavefronts x 32 q rows each:
//   S^T[kv, q] = K[kv, :] . Q[q, :]      K from LDS (A operand), Q fragments in registers
//   P^T        = exp2(S^T * scale - m)   per-q statistics are lane-local: lane % 32 == q
//   O^T[d, q] += V^T[d, kv] . P^T[kv, q] V^T from LDS (transposed while staging)
// Computing the transposed products keeps each q column in one lane pair, so
// the softmax needs one cross-lane exchange per block, and the accumulator
// layout of S^T is already the B-operand layout of the second product.
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
    int64_t timeout_ticks;
    int32_t num_waves;
    int32_t Z, H, Sq, Skv;
    int32_t causal;
    int32_t num_tiles;
    float qk_scale;       // sm_scale * 1.44269504 (template.py:178-179)
};

constexpr int kAttnThreads = 256;
constexpr int kHeadDim = 128;
constexpr int kBlockM = 128;
constexpr int kBlockN = 128;
constexpr int kKRowBytes = kHeadDim * 2;            // 256
constexpr int kVtPitch = kBlockN * 2 + 8;           // 264: rows of V^T, padded against bank conflicts
constexpr int kKBytes = kBlockN * kKRowBytes;       // 32768
constexpr int kVtBytes = kHeadDim * kVtPitch;       // 33792
constexpr int kAttnLdsBytes = kKBytes + kVtBytes;

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

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// low/high 16-bit halves of two dwords -> one dword
__device__ __forceinline__ uint32_t pack_lo(uint32_t a, uint32_t b) { return (a & 0xffffu) | (b << 16); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xffff0000u); }


// One kv block into registers: K as 8 row-chunks of 16 bytes, V as two 4x8 units.
template <typename T>
__device__ __forceinline__ void load_kv_block(u32x4_t (&rk)[8], u32x4_t (&rv)[8], const T* k_src,
                                              const T* v_src, int n) {
    const size_t blk = (size_t)n * kBlockN * kHeadDim;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        rk[i] = *reinterpret_cast<const u32x4_t*>(k_src + blk + (size_t)(16 * i) * kHeadDim);
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            rv[4 * u + i] = *reinterpret_cast<const u32x4_t*>(v_src + blk + (size_t)i * kHeadDim + 64 * u);
}

template <typename T>
__global__ void __launch_bounds__(kAttnThreads) attn_fwd_kernel(const AttnParams p) {
    typedef typename AttnMfma<T>::frag_t frag_t;
    typedef T vec4_t __attribute__((ext_vector_type(4)));

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int s_abort;
    unsigned char* k_lds = smem;
    unsigned char* vt_lds = smem + kKBytes;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r = lane & 31;
    const int half = lane >> 5;

    if (tid == 0) s_abort = 0;
    __syncthreads();

    // K staging: 16-byte chunk c of row (tid/16 + 16*i)
    const int k_c = tid & 15;
    const int k_row = tid >> 4;
    const int k_st = k_row * kKRowBytes + ((k_c ^ (k_row & 15)) << 4);
    // V staging: unit (a, b) = 4 kv rows x 8 d columns, two units per thread
    const int v_a = tid & 31;
    const int v_b = tid >> 5;          // 0..7, second unit at +8

    const T* __restrict__ Q = reinterpret_cast<const T*>(p.q);
    const T* __restrict__ K = reinterpret_cast<const T*>(p.k);
    const T* __restrict__ V = reinterpret_cast<const T*>(p.v);
    T* __restrict__ O = reinterpret_cast<T*>(p.o);

    for (int tile_id = blockIdx.x; tile_id < p.num_tiles; tile_id += gridDim.x) {
        // ---- tile id -> wave -> (z, h, q block, kv range) ----
        int w = 0;
        while (w < p.num_waves && p.cum_wave_sizes[w] / kBlockM <= tile_id) ++w;
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

        // causal: kv blocks strictly above the diagonal contribute nothing
        const int kv_end = p.causal ? min(kv_hi, qb + 1) : kv_hi;
        if (kv_lo >= kv_end) continue;

        if (sig >= 0) {
            if (tid == 0) {
                const bool ok = spin_until_equal(p.flags + sig, 1ull, p.timeout_ticks);
                if (!ok) {
                    report_status(p.status, SYN_STATUS_SPIN_TIMEOUT, w, (int)blockIdx.x, sig);
                    s_abort = 1;
                }
            }
            __syncthreads();
            acquire_fence_agent();
            if (s_abort) return;
        }

        const size_t head = (size_t)z * p.H + h;
        const int q_row = qb * kBlockM + wave * 32 + r;              // this lane's q position
        const T* q_src = Q + (head * p.Sq + q_row) * kHeadDim + 8 * half;
        const T* k_base = K + head * (size_t)p.Skv * kHeadDim;
        const T* v_base = V + head * (size_t)p.Skv * kHeadDim;

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

        u32x4_t rk[8], rv[8];
        const T* k_src = k_base + (size_t)k_row * kHeadDim + k_c * 8;
        const T* v_src = v_base + (size_t)(4 * v_a) * kHeadDim + v_b * 8;
        load_kv_block<T>(rk, rv, k_src, v_src, kv_lo);

        for (int n = kv_lo; n < kv_end; ++n) {
            __syncthreads();                 // LDS of the previous block has been consumed
#pragma unroll
            for (int i = 0; i < 8; ++i)
                *reinterpret_cast<u32x4_t*>(k_lds + k_st + i * 16 * kKRowBytes) = rk[i];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                // transpose 4 kv x 8 d: for each d, the 4 kv values become one 8-byte word
                const u32x4_t x0 = rv[4 * u + 0], x1 = rv[4 * u + 1], x2 = rv[4 * u + 2], x3 = rv[4 * u + 3];
                unsigned char* dst = vt_lds + ((v_b + 8 * u) * 8) * kVtPitch + v_a * 8;
#pragma unroll
                for (int dw = 0; dw < 4; ++dw) {
                    uint2 even, odd;
                    even.x = pack_lo(x0[dw], x1[dw]);
                    even.y = pack_lo(x2[dw], x3[dw]);
                    odd.x = pack_hi(x0[dw], x1[dw]);
                    odd.y = pack_hi(x2[dw], x3[dw]);
                    *reinterpret_cast<uint2*>(dst + (2 * dw) * kVtPitch) = even;
                    *reinterpret_cast<uint2*>(dst + (2 * dw + 1) * kVtPitch) = odd;
                }
            }
            __syncthreads();
            // prefetch the next block (the last iteration re-reads its own block: no branch)
            load_kv_block<T>(rk, rv, k_src, v_src, min(n + 1, kv_end - 1));

            // ---- S^T = K . Q^T : 4 tiles of [32 kv, 32 q] ----
            f32x16_t s[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) s[j][e] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const int chunk = ((2 * ks + half) ^ (r & 15)) << 4;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const frag_t kf = *reinterpret_cast<const frag_t*>(
                        k_lds + (32 * j + r) * kKRowBytes + chunk);
                    s[j] = AttnMfma<T>::run(kf, qf[ks], s[j]);
                }
            }

            // ---- online softmax in base 2 ----
            if (p.causal && n == qb) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int kv_pos = n * kBlockN + 32 * j + 8 * (e >> 2) + 4 * half + (e & 3);
                        if (kv_pos > q_row) s[j][e] = -INFINITY;
                    }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[j][e]);
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_i, mx * p.qk_scale);
            const float alpha = fast_exp2(m_i - m_new);
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
            l_i = l_i * alpha + row_sum;
            m_i = m_new;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;

            // ---- O^T += V^T . P^T ----
#pragma unroll
            for (int t2 = 0; t2 < 8; ++t2) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const unsigned char* src = vt_lds + (32 * i + r) * kVtPitch + (16 * t2 + 4 * half) * 2;
                    const uint2 lo = *reinterpret_cast<const uint2*>(src);
                    const uint2 hi = *reinterpret_cast<const uint2*>(src + 16);
                    const u32x4_t both = {lo.x, lo.y, hi.x, hi.y};
                    const frag_t vf = __builtin_bit_cast(frag_t, both);
                    o_acc[i] = AttnMfma<T>::run(vf, pf[t2], o_acc[i]);
                }
            }
        }

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
        }
        __syncthreads();
        acquire_fence_agent();
        if (s_abort) return;

        const bool is_first = __hip_atomic_load(p.first + lock_idx, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT) == 0;
        float w_old = 0.f, w_new = 1.f, lse_out = lse2;
        float* lse_ptr = p.lse + head * p.Sq + q_row;
        if (!is_first) {
            // merge with the stored partial (template.py:335-349)
            const float m_old = *lse_ptr;
            const float delta = m_old - lse2;
            const float mmax = fmaxf(m_old, lse2);
            lse_out = mmax + fast_log2(1.0f + fast_exp2(-fabsf(delta)));
            w_old = fast_exp2(m_old - lse_out);
            w_new = fast_exp2(lse2 - lse_out);
        }
        T* o_row = O + (head * p.Sq + q_row) * kHeadDim + 4 * half;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float x[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) x[c] = o_acc[i][4 * g + c] * inv_l * w_new;
                T* dst = o_row + 32 * i + 8 * g;
                if (!is_first) {
                    const vec4_t old = *reinterpret_cast<const vec4_t*>(dst);
#pragma unroll
                    for (int c = 0; c < 4; ++c) x[c] += (float)old[c] * w_old;
                }
                vec4_t out;
#pragma unroll
                for (int c = 0; c < 4; ++c) out[c] = (T)x[c];
                *reinterpret_cast<vec4_t*>(dst) = out;
            }
        if (half == 0) *lse_ptr = lse_out;

        __threadfence();
        __syncthreads();
        if (tid == 0) {
            __hip_atomic_store(p.first + lock_idx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(p.lock + lock_idx, 0, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <typename T>
static int launch_attn(const AttnParams& p, int grid, hipStream_t stream) {
    static bool attr_done[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev >= 0 && dev < 64 && !attr_done[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_kernel<T>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kAttnLdsBytes);
        if (e != hipSuccess) return (int)e;
        attr_done[dev] = true;
    }
    hipLaunchKernelGGL((attn_fwd_kernel<T>), dim3(grid), dim3(kAttnThreads), kAttnLdsBytes, stream, p);
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
    p.timeout_ticks = timeout_ticks(d->spin_timeout_us);
    p.num_waves = d->num_waves;
    p.Z = d->Z;
    p.H = d->H;
    p.Sq = d->Sq;
    p.Skv = d->Skv;
    p.causal = d->causal ? 1 : 0;
    p.num_tiles = (int)tiles;
    p.qk_scale = d->sm_scale * 1.44269504f;

    int grid = d->num_programs > 0 ? d->num_programs : (int)tiles;
    if (grid > tiles) grid = (int)tiles;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    return d->dtype == SYN_DTYPE_BF16 ? launch_attn<__bf16>(p, grid, s)
                                      : launch_attn<_Float16>(p, grid, s);
}

}  // extern "C"
