// Chunk-scheduled persistent GEMM for gfx950 (MI355X): C = A * B^T, fp32 accumulate.
//
// One 256-thread workgroup (4 wavefronts, 2x2) owns a BM x BN tile of C and
// walks tile ids pid, pid + NUM_SMS, ... in the wave order of the schedule
// (syncopate/computation/gemm/template.py:69-136).  A and B are both
// K-contiguous, so a k-slab of either is a set of 128-byte rows: slabs are
// staged through LDS in a double buffer (global -> registers -> LDS, 16 bytes
// per lane), rows XOR-swizzled in 16-byte chunks so that the 128-bit fragment
// reads of v_mfma_f32_32x32x16 are bank-conflict free.
//
// Consumer form: before the first tile of a wave whose signal offset is >= 0
// lane 0 spins on the flag word, then the whole workgroup takes an acquire
// fence (template.py:121-128).  Producer form: after the C tile is stored the
// workgroup bumps counters[wave] and the last tile of the wave publishes the
// flag (template.py:343-348).
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
};

constexpr int kGemmThreads = 256;
constexpr int kBlockK = 64;          // elements; one LDS row = 128 bytes
constexpr int kRowBytes = kBlockK * 2;

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
    v[0] = (T)x0;  // round-to-nearest-even (v_cvt_pk_bf16_f32 / v_cvt_pkrtz is not used for f16)
    v[1] = (T)x1;
    v[2] = (T)x2;
    v[3] = (T)x3;
    return __builtin_bit_cast(uint2, v);
}


template <int BM, int BN>
constexpr int gemm_lds_bytes() {
    return 2 * (BM + BN) * kRowBytes;
}


// 16 bytes per lane and load: rows ld_row + 32*i of a slab (src already points
// at this lane's row and 16-byte chunk)
template <typename T, int LOADS>
__device__ __forceinline__ void load_slab(uint4 (&r)[LOADS], const T* src, int K) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
        r[i] = *reinterpret_cast<const uint4*>(src + (size_t)(32 * i) * K);
}

template <int LOADS>
__device__ __forceinline__ void store_slab(unsigned char* dst, const uint4 (&r)[LOADS]) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
        *reinterpret_cast<uint4*>(dst + i * 32 * kRowBytes) = r[i];
}

// One 64-deep slab: four k16 steps of TM x TN MFMAs.  B is the first operand,
// so each accumulator holds the transposed 32x32 tile D'[n][m].
template <typename T, int TM, int TN>
__device__ __forceinline__ void mma_slab(f32x16_t (&acc)[TM][TN], const unsigned char* sbase,
                                         int a_rd, int b_rd, int frag_half, int frag_swz) {
    typedef typename Mfma32<T>::frag_t frag_t;
#pragma unroll
    for (int kk = 0; kk < kBlockK / 16; ++kk) {
        const int chunk = ((kk * 2 + frag_half) ^ frag_swz) << 4;
        frag_t fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
            fa[i] = *reinterpret_cast<const frag_t*>(sbase + a_rd + i * 32 * kRowBytes + chunk);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[j] = *reinterpret_cast<const frag_t*>(sbase + b_rd + j * 32 * kRowBytes + chunk);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = Mfma32<T>::run(fb[j], fa[i], acc[i][j]);
    }
}

template <typename T, int BM, int BN, bool PRODUCER>
__global__ void __launch_bounds__(kGemmThreads) gemm_wave_kernel(const GemmParams p) {
    typedef typename Mfma32<T>::frag_t frag_t;
    constexpr int WM = BM / 2, WN = BN / 2;       // wavefront tile
    constexpr int TM = WM / 32, TN = WN / 32;     // 32x32 MFMA tiles per wavefront
    constexpr int A_LOADS = BM / 32, B_LOADS = BN / 32;
    constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes;
    constexpr int STAGE_BYTES = A_BYTES + B_BYTES;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int s_abort;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int pid = logical_program_id((int)blockIdx.x, (int)gridDim.x, p.xcd_remap != 0);
    const int num_sms = p.num_sms;
    const int num_tiles = p.num_tiles;
    const int tiles_here = num_tiles / num_sms + (pid < num_tiles % num_sms ? 1 : 0);

    const int K = p.K, N = p.N;
    const int k_steps = K / kBlockK;

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

    // --- per-thread staging geometry ---
    const int ld_row = tid >> 3;                       // 0..31, +32 per load
    const int ld_chunk = tid & 7;                      // 16-byte chunk inside the 128-byte row
    const int st_off = ld_row * kRowBytes + ((ld_chunk ^ (ld_row & 7)) << 4);

    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    const int frag_swz = lane & 7;
    const int a_rd = (wm * WM + frag_row) * kRowBytes;
    const int b_rd = A_BYTES + (wn * WN + frag_row) * kRowBytes;

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

        const T* a_src = A + (m0 + ld_row) * (size_t)K + ld_chunk * 8;
        const T* b_src = B + (n0 + ld_row) * (size_t)K + ld_chunk * 8;

        f32x16_t acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

        uint4 ra[A_LOADS], rb[B_LOADS];

        __syncthreads();                 // previous tile's LDS reads are done
        load_slab<T, A_LOADS>(ra, a_src, K);
        load_slab<T, B_LOADS>(rb, b_src, K);
        store_slab<A_LOADS>(smem + st_off, ra);
        store_slab<B_LOADS>(smem + A_BYTES + st_off, rb);
        __syncthreads();

        // steady state: prefetch slab ks+1 into registers, multiply slab ks out
        // of LDS, then park the prefetched slab in the other LDS stage
        for (int ks = 0; ks + 1 < k_steps; ++ks) {
            const int stage = ks & 1;
            load_slab<T, A_LOADS>(ra, a_src + (size_t)(ks + 1) * kBlockK, K);
            load_slab<T, B_LOADS>(rb, b_src + (size_t)(ks + 1) * kBlockK, K);
            mma_slab<T, TM, TN>(acc, smem + stage * STAGE_BYTES, a_rd, b_rd, frag_half, frag_swz);
            unsigned char* nxt = smem + (stage ^ 1) * STAGE_BYTES + st_off;
            store_slab<A_LOADS>(nxt, ra);
            store_slab<B_LOADS>(nxt + A_BYTES, rb);
            __syncthreads();
        }
        mma_slab<T, TM, TN>(acc, smem + ((k_steps - 1) & 1) * STAGE_BYTES, a_rd, b_rd, frag_half, frag_swz);

        // Epilogue.  With B as the first MFMA operand a lane holds, for column
        // m = lane % 32 of D', rows n = 8g + 4*(lane/32) + 0..3: four consecutive
        // elements of one row of C -> one 8-byte store.
        {
            T* c_row = C + (m0 + wm * WM + frag_row) * (size_t)N + n0 + wn * WN + 4 * frag_half;
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

template <typename T, int BM, int BN, bool PRODUCER>
static int launch_gemm(const GemmParams& p, int grid, hipStream_t stream) {
    constexpr int lds = gemm_lds_bytes<BM, BN>();
    static bool attr_done[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev >= 0 && dev < 64 && !attr_done[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_wave_kernel<T, BM, BN, PRODUCER>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return (int)e;
        attr_done[dev] = true;
    }
    hipLaunchKernelGGL((gemm_wave_kernel<T, BM, BN, PRODUCER>), dim3(grid), dim3(kGemmThreads), lds, stream, p);
    return (int)hipGetLastError();
}

template <typename T, bool PRODUCER>
static int dispatch_tile(const GemmParams& p, int bm, int bn, int grid, hipStream_t stream) {
    if (bm == 256 && bn == 256) return launch_gemm<T, 256, 256, PRODUCER>(p, grid, stream);
    if (bm == 128 && bn == 256) return launch_gemm<T, 128, 256, PRODUCER>(p, grid, stream);
    if (bm == 256 && bn == 128) return launch_gemm<T, 256, 128, PRODUCER>(p, grid, stream);
    if (bm == 128 && bn == 128) return launch_gemm<T, 128, 128, PRODUCER>(p, grid, stream);
    return SYN_EINVAL;
}

static int gemm_entry(const syn_gemm_desc* d, hipStream_t stream, bool producer) {
    if (d == nullptr) return SYN_EINVAL;
    if (!d->a || !d->b || !d->c || !d->wave_sizes || !d->wave_offsets || !d->signal_offsets)
        return SYN_EINVAL;
    if (d->num_waves <= 0 || d->M <= 0 || d->N <= 0 || d->K <= 0) return SYN_EINVAL;
    if (d->block_k != kBlockK) return SYN_EINVAL;
    if (d->group_m <= 0 || d->num_sms <= 0) return SYN_EINVAL;
    if (d->dtype != SYN_DTYPE_BF16 && d->dtype != SYN_DTYPE_FP16) return SYN_EINVAL;
    if (d->M % d->block_m || d->N % d->block_n || d->K % kBlockK) return SYN_EINVAL;
    if (!aligned16(d->a) || !aligned16(d->b) || !aligned16(d->c)) return SYN_EALIGN;
    if (producer && d->counters == nullptr) return SYN_EINVAL;
    if (d->flags == nullptr) return SYN_EINVAL;
    if (d->visit_log && !aligned16(d->visit_log)) return SYN_EALIGN;

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

    if (d->dtype == SYN_DTYPE_BF16) {
        return producer ? dispatch_tile<__bf16, true>(p, d->block_m, d->block_n, grid, stream)
                        : dispatch_tile<__bf16, false>(p, d->block_m, d->block_n, grid, stream);
    }
    return producer ? dispatch_tile<_Float16, true>(p, d->block_m, d->block_n, grid, stream)
                    : dispatch_tile<_Float16, false>(p, d->block_m, d->block_n, grid, stream);
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
