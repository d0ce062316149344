/*
 * syncopate_hip.h — C ABI of libsyncopate_hip.so (MI355X / gfx950).
 *
 * Hand-written CDNA4 kernels for the per-rank chunk-scheduled compute path of
 * Syncopate: the AG+GEMM consumer, the GEMM+RS producer and its chunked ring
 * reduce, the chunked-KV flash attention, and the tiny stream-side flag
 * primitives a single-GPU producer needs.  Every entry point takes plain
 * pointers and sizes (device pointers unless a parameter says "host"), never
 * allocates device memory, launches on the stream it is given and returns
 * 0 on success, a negative SYN_E* code for rejected arguments, or a positive
 * hipError_t.
 *
 * Units follow the reference's generated-kernel convention: wave sizes and
 * offsets are in ELEMENTS and are divided by the block sizes inside the
 * kernel (syncopate/computation/gemm/template.py:82-87,
 * syncopate/computation/transform/transformer.py:616-621).
 */
#ifndef SYNCOPATE_HIP_H
#define SYNCOPATE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
#define SYN_DTYPE_BF16 0
#define SYN_DTYPE_FP16 1

/* argument errors (negative so they never collide with hipError_t) */
#define SYN_EINVAL (-22)   /* malformed argument / unsupported configuration */
#define SYN_ERANGE (-34)   /* wave table addresses tiles outside the operand  */
#define SYN_EALIGN (-75)   /* pointer or extent not aligned as the kernel needs */
#define SYN_E2BIG (-7)     /* more waves than the static scratch of syn_gemm_producer_static holds */

/* capacity of syn_gemm_producer_static: waves per launch (one int32 counter each, 16 KB per device) */
#define SYN_STATIC_MAX_WAVES 4096

/* device-side status words (int32[SYN_STATUS_WORDS], caller-zeroed) */
#define SYN_STATUS_WORDS 4
#define SYN_STATUS_OK 0
#define SYN_STATUS_SPIN_TIMEOUT 1   /* [1]=wave index, [2]=program id, [3]=signal offset */
#define SYN_STATUS_BAD_PAIRING 2    /* SYN_ATTN_PAIR_Q_BLOCKS on a wave with an odd number of q blocks:
                                       [1]=wave index, [2]=program id, [3]=q blocks of the wave */
#define SYN_STATUS_BAD_CHAIN 3      /* SYN_ATTN_CHAIN_Q_BLOCKS: [1]=wave whose (z, h, q) ranges differ from wave 0's, or 0
                                       and [3]=pairs per wave when the grid is not that many programs;
                                       SYN_ATTN_WORK_LIST: [1]=wave, [3]=tile id of an entry that cannot continue
                                       its segment (other q blocks, or nothing below the diagonal) */

/* gemm option bits */
#define SYN_GEMM_XCD_REMAP 1u       /* permute hardware workgroup ids so that consecutive
                                       logical program ids share an XCD (and its L2)      */
#define SYN_GEMM_EIGHT_WAVES 2u     /* 512-thread workgroups (two wavefronts per SIMD)     */
#define SYN_GEMM_RING_PIPE 4u       /* four LDS stages of 32-deep K slabs instead of the default
                                       two or three stages of 64-deep slabs; needs K % 128 == 0,
                                       otherwise the default pipeline runs                 */
#define SYN_GEMM_NO_K_STAGGER 8u    /* every tile sweeps K from 0 (default: neighbouring
                                       tiles start 128 elements apart and wrap around, which
                                       spreads lockstep programs over the memory channels;
                                       the fp32 sums are then taken in rotated order)      */
#define SYN_GEMM_TWO_STAGE 16u      /* two LDS stages even for tiles of which three fit (every
                                       shape but 256x256): one slab in flight instead of two */
#define SYN_GEMM_MFMA_32X32 32u     /* the default K loops on 32x32x16 MFMAs instead of 16x16x32
                                       ones, which cost less energy per product on a power-limited
                                       board; same results bit for bit                       */

#define SYN_GEMM_ACQUIRE_ALWAYS 64u  /* take the agent-scope acquire fence behind EVERY flag wait.  Without
                                       it a program whose flag is already up when it looks reads the chunk
                                       without a fence (the fence empties the XCD's L2 of the operand panels
                                       its neighbours reuse), which is safe only if the caller sees to it that
                                       (1) nothing on the device - an earlier iteration still running, another
                                       kernel - reads the gathered buffer between the start of this kernel and
                                       a chunk's flag, and (2) no flag word is raised more than once during
                                       the launch.  The reference always acquires (dl.wait,
                                       gemm/template.py:92-97,121-128); callers that cannot promise (1) and (2)
                                       set this bit. */

typedef void* syn_stream_t;        /* hipStream_t */

/*
 * Wave table of a GEMM launch: num_waves rows, row w = one wave (one arrived
 * chunk).  wave_sizes[w] = {rows, cols} and wave_offsets[w] = {row0, col0} of
 * the C region the wave covers, in elements; signal_offsets[w] = index of the
 * flag word that gates (consumer) or publishes (producer) the wave, or -1.
 * Produced by RawSchedule.gen_block_shape_lists / gen_block_offset_lists /
 * gen_signal_lists (syncopate/interface/tile_schedule.py:90-115).
 */
typedef struct syn_gemm_desc {
    const void* a;                  /* [M, K] row-major                                    */
    const void* b;                  /* [N, K] row-major (K contiguous), template.py:53-58  */
    void* c;                        /* [M, N] row-major                                    */
    uint64_t* flags;                /* flag words, value 1 = set                           */
    const int32_t* wave_sizes;      /* device, [num_waves, 2]                              */
    const int32_t* wave_offsets;    /* device, [num_waves, 2]                              */
    const int32_t* signal_offsets;  /* device, [num_waves]                                 */
    int32_t* counters;              /* producer only: device int32[num_waves], zeroed      */
    int32_t* visit_log;             /* optional device int32[num_tiles, 4]:
                                       {program id, wave, pid_m, pid_n} per tile id         */
    int32_t* status;                /* optional device int32[SYN_STATUS_WORDS]             */
    int32_t num_waves;
    int32_t M, N, K;
    int32_t dtype;                  /* SYN_DTYPE_*                                         */
    int32_t block_m, block_n, block_k;
    int32_t group_m;                /* GROUP_SIZE_M of get_pid_mn, template.py:10-18       */
    int32_t num_sms;                /* NUM_SMS: tile id stride of the persistent walk      */
    int64_t cum_tiles;              /* sum rows*cols over waves (elements); 0 = M*N        */
    int64_t spin_timeout_us;        /* <=0: default (2 s); flag waits give up after this   */
    uint32_t options;               /* SYN_GEMM_* bits                                     */
} syn_gemm_desc;

/*
 * AG+GEMM consumer: C = A * B^T with fp32 accumulation, output tiles visited
 * in wave order by a persistent grid; before the first tile of a wave whose
 * signal offset is >= 0 the workgroup spins (acquire) until that flag == 1.
 * Replaces kernel_gemm_consumer / gemm_consumer
 * (syncopate/computation/gemm/template.py:21-220) and the generated
 * consumer form (syncopate/computation/transform/transformer.py:759-879).
 */
int syn_gemm_consumer(const syn_gemm_desc* desc, syn_stream_t stream);

/*
 * GEMM+RS producer: same GEMM and walk; after each C tile of a wave with a
 * signal offset >= 0 the workgroup does counters[wave]++ (release) and the
 * one that observes rows*cols/(BM*BN) - 1 sets flags[signal] = 1.
 * Replaces kernel_gemm_producer / gemm_producer
 * (syncopate/computation/gemm/template.py:224-412).
 */
int syn_gemm_producer(const syn_gemm_desc* desc, syn_stream_t stream);

/*
 * syn_gemm_producer for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference, whose launcher allocates a zeroed counter tensor per call (template.py:388).
 * desc->counters must be NULL: the per-wave tile counters live in a static device array of
 * SYN_STATIC_MAX_WAVES words inside the library (each device holds its own copy until the
 * process ends), cleared by a small fill kernel on `stream` in front of the GEMM.  The call
 * itself allocates nothing and frees nothing.  More than SYN_STATIC_MAX_WAVES waves:
 * SYN_E2BIG.  Every call on a device shares that device's array: calls that overlap on one
 * device (two streams, two threads) race on the counters and must be serialised by the caller.
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that
 * call outside stream capture.
 */
int syn_gemm_producer_static(const syn_gemm_desc* desc, syn_stream_t stream);

/* Test hook of syn_gemm_producer_static: copies the first `count` words of the current device's static counter
 * array to host memory (a synchronous hipMemcpy; allocates nothing).  No counterpart in the reference. */
int syn_gemm_static_counters_peek(int32_t* host_out, int32_t count);

/*
 * A GEMM in both roles: the producer above that, before the first tile of a wave, also waits
 * (acquire) until wait_flags[wait_signal_offsets[wave]] == 1 where that index is >= 0 - e.g. the
 * GEMM of a tensor-parallel layer whose A arrives by all-gather and whose C leaves by
 * reduce-scatter.  `wait_flags` (device, 8-byte words) is a flag array of its own: `desc->flags`
 * stays what the launch SETS.  Replaces the kernel the reference's transformer generates when a
 * source carries consumer and producer annotations at once
 * (syncopate/computation/transform/transformer.py:759-901, both passes applied).
 */
int syn_gemm_consumer_producer(const syn_gemm_desc* desc, const uint64_t* wait_flags,
                               const int32_t* wait_signal_offsets, syn_stream_t stream);

/*
 * Remote bindings of a GEMM launch: per wave, A is read from a peer's shard and / or the C
 * tile goes into a peer's buffer instead of the local one.  Counterpart of the reference's
 * dl.symm_at(ptr, target_rank) rebinding: kernel_gemm_ag_read_remote
 * (syncopate/computation/gemm/template_ag.py:43-187: A rows of wave w come from
 * a_peers[a_target_rank[w]] at the wave-local row, C is written at the global row),
 * kernel_gemm_rs_producer_persistent (template_rs.py:37-209: the C tile is atomically added
 * into c_peers[c_target_rank[w]] at the wave-local row) and the generated form with
 * target_rank / dst_offsets arguments (transform/transformer.py:1158-1178,
 * tests/test_gemm_rs_direct_reduce.py:166-189).  On one GPU the peers are buffers of the same
 * process; on a node they are peer-mapped allocations.
 */
typedef struct syn_gemm_remote {
    const void* const* a_peers;     /* device array of pointers to [rows, K] shards, or NULL   */
    const int32_t* a_target_rank;   /* device int32[num_waves]: index into a_peers             */
    void* const* c_peers;           /* device array of pointers to peer C buffers, or NULL     */
    const int32_t* c_target_rank;   /* device int32[num_waves]: index into c_peers             */
    const int32_t* c_dst_offsets;   /* device int32[num_waves, 2]: {row, col} of the wave's
                                       region inside the peer C, in elements                   */
    int32_t c_ld;                   /* row length of a peer C buffer (multiple of 4)           */
    int32_t c_atomic_add;           /* 1: add into the peer C (packed 16-bit float atomics),
                                       0: store                                                */
    const int32_t* k_ranges;        /* device int32[num_waves, 2] or NULL: {first k, count} of
                                       the part of K a wave contracts over, multiples of 64
                                       (split-K waves: the generated GEMM with a K range axis,
                                       tests/computation/transform/examples/example_splitk_gemm.py:
                                       36-112, consumer of tests/test_all2all_gemm.py:113-160);
                                       needs c_atomic_add and a zeroed C                       */
} syn_gemm_remote;

/*
 * The consumer walk (flags honoured where a wave has one) with the bindings above.  desc->a
 * may be NULL when a_peers is given, desc->c when c_peers is.  Default pipeline only.
 */
int syn_gemm_remote_binding(const syn_gemm_desc* desc, const syn_gemm_remote* remote,
                            syn_stream_t stream);

/*
 * Host-only check of a GEMM wave table against the operand shapes, block
 * sizes and flag-array length; the launch entry points cannot do it because
 * the tables they get live in device memory.  All pointers are HOST pointers.
 * Returns 0, SYN_EINVAL or SYN_ERANGE.  No reference counterpart: the
 * reference launches unchecked (template.py:177-185 asserts shapes only).
 *
 * CALLERS FROM C: syn_gemm_consumer / _producer / _consumer_producer /
 * _remote_binding and syn_attn_fwd do NOT validate wave tables (they are in
 * device memory); a table that names rows beyond an operand or a flag beyond
 * its array makes the kernel read or write out of bounds.  Call
 * syn_gemm_check_waves / syn_attn_check_waves on the host copy of every new
 * table before its first launch, as the Python launchers do.
 */
int syn_gemm_check_waves(const int32_t* wave_sizes, const int32_t* wave_offsets,
                         const int32_t* signal_offsets, int32_t num_waves,
                         int32_t M, int32_t N, int32_t K,
                         int32_t block_m, int32_t block_n, int32_t block_k,
                         int64_t cum_tiles, int64_t num_flags);

/* Number of workgroups syn_gemm_* will launch: min(num_sms, tiles)
 * (template.py:193-197). */
int syn_gemm_grid(int64_t cum_tiles, int32_t M, int32_t N, int32_t block_m,
                  int32_t block_n, int32_t num_sms);

/*
 * Chunked ring reduce of GEMM+RS:
 *   out[m, n] = local[rank*Mr + m, n] + sum_{i=1..W-1} recv[(rank+i) % W, m, n]
 * added left to right.  acc_mode 0 rounds the running sum to the element type
 * after every add (what the reference's `accum += data` on dtype tensors does,
 * tests/test_gemm_rs.py:64-70); acc_mode 1 keeps the running sum in fp32 and
 * rounds once.  recv is [W, Mr, N] (slot `rank` is never read), local is
 * [W*Mr, N], out is [Mr, N]; Mr*N must be a multiple of 8.
 * Replaces kernel_ring_reduce_tma / ring_reduce_tma (tests/test_gemm_rs.py:22-121).
 */
int syn_ring_reduce(const void* recv, const void* local, void* out,
                    int32_t world, int32_t rank, int64_t rows_per_rank, int64_t N,
                    int32_t dtype, int32_t acc_mode, syn_stream_t stream);
/* The same with the W blocks of recv `recv_block_stride` elements apart (>= Mr*N, a multiple of 8)
 * instead of back to back: what a [W, Mr, N] view of a padded receive buffer hands over
 * (torch's input.stride(0) in ring_reduce_tma's call, tests/test_gemm_rs.py:75-121).  Eight
 * blocks of exactly 16 MiB start in the same DRAM banks and channels; 4 KiB of padding per block
 * is worth 8 % of read bandwidth. */
int syn_ring_reduce_strided(const void* recv, int64_t recv_block_stride, const void* local, void* out,
                            int32_t world, int32_t rank, int64_t rows_per_rank, int64_t N,
                            int32_t dtype, int32_t acc_mode, syn_stream_t stream);

/*
 * Chunked-KV flash attention forward.  One workgroup per tile id; tile id ->
 * (wave, z, h, q block, kv block range) exactly as the reference's wave lookup
 * (syncopate/computation/attn/template.py:39-44,80-121; generated form
 * transformer.py:555-660).  Table rows are {Z, H, Q, KV} sizes/offsets in
 * ELEMENTS along Q and KV (divided by block_m / block_n in the kernel) and
 * cum_wave_sizes is the inclusive prefix sum of Z*H*Q elements.  Each program
 * computes its partial (O, lse2) with a base-2 online softmax and merges it
 * into o / lse under a per-q-block lock (template.py:307-361).  With
 * causal != 0, kv blocks wholly above the diagonal are skipped and the
 * diagonal block is masked (col > row); q and kv positions are global
 * sequence positions, so it needs Sq == Skv indexing (q row i attends kv <= i).
 * lse is fp32 [Z, H, Sq] (base-2 log-sum-exp), lock and first are zeroed
 * int32 [Z, H, Sq / block_m] scratch owned by the caller.
 */
typedef struct syn_attn_desc {
    const void* q;                  /* (z, h, q row, d), see *_strides                    */
    const void* k;                  /* (z, h, kv row, d)                                  */
    const void* v;                  /* (z, h, kv row, d)                                  */
    void* o;                        /* (z, h, q row, d)                                   */
    float* lse;                     /* [Z, H, Sq]                                         */
    int32_t* lock;                  /* [Z, H, Sq/block_m], zeroed; left in an unspecified state      */
    int32_t* first;                 /* [Z, H, Sq/block_m], zeroed                         */
    uint64_t* flags;
    const int32_t* wave_offsets;    /* device, [num_waves, 4]                             */
    const int32_t* wave_sizes;      /* device, [num_waves, 4]                             */
    const int32_t* cum_wave_sizes;  /* device, [num_waves]                                */
    const int32_t* signal_offsets;  /* device, [num_waves]                                */
    int32_t* visit_log;             /* optional device int32[num_tiles, 8]:
                                       {wave, z, h, q_block, kv_lo, kv_hi, signal, program}      */
    int32_t* status;                /* optional device int32[SYN_STATUS_WORDS]            */
    int32_t num_waves;
    int32_t Z, H, Sq, Skv, D;
    int32_t dtype;
    int32_t block_m, block_n;
    int32_t causal;
    int32_t num_programs;           /* persistent grid: workgroup b runs tiles b, b+grid, ...;
                                       <= 0 launches one workgroup per tile as the reference */
    float sm_scale;
    int64_t cum_tiles;              /* total Z*H*Q elements over all waves                */
    int64_t spin_timeout_us;
    /* element strides {batch, head, row} of q, k, v and o; d is contiguous.  All zero selects
       the contiguous [Z, H, S, D] layout of the reference's bhsd kernels
       (tests/computation/transform/examples/example_attn.py); {S*H*D, D, H*D} is its bshd
       layout (example_attn_bshd.py).  Strides must be multiples of 8 elements.            */
    int64_t q_strides[3];
    int64_t k_strides[3];
    int64_t v_strides[3];
    int64_t o_strides[3];
    int32_t* counters;              /* optional device int32[num_waves], zeroed: producer form (the
                                       generated launcher's counter_ptr, transform/transformer.py:
                                       880-901, 1125-1137): no flag is waited for; every finished
                                       tile bumps counters[wave] and the tile that completes a wave
                                       (Z*H*Q blocks of it) sets flags[signal_offsets[wave]] to 1   */
    int32_t options;                /* SYN_ATTN_* bits                                                */
    const uint64_t* wait_flags;     /* with counters only, both or neither: a second flag array and the   */
    const int32_t* wait_signal_offsets; /* index per wave (-1: none) this launch WAITS for before it reads
                                       a wave's K and V, while it sets `flags` as a producer - the
                                       transform pass with enable_consumer and enable_producer
                                       (consumer_signal_ptr / consumer_signal_offsets beside the
                                       producer's, transformer.py:1077-1123,
                                       tests/test_all2all_attn_all2all.py:192-210)                    */
    const int32_t* work_list;       /* with SYN_ATTN_WORK_LIST, else NULL: device int32: num_programs + 1 entry
                                       offsets, then the entries (see SYN_ATTN_WORK_LIST)              */
} syn_attn_desc;

/* syn_attn_desc.options: one workgroup of eight wavefronts takes two consecutive q blocks (tiles
 * 2i and 2i + 1) and runs them half a kv block apart, so that the softmax of one overlaps the
 * matrix products of the other and both read K and V from the same LDS blocks.  No counterpart in
 * the reference (one program per tile there); results and merge protocol are the same.  The
 * caller vouches that every wave holds an even number of q blocks (and, with `causal`, that every wave's q and
 * kv ranges begin at even blocks); not with `counters`. */
#define SYN_ATTN_PAIR_Q_BLOCKS 1u
/* workgroup b takes tile (b % 8) * (grid / 8) + b / 8 instead of tile b: the workgroups of one XCD
 * then work on consecutive tiles - the q blocks of one head - and that head's K and V pass through
 * one L2 instead of eight.  The visit log records the program each tile ran on either way. */
#define SYN_ATTN_XCD_REMAP 2u
/* with SYN_ATTN_PAIR_Q_BLOCKS: the caller vouches that every wave lists the same (z, h, q) ranges
 * (the waves differ in their kv range and flag only, as in the all-gather attention) and passes
 * num_programs = the number of q block pairs of one wave.  Program b's tiles are then pair b of
 * wave 0, of wave 1, ... in this order - the same programs and the same order as without the
 * option - and the kernel walks on from one wave's kv range into the next one's behind that wave's
 * flag, with the running maxima, sums and output in registers: every q block is written once, and
 * neither `lock` nor a stored partial result is read.  A table or grid that is not of that shape
 * ends the launch with SYN_STATUS_BAD_CHAIN in `status`.  No counterpart in the reference. */
#define SYN_ATTN_CHAIN_Q_BLOCKS 4u
/* the attention kernels' form of SYN_GEMM_ACQUIRE_ALWAYS: the acquire fence behind every flag wait, for callers
 * who cannot promise that K and V are not read on the device before a chunk's flag and that no flag is raised
 * twice during the launch (the reference always acquires: dl.wait, attn/template.py:90-96) */
#define SYN_ATTN_ACQUIRE_ALWAYS 8u
/* with SYN_ATTN_PAIR_Q_BLOCKS: `work_list` says which program visits which tiles, in which order.  The tile ->
 * (wave, z, h, q block, kv range) mapping stays the table's (and the reference's); what the list chooses is the
 * part the reference leaves to the hardware scheduler - which program runs a tile - and, beyond it, that a
 * program which visits the same pair of q blocks several times in a row keeps the running maxima, sums and output
 * in registers from one visit to the next (a SEGMENT) and merges into the output once.  Layout: words
 * [0, num_programs] are offsets into the entries that follow at work_list + num_programs + 1; program b makes the
 * visits entries[offset[b]] .. entries[offset[b + 1] - 1] in that order.  An entry is a pair index (tiles 2 * pair and
 * 2 * pair + 1 of the table) in SYN_ATTN_WORK_PAIR_MASK, SYN_ATTN_WORK_CONTINUES when the next entry visits the same
 * (z, h, q blocks) and continues the segment, and - on a segment's first entry - SYN_ATTN_WORK_SOLE_WRITER when no
 * other segment of the launch writes these q blocks (they are then stored without taking their locks).  Every
 * visit of the table appears exactly once; under `causal` the visits that lie wholly above the diagonal may be
 * left out (they add nothing; listed, they are logged in the visit log and skipped) and must not be part of a
 * segment, and every wave's q and kv ranges begin at even blocks.  num_programs is the grid.  Flags are waited for
 * visit by visit, in list order: a program's entries should follow the order in which their waves arrive.
 * syn_attn_check_work_list (HOST pointers) checks all of this; the kernel trusts a list that passed and ends a
 * launch whose list breaks a segment's promise with SYN_STATUS_BAD_CHAIN.  No counterpart in the reference. */
#define SYN_ATTN_WORK_LIST 16u
#define SYN_ATTN_WORK_PAIR_MASK 0x0fffffff
#define SYN_ATTN_WORK_CONTINUES 0x10000000
#define SYN_ATTN_WORK_SOLE_WRITER 0x20000000
int syn_attn_check_work_list(const int32_t* wave_offsets, const int32_t* wave_sizes, const int32_t* cum_wave_sizes,
                             int32_t num_waves, int32_t block_m, int32_t block_n, int32_t causal,
                             const int32_t* work_list, int64_t work_list_words, int32_t num_programs,
                             int32_t require_masked_visits);
/* syn_attn_fwd trusts its tables: pass them through syn_attn_check_waves first.  (A real wave behind a zero
 * row of padding, which the check rejects, would never be selected by the wave lookup.) */
int syn_attn_fwd(const syn_attn_desc* desc, syn_stream_t stream);

/* Host-only check of an attention wave table (HOST pointers). */
int syn_attn_check_waves(const int32_t* wave_offsets, const int32_t* wave_sizes,
                         const int32_t* cum_wave_sizes, const int32_t* signal_offsets,
                         int32_t num_waves, int32_t Z, int32_t H, int32_t Sq, int32_t Skv,
                         int32_t block_m, int32_t block_n, int64_t cum_tiles,
                         int64_t num_flags);

/*
 * Stream-side primitives of the single-GPU producer; counterparts of the
 * reference runtime's cudaMemcpyAsync / cuStreamWriteValue / cuStreamWaitValue
 * calls (syncopate/communication/comm_runtime/communication_context.py:129-160).
 */
int syn_copy_async(void* dst, const void* src, int64_t nbytes, syn_stream_t stream);
/* The same copy done by `num_blocks` 256-thread workgroups with streaming (non-temporal)
 * loads and stores; nbytes and both pointers must be multiples of 16.  Counterpart of the
 * reference's SM-driven copy (comm_runtime/non_tma_persistent_copy.py:191-304) for the
 * contiguous case. */
int syn_copy_kernel_async(void* dst, const void* src, int64_t nbytes, int32_t num_blocks,
                          syn_stream_t stream);
/* Element kinds of syn_box_copy_async: float types (sums allowed) and plain sizes (copies only) */
#define SYN_ELEM_BF16 0
#define SYN_ELEM_FP16 1
#define SYN_ELEM_FP32 2
#define SYN_ELEM_1B 3
#define SYN_ELEM_2B 4
#define SYN_ELEM_4B 5
#define SYN_ELEM_8B 6
/* A chunk copy that sets the chunk's flag itself (`*flag = value` once every byte has landed):
 * one kernel where the reference issues a copy and a stream write
 * (communication_context.py:129-150), with at most `num_blocks` workgroups of 1024 threads.
 * `ticket` is one zeroed 32-bit word of device memory that the copies of ONE stream share: the
 * kernel counts its workgroups in it and leaves it zero again.  16-byte alignment as for
 * syn_copy_kernel_async. */
int syn_copy_flag_async(void* dst, const void* src, int64_t nbytes, uint64_t* flag, uint64_t value,
                        uint32_t* ticket, int32_t num_blocks, syn_stream_t stream);
/* A list of such copies as ONE kernel: record k is copied, then *flag = value, in list order, by at
 * most `num_blocks` workgroups of 1024 threads that walk the list (a workgroup goes on to the next
 * record while others still finish the last one).  `ops` is a DEVICE array of `count` records
 * (every dst / src 16-byte aligned, `bytes16` = length in 16-byte units), `tickets` `count` zeroed
 * 32-bit words of device memory, left zero again.  `delay_ticks` > 0 lets that many ticks of the
 * device's wall clock (100 MHz) pass in front of a record: a slow link.  A record whose `flag` is NULL is a piece
 * of a transfer in several pieces (the rows of a strided box): it is copied, and the flag of the next record that
 * has one covers it.  The data is stored through the L2, so no
 * kernel boundary - with its cache write-back and invalidate - falls into a consumer kernel that
 * runs beside the list.  Replaces a whole stream of cudaMemcpyAsync + cuStreamWriteValue pairs of the
 * reference's executor (communication_context.py:129-150). */
typedef struct syn_copy_flag_op {
    void* dst;
    const void* src;
    int64_t bytes16;
    uint64_t* flag;
    uint64_t value;
    int64_t delay_ticks;
} syn_copy_flag_op;
int syn_copy_flag_list_async(const syn_copy_flag_op* ops, int32_t count, uint32_t* tickets, int32_t num_blocks,
                             syn_stream_t stream);
/* What syn_box_copy_async does with the destination */
#define SYN_BOX_COPY 0            /* dst = src */
#define SYN_BOX_ADD_ATOMIC 1      /* dst += src by atomic adds: several senders may add into one
                                     destination at a time (the reference's tl.atomic_add) */
#define SYN_BOX_ADD_EXCLUSIVE 2   /* dst += src by plain read-modify-write, several times faster:
                                     for a destination that has one writer at a time */
/* Copy or accumulate (one rounding in the element type per addition) a box of 1..5 dimensions
 * with at most `num_blocks` 1024-thread workgroups.  `shape` and the strides count elements; the
 * last dimension is contiguous (stride 1) on both sides.  Accesses are 16 bytes wide when row
 * length, base addresses and strides allow, narrower otherwise, down to one element.  Counterpart
 * of the reference's SM-driven copies persistent_naive_copy_last_contig /
 * persistent_tma_copy_last_contig (comm_runtime/non_tma_persistent_copy.py:106-304,
 * tma_persistent_copy.py), which replay SMCopyOp (communication_context.py:161-189); five
 * dimensions at most there too (MAX_RANK). */
int syn_box_copy_async(void* dst, const void* src, int32_t ndim, const int64_t* shape,
                       const int64_t* src_strides, const int64_t* dst_strides, int32_t elem_kind,
                       int32_t reduce_mode, int32_t num_blocks, syn_stream_t stream);
int syn_flag_set(uint64_t* flag, uint64_t value, syn_stream_t stream);
/* The same flag write as a stream memory operation (hipStreamWriteValue64, the counterpart of the
 * reference's cuStreamWriteValue, communication_context.py:150): no kernel, so no compute unit, and none
 * of the cache maintenance a kernel boundary brings.  For streams driven from the host: recorded into a
 * HIP graph such a write has been seen to take effect on the first replay only. */
int syn_flag_write_value(uint64_t* flag, uint64_t value, syn_stream_t stream);
int syn_flag_wait(const uint64_t* flag, uint64_t value, int64_t spin_timeout_us,
                  int32_t* status, syn_stream_t stream);
/* Occupy the stream for about `us` microseconds with one sleeping wavefront
 * (models a slow link in front of a chunk copy). */
int syn_delay_us(int64_t us, syn_stream_t stream);

/* A stream whose kernels run only on the compute units whose bits are set in `mask` (`words`
 * 32-bit words, bit i of the device: XCD i % 8, and within the XCD the compute units in turn over
 * its shader engines), with a hardware queue of its own.  Two streams with disjoint masks split
 * the device between communication and compute kernels: the counterpart of the reference's green
 * contexts (comm_runtime/split_green_ctx.py:121-215, used when CommInfo.need_green_ctx is set,
 * communication_context.py:66-72).  Destroy the stream with syn_stream_destroy when its work is
 * done. */
int syn_stream_create_cu_mask(const uint32_t* mask, uint32_t words, syn_stream_t* stream);
int syn_stream_destroy(syn_stream_t stream);
/* Launch `workgroups` workgroups that each record where they ran: out[2 b] = hardware id word
 * (compute unit, shader array, shader engine in bits 8..15), out[2 b + 1] = XCD id, and stay for
 * `dwell` short sleeps so that the grid spreads over every compute unit the stream may use.
 * No counterpart in the reference; it is how a partition of the device is checked. */
int syn_where_async(uint32_t* out, int32_t workgroups, int32_t dwell, syn_stream_t stream);

/* Measurement aid, no counterpart in the reference: `workgroups` workgroups of four wavefronts
 * each run `iters` rounds of 64 v_mfma_f32_32x32x16_bf16 per wavefront (the GEMM kernels' 4 x 4
 * accumulator pattern) on register-resident operands - no LDS, no memory.  pattern 0: zero
 * operands, 1: all ones, 2: pseudo-random N(0, 0.02)-like values.  flop = workgroups * 4 * iters *
 * 64 * 32768.  sink: device float[workgroups * 256].  The rate with pattern 2 is what the matrix
 * pipes sustain under the board's power limit when operand bits toggle.  pattern + 4: the same
 * operands and flop on 128 v_mfma_f32_16x16x32_bf16 per round (8 x 8 accumulators), the form of
 * the 256x256 tile's K loop. */
int syn_probe_mfma_rate(float* sink, int32_t workgroups, int32_t iters, int32_t pattern,
                        syn_stream_t stream);

/* Measurement aid, no counterpart in the reference: `workgroups` workgroups of 256 lanes read
 * `streams` (1 or 8) streams of `stream_bytes` each (a multiple of 16384), `stride_bytes` apart
 * from `base`, in the chunked reduce's access pattern (four 16-byte groups per lane and pass, every
 * load of a pass issued before the first is used, non-temporal) and write nothing.
 * bytes read = streams * stream_bytes.  sink: device memory of 16 bytes per workgroup.  The rate is
 * what the memory system gives the reduce's reads at that placement of its operands. */
int syn_probe_read_streams(const void* base, int64_t stream_bytes, int64_t stride_bytes, int32_t streams,
                           int32_t workgroups, void* sink, syn_stream_t stream);
/* The same eight streams (`stream_bytes` a multiple of 32768) read the way the chunked reduce walks a chunk of at
 * least 16 MiB per stream: a workgroup takes eight consecutive 4 KB blocks of every stream and reads, in step t,
 * block t - i of stream i - streams that lie a multiple of the DRAM interleave apart are then never asked for the
 * same bank at the same time. */
int syn_probe_read_streams_skewed(const void* base, int64_t stream_bytes, int64_t stride_bytes, int32_t workgroups,
                                  void* sink, syn_stream_t stream);

/* Measurement aid, no counterpart in the reference: the slot of the paired attention kernel, piece by piece.
 * `workgroups` workgroups of eight wavefronts (two per SIMD) run `iters` slots; in a slot wavefronts 0-3 run that
 * kernel's 64 MFMAs 32x32x16 and wavefronts 4-7 one softmax pass over 64 scores per lane, then all meet at a
 * barrier.  `what` is a sum of: 1 the products run, 2 the softmax runs (a half that does not run only joins the
 * barriers), 4 the products' K and V fragments come from LDS through the kernel's reads (else register
 * operands), 8 every wavefront issues four 1 KB LDS-DMA fills per slot from `pool`, 16 (with 4) the first
 * fragments of a phase are asked for in the tail of the previous one, 32 pseudo-random operands instead of a
 * constant, 64 a workgroup's fills read a region of its own (L2 misses; else all workgroups read the same 32 KB
 * piece per slot: L2 hits but for the first reader of an XCD), 128 (with 1) every 32x32x16 MFMA is replaced by two
 * 16x16x32 MFMAs that share its A operand - the same flop and LDS reads, the form attn_pair_kernel uses.  pool: device memory of at least 65536 * workgroups + 32 MiB bytes, 16-byte aligned.  sink: device
 * float[512 * workgroups].  cycles: device int64[2], the shader-clock cycles workgroup 0 spent in the loop
 * (wavefront 0, wavefront 4); with the launch's duration they give the clock the device held.
 * matrix-pipe cycles per slot: 2048. */
int syn_probe_attn_slot(const void* pool, int64_t pool_bytes, int32_t workgroups, int32_t iters, int32_t what,
                        float* sink, int64_t* cycles, syn_stream_t stream);

/* Library/ABI version: major*10000 + minor*100 + patch. */
int syn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SYNCOPATE_HIP_H */
