/*
 * C ABI of libfa_mi355x.so: FlashAttention-2 forward for AMD MI355X (gfx950).
 *
 * This is the native boundary that the `flash_attn` Python API binds.  It replaces the three
 * forward entry points of the reference's pybind11 module `flash_attn_2_cuda`
 * (csrc/flash_attn/flash_api.cpp:1281-1288).  Plain pointers and sizes only: no torch types, no
 * allocation, no retained state.  Every buffer is owned by the caller; kernels are enqueued on the
 * given HIP stream and the call returns without synchronising.
 *
 * Return value of every int function: 0 on success, non-zero on error; fa_last_error() then
 * holds a message (thread-local).  The library never aborts the process.
 */
#ifndef FA_MI355X_H
#define FA_MI355X_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_DTYPE_FP16 0
#define FA_DTYPE_BF16 1
#define FA_DTYPE_FP32 2   /* rotary tables only */

#define FA_MAX_SPLITS 128

/*
 * Problem description.  POD mirror of the reference's Flash_fwd_params
 * (csrc/flash_attn/src/flash.h:24-130), with 64-bit element strides so that tensors of 2^31
 * elements and more are addressable.
 *
 * Layouts (all strides in ELEMENTS, last dimension contiguous):
 *   q      (b, seqlen_q, h,   d)   or packed (total_q, h, d)   when cu_seqlens_q != NULL
 *   k, v   (b_k, seqlen_k, h_k, d) or packed (total_k, h_k, d) when cu_seqlens_k is cumulative
 *   o      like q
 *   softmax_lse  (b, h, seqlen_q) fp32, natural log; +inf for a row that sees no key
 *   o_accum      (num_splits, b, h, seqlen_q, d_rounded) fp32, d_rounded = d rounded up to 32
 *   lse_accum    (num_splits, b, h, seqlen_q) fp32   (scratch of the call: slots that hold no keys may be left
 *                                                    unwritten)
 * Masking is bottom-right aligned: query i sees key j iff
 *   i + sk - sq - window_left <= j <= i + sk - sq + window_right and j < sk,
 * a negative window bound meaning unbounded; is_causal forces window_right = 0.
 */
typedef struct fa_fwd_params {
    const void *q, *k, *v;
    void *o;
    float *softmax_lse;
    float *o_accum;   /* needed when the resolved split count is > 1 (see fa_plan_splits) */
    float *lse_accum;

    /* new keys/values appended to the cache before attention (fa_fwd_kvcache only), or NULL:
     * (b, seqlen_knew, h_k, d) */
    const void *k_new, *v_new;
    /* rotary tables (seqlen_ro, rotary_dim/2) in the q dtype, contiguous, or NULL */
    const void *rotary_cos, *rotary_sin;

    const int32_t *cu_seqlens_q;    /* (b+1) prefix sums, or NULL for a dense batch */
    const int32_t *cu_seqlens_k;    /* (b+1) prefix sums if is_seqlens_k_cumulative, else (b)
                                       per-batch key lengths (cache_seqlens), or NULL */
    const int32_t *cache_batch_idx; /* (b) row of k/v used (and updated) for batch i, or NULL */
    int32_t *work_counter;          /* optional: work_counter_len (>= FA_WORK_COUNTER_WORDS) int32 words of
                                       device memory, 8-byte aligned.  The first FA_WORK_COUNTER_WORDS words are
                                       the ticket and exit counters of the ticket-scheduled kernels; every
                                       launch that completes leaves them zero, and a launch treats whatever
                                       else it finds there (a launch that was torn down mid-way, words the
                                       caller never cleared) as zero too: each call tags its counters with a
                                       number of its own, so no clearing launch is needed (allocate them zeroed
                                       all the same).
                                       When set, split-KV decode launches run as a persistent kernel whose
                                       workgroups draw (batch, kv head, key chunk) items from a ticket and
                                       whose item that reaches the new rows appends them to the cache (no
                                       append launch); fa_fwd_kvcache launches of a few query positions (or one
                                       position on more than 16 grouped heads) over per-batch cache lengths run
                                       the tiled kernel under the same ticket schedule.  Words past the first
                                       FA_WORK_COUNTER_WORDS are scratch with no required contents: when there
                                       are at least
                                       fa_work_list_words(p) words, fa_varlen_fwd first builds its work
                                       list there on the device (sequences by falling length, no empty
                                       workgroups between working ones).  Must not be shared by calls
                                       that overlap on the GPU.  NULL: one workgroup per chunk, a
                                       separate append launch, arithmetic work order. */

    int64_t q_batch_stride, q_row_stride, q_head_stride;
    int64_t k_batch_stride, k_row_stride, k_head_stride;
    int64_t v_batch_stride, v_row_stride, v_head_stride;
    int64_t o_batch_stride, o_row_stride, o_head_stride;
    int64_t knew_batch_stride, knew_row_stride, knew_head_stride;
    int64_t vnew_batch_stride, vnew_row_stride, vnew_head_stride;

    int32_t b;            /* batch size of q */
    int32_t h, h_k;       /* query heads, key/value heads (h % h_k == 0) */
    int32_t seqlen_q;     /* rows per batch entry; max_seqlen_q for packed input */
    int32_t seqlen_k;     /* keys per batch entry (cache capacity); max_seqlen_k for packed input */
    int32_t seqlen_knew;  /* rows of k_new / v_new, 0 if none */
    int32_t d;            /* head dimension, multiple of 8, <= 256 */
    int32_t rotary_dim;   /* 0 = no rotary; multiple of 16, <= d */

    int32_t window_left, window_right;
    int32_t is_causal;
    int32_t is_seqlens_k_cumulative;
    int32_t is_rotary_interleaved;
    int32_t num_splits;   /* request: 0 = library decides, 1 = never split, n = at most n chunks */
    int32_t dtype;        /* FA_DTYPE_* */
    float softmax_scale;

    /* Dropout on the attention probabilities (fa_fwd and fa_varlen_fwd; csrc/flash_attn/flash_api.cpp:
     * 99-107, 396-408).  p_dropout is the probability of DROPPING an entry, 0 = none.  The mask is a pure
     * function of (rng_state[0] = seed, rng_state[1] = offset, batch, head, row, key): the backward
     * regenerates it from the same two words.  The keep probability is quantised to 8 bits as in
     * the reference (:104).  With dropout the key range is never split (:380). */
    float p_dropout;
    const uint64_t *rng_state;   /* device memory, 2 words; required when p_dropout > 0 */
    /* Optional, for testing (the reference's return_softmax): (b, h, sdm_rows, sdm_cols) in the q
     * dtype, row-major, receives the softmax probability of every (row, key), negated where dropout
     * removed it, 0 outside the mask.  Unlike the reference's S_dmask (which is stored in the order
     * of its CUDA MMA fragments) entry [i][j] is plainly row i, key j. */
    void *s_dmask;
    int32_t sdm_rows, sdm_cols;  /* >= seqlen_q, >= seqlen_k */
    int32_t work_counter_len;    /* int32 words behind work_counter */
    int32_t reserved0;
} fa_fwd_params;

/* words the ticket-scheduled kernels need behind work_counter: two 64-bit counters (tickets drawn, workgroups
 * that have left), each (call tag << 32) | count */
#define FA_WORK_COUNTER_WORDS 4

/*
 * Words behind work_counter with which every launch of fa_varlen_fwd on these params (b, h, h_k, seqlen_q =
 * max_seqlen_q) can build its work list; FA_WORK_COUNTER_WORDS when the batch does not qualify (more than
 * 2048 sequences, or kv heads that do not spread evenly over the 8 XCDs).  No counterpart in the
 * reference, whose grid order is fixed (flash_fwd_launch_template.h:33-77).  Results do not depend on it.
 */
int64_t fa_work_list_words(const fa_fwd_params *p);

/*
 * Dense batch forward.  Replaces mha_fwd (csrc/flash_attn/flash_api.cpp:248-424): same masking
 * rules (seqlen_q == 1 disables causal, :296), same outputs (o and softmax_lse).  Splits the key
 * range when p->num_splits resolves to > 1 (then o_accum / lse_accum must be set).
 */
int fa_fwd(const fa_fwd_params *p, void *hip_stream);

/*
 * Packed variable-length forward.  Replaces mha_varlen_fwd (flash_api.cpp:426-585): cu_seqlens_q
 * and cu_seqlens_k are int32 prefix sums; softmax_lse is (b, h, max_seqlen_q) and rows beyond a
 * sequence's length are left unwritten (:527).  Never splits.
 */
int fa_varlen_fwd(const fa_fwd_params *p, void *hip_stream);

/*
 * KV-cache forward.  Replaces mha_fwd_kvcache (flash_api.cpp:1038-1279): optional append of
 * k_new/v_new at rows cache_seqlens[b] .. of cache row cache_batch_idx[b] (new keys rotated when
 * rotary tables are given, :763-852 of flash_fwd_kernel.h), q rotated on load (:854-891), then
 * attention over cache_seqlens[b] + seqlen_knew keys.  Mutates k and v in place.  With rotary tables and 96 or
 * more query rows, o holds the rotated q rows before the results land in it, but only when the address ranges
 * of q and o do not meet; when they do (o == q, or views of one tensor) the kernel that rotates while it loads
 * runs instead.  As in the reference, o may be q itself but must not overlap it in any other way.
 */
int fa_fwd_kvcache(const fa_fwd_params *p, void *hip_stream);

/*
 * fa_fwd_kvcache for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * mha_fwd_kvcache always allocates its split accumulators (flash_api.cpp:1241-1257).  Same arguments
 * and results as fa_fwd_kvcache, except that p->o_accum, p->lse_accum and p->work_counter are ignored:
 * the ticket words and the fp32 partial results of a split launch live in FA_NOALLOC_SCRATCH_BYTES of
 * device memory that the library itself holds on every GPU it runs on (a static device array, kept
 * until the process ends).  The call allocates and frees nothing.  A problem whose partials do not fit
 * (splits x b x h x seqlen_q x (4 + 4 x d rounded up to 32) bytes + 64 KiB of counters) is rejected with an error;
 * num_splits = 1 always fits.  All calls on one GPU share the array: calls that overlap in time on the
 * same GPU (two streams, two threads) race on it and must be serialised by the caller.  The first call
 * on a device looks the array's address up (hipGetSymbolAddress): make one call before capturing a
 * graph.
 */
#define FA_NOALLOC_SCRATCH_BYTES (48u << 20)
int fa_fwd_kvcache_noalloc(const fa_fwd_params *p, void *hip_stream);

/*
 * Resolves the split count the library will use for this problem, so that the caller can size
 * o_accum / lse_accum before the call (the reference does this inside mha_fwd / mha_fwd_kvcache,
 * flash_api.cpp:373-389, 1241-1257, with num_splits_heuristic :212-246; this library uses its
 * own rule for 256 CUs).  `api` is 0 for fa_fwd, 2 for fa_fwd_kvcache.  Writes the number of
 * partial slots (1..FA_MAX_SPLITS) to *num_splits: o_accum / lse_accum must hold that many.  The
 * subsequent call takes the SAME params (same num_splits request, same work_counter): it repeats
 * the same deterministic plan.
 */
int fa_plan_splits(const fa_fwd_params *p, int32_t api, int32_t *num_splits);

/*
 * The reference's own split-count rule, kept as a pure utility for callers that rely on it
 * (num_splits_heuristic, flash_api.cpp:212-246).
 */
int fa_num_splits_heuristic_reference(int32_t batch_nheads_mblocks, int32_t num_sms,
                                      int32_t num_n_blocks, int32_t max_splits);

/*
 * Writes {seed, offset} to the two 64-bit words at rng_state (device memory) from a one-thread kernel
 * on `hip_stream`: how the host side hands the dropout generator state to fa_fwd / fa_varlen_fwd
 * without a host-to-device copy.  Stands where the reference stores its Philox seed and offset into
 * rng_state inside the forward kernel (csrc/flash_attn/src/flash_fwd_kernel.h:1142-1148).
 */
int fa_set_rng_state(uint64_t *rng_state, uint64_t seed, uint64_t offset, void *hip_stream);

/*
 * Which attention kernel the calling thread's last successful forward launch used (fa_fwd, fa_varlen_fwd,
 * fa_fwd_kvcache, fa_fwd_kvcache_noalloc); 0 before any.  Host-side bookkeeping only: no device work, no
 * synchronisation.  No counterpart in the reference, whose dispatch (run_mha_fwd, flash_api.cpp:194-204, and
 * flash_fwd_launch_template.h:140-336) is not observable either; tests use it to assert that a case written for
 * one kernel still reaches it when the dispatch thresholds move.
 *   bits 0-7   FA_KERNEL_* below
 *   bit  8     the dropout instantiation ran
 *   bit  9     the key range was split (partial results + merge launch)
 *   bits 16-31 head dims the products ran over (the bucket, or less: 96 on the 128 bucket, 160 / 192 / 224 on 256)
 */
#define FA_KERNEL_NONE 0
#define FA_KERNEL_TILED 1               /* general tiled kernel, one workgroup per row block (and key chunk) */
#define FA_KERNEL_TILED_TICKETS 2       /* the same under the ticket schedule */
#define FA_KERNEL_PIPELINED 3           /* software-pipelined 128-row kernel, head dims up to 128 */
#define FA_KERNEL_PINGPONG 4            /* 8-wave 256-row kernel, head dim 65-128 */
#define FA_KERNEL_WIDE 5                /* head dims 129-256, whole head dim per wave */
#define FA_KERNEL_WIDE_PAIR 6           /* head dims 129-256, wave pairs */
#define FA_KERNEL_DECODE 7              /* up to 16 packed query rows, one workgroup per key chunk */
#define FA_KERNEL_DECODE_TICKETS 8      /* the same under the ticket schedule */
#define FA_KERNEL_PINGPONG_WIDE 9       /* 8-wave 128-row kernel, head dims 129-256 */
#define FA_KERNEL_PINGPONG_WIDE32 10    /* the same with 32 query rows per wave (256-row blocks), head dims 129-192 */
#define FA_KERNEL_FLAG_DROPOUT (1 << 8)
#define FA_KERNEL_FLAG_SPLIT (1 << 9)
int32_t fa_last_kernel(void);

/* Message of the last failure on the calling thread ("" if none). */
const char *fa_last_error(void);

/* Library version, (major << 16) | minor. */
int32_t fa_version(void);

/* sizeof(fa_fwd_params) as the library was compiled: lets a foreign-language binding verify its
 * mirror of the struct.  No counterpart in the reference (pybind11 passes tensors). */
int32_t fa_sizeof_params(void);

/*
 * Standalone rotary embedding: out[..., :rotary_dim] = x * cos + rotate_half(x) * sin per
 * (token, head) row, remaining columns copied through; math in fp32, one rounding to the dtype of
 * x.  Replaces the reference's Triton op apply_rotary (flash_attn/ops/triton/rotary.py:144-240)
 * behind apply_rotary_emb (flash_attn/layers/rotary.py:34-124): same arguments.
 *   x, out        (b, seqlen, h, d) with the strides below, or packed (total, h, d) when
 *                 cu_seqlens != NULL (then seqlen = max_seqlen); out may be x (in place)
 *   cos, sin      (seqlen_ro, rotary_dim/2), row stride cs_row_stride, dtype cs_dtype
 *   position of token t of batch entry i: t + (seqlen_offsets ? seqlen_offsets[i] : seqlen_offset);
 *                 positions outside the table leave the row unrotated
 *   interleaved   pairs (2i, 2i+1) instead of (i, i + rotary_dim/2)
 *   conjugate     rotate by -angle (the backward of the operation)
 * Any even rotary_dim <= d, any d, any strides, as the reference's op (flash_attn/ops/triton/rotary.py:176-208).
 * The memory-bound form with 16-byte accesses runs when rotary_dim is a multiple of 16, d and all strides are
 * multiples of 8 elements and x, out, cos, sin are 16-byte aligned; other shapes take an element-wise kernel.
 */
typedef struct fa_rotary_params {
    const void *x;
    void *out;
    const void *cos, *sin;
    const int32_t *cu_seqlens;       /* (b+1) or NULL */
    const int32_t *seqlen_offsets;   /* (b) or NULL */
    int64_t x_batch_stride, x_row_stride, x_head_stride;
    int64_t o_batch_stride, o_row_stride, o_head_stride;
    int64_t cs_row_stride;
    int32_t b, seqlen, h, d, rotary_dim, seqlen_ro, seqlen_offset;
    int32_t interleaved, conjugate;
    int32_t dtype;                   /* FA_DTYPE_FP16 / FA_DTYPE_BF16 */
    int32_t cs_dtype;                /* FA_DTYPE_FP16 / FA_DTYPE_BF16 / FA_DTYPE_FP32 */
} fa_rotary_params;

int fa_rotary(const fa_rotary_params *p, void *hip_stream);

/* sizeof(fa_rotary_params) as compiled, for foreign-language bindings (no reference counterpart). */
int32_t fa_sizeof_rotary_params(void);

/*
 * Backward pass: gradients of q, k, v given the gradient of the output.  Replaces the reference's
 * mha_bwd and mha_varlen_bwd (csrc/flash_attn/flash_api.cpp:609-832, 834-1036); the struct is the
 * POD counterpart of Flash_bwd_params (csrc/flash_attn/src/flash.h:134-175).
 *
 * Layouts as in fa_fwd_params: q, out, dout, dq are (b, seqlen_q, h, d) or packed (total_q, h, d)
 * with cu_seqlens_q; k, v, dk, dv are (b, seqlen_k, h_k, d) or packed (total_k, h_k, d) with
 * cu_seqlens_k.  softmax_lse is the forward's (b, h, seqlen_q) fp32 result (seqlen_q = max_seqlen_q
 * for packed input).  softmax_d is caller-provided work space AND a result, as in the reference:
 * (b, h, seqlen_q_rounded) fp32, seqlen_q_rounded >= seqlen_q, receiving rowsum(dout * out).
 * dk and dv are written at h_k heads: the sum over the query heads of a group happens inside the
 * kernel, no expanded buffer is needed.  Results are deterministic (no
 * atomics): dq is produced by one pass over query tiles, dk / dv by one pass over key tiles.
 */
typedef struct fa_bwd_params {
    const void *dout, *q, *k, *v, *out;
    const float *softmax_lse;
    void *dq, *dk, *dv;
    float *softmax_d;
    const int32_t *cu_seqlens_q;    /* (b+1) prefix sums, or NULL for a dense batch */
    const int32_t *cu_seqlens_k;    /* (b+1) prefix sums, or NULL for a dense batch */

    int64_t q_batch_stride, q_row_stride, q_head_stride;
    int64_t k_batch_stride, k_row_stride, k_head_stride;
    int64_t v_batch_stride, v_row_stride, v_head_stride;
    int64_t o_batch_stride, o_row_stride, o_head_stride;
    int64_t do_batch_stride, do_row_stride, do_head_stride;
    int64_t dq_batch_stride, dq_row_stride, dq_head_stride;
    int64_t dk_batch_stride, dk_row_stride, dk_head_stride;
    int64_t dv_batch_stride, dv_row_stride, dv_head_stride;

    int32_t b, seqlen_q, seqlen_k;  /* seqlen_* are the maxima for packed input */
    int32_t h, h_k, d;              /* d a multiple of 8, <= 256 */
    int32_t seqlen_q_rounded;       /* row pitch of softmax_d */
    float softmax_scale;
    int32_t is_causal;
    int32_t window_left, window_right;
    int32_t dtype;                  /* FA_DTYPE_* */
    float p_dropout;                /* as in the forward; 0 = none */
    const uint64_t *rng_state;      /* device memory, the forward's {seed, offset}; required when p_dropout > 0 */
} fa_bwd_params;

/* mha_bwd (flash_api.cpp:609-832): dense batch; cu_seqlens_* must be NULL. */
int fa_bwd(const fa_bwd_params *p, void *hip_stream);

/* mha_varlen_bwd (flash_api.cpp:834-1036): packed sequences; both cu_seqlens_* required. */
int fa_varlen_bwd(const fa_bwd_params *p, void *hip_stream);

/* sizeof(fa_bwd_params) as compiled into the library. */
int32_t fa_sizeof_bwd_params(void);

/*
 * Matrix-pipe microbenchmark (measurement aid; no counterpart in the reference): launches a kernel that
 * executes only independent v_mfma_f32_32x32x16_bf16 instructions on every SIMD of the device, `iters`
 * x 16 per wave, on random bf16 operands (random_operands != 0) or on zeros, and writes the number of
 * floating-point operations of the launch to *flops.  The caller times the launch on `hip_stream`.
 * `sink` is 4 bytes of device memory (never written in practice).
 */
int fa_mfma_peak(float *sink, int32_t iters, int32_t random_operands, int64_t *flops, void *hip_stream);
/* The same with the instruction shape chosen: 0 = v_mfma_f32_32x32x16_bf16 (fa_mfma_peak), 1 = v_mfma_f32_16x16x32_bf16,
 * twice as many instructions for the same flops.  On random operands the part is power-bound and the two differ. */
int fa_mfma_peak_shape(float *sink, int32_t iters, int32_t random_operands, int32_t shape, int64_t *flops, void *hip_stream);

/*
 * Memory microbenchmark (measurement aid; no counterpart in the reference): launches a kernel that reads
 * `bytes` (a multiple of 16, at a 16-byte aligned device address) once, with non-temporal loads
 * (nontemporal != 0) or ordinary ones, and writes nothing.  The caller times the launch on `hip_stream`.
 * `sink` is 4 bytes of device memory (never written in practice).
 */
int fa_hbm_read_peak(const void *src, int64_t bytes, int32_t nontemporal, void *sink, void *hip_stream);

/*
 * LDS microbenchmark (measurement aid; no counterpart in the reference): `workgroups` workgroups of `waves`
 * waves (1..16) each issue iters x 16 conflict-free ds_read_b128 instructions (1 KB per wave instruction) and
 * write the shader-clock cycles of that loop to cycles[workgroup] (device memory, `workgroups` x 8 bytes);
 * *bytes_per_workgroup receives the LDS bytes one workgroup read.  bytes / cycles is the LDS read rate of a
 * CU in bytes per clock when one workgroup runs per CU.  `sink` is 4 bytes of device memory (never written).
 */
int fa_lds_read_peak(uint64_t *cycles, int32_t workgroups, int32_t waves, int32_t iters, int64_t *bytes_per_workgroup,
                     void *sink, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* FA_MI355X_H */
