// Host-side launcher declarations shared by the kernel translation units and the C ABI.
#pragma once
#include "fa_common.h"

namespace fa {
struct BwdKParams;
// What fa_last_kernel() reports: every attention launcher notes the kernel it enqueued (FA_KERNEL_* | flags |
// computed head dims << 16) for the calling thread.  Host-side only.
extern thread_local int32_t g_last_kernel;
inline int note_kernel(int launch_error, int id, bool dropout, bool split, int head_dims) {
    if (launch_error == 0) g_last_kernel = id | (dropout ? FA_KERNEL_FLAG_DROPOUT : 0) | (split ? FA_KERNEL_FLAG_SPLIT : 0) | (head_dims << 16);
    return launch_error;
}
#define FA_DECL_PREFILL(name) int name(const KParams& kp, hipStream_t stream);
FA_DECL_PREFILL(launch_prefill_bf16_64)
FA_DECL_PREFILL(launch_prefill_bf16_128)
FA_DECL_PREFILL(launch_prefill_bf16_256)
FA_DECL_PREFILL(launch_prefill_fp16_64)
FA_DECL_PREFILL(launch_prefill_fp16_128)
FA_DECL_PREFILL(launch_prefill_fp16_256)
#undef FA_DECL_PREFILL

int prefill_block_n(int d_bucket);   // key-tile length of the prefill kernel for a bucket
int prefill_block_m(int d_bucket);
// Query rows from which an unsplit launch without q rotary takes the pipelined / ping-pong kernels instead of
// the general tiled kernel (measured on 32..511 rows x 128..16384 keys, bf16, with and without a causal mask:
// head dims 64 and 128 +15-45 % from 128 rows on, 0..+28 % at 100-127 rows, -9..+14 % at 64 rows; head dim 256
// +25-57 % from 32 rows on, +50-100 % from 128).
inline int prefill_long_rows(int d_bucket) { return d_bucket > 128 ? 32 : 96; }

int launch_decode(const KParams& kp, hipStream_t stream);      // small-q split-KV kernel
int launch_combine(const KParams& kp, hipStream_t stream);     // merge of split partials
// k_new/v_new (+rotary) -> cache
int launch_append_kv(const KParams& kp, hipStream_t stream);
int launch_rotate_q(const KParams& kp, hipStream_t stream);     // q rows rotated to their positions -> rows of o
int launch_attn_probs(const KParams& kp, hipStream_t stream);  // s_dmask: signed softmax probabilities (testing)
int launch_rotary(const fa_rotary_params& p, hipStream_t stream);   // standalone rotary embedding
// Packed batches: builds the work list of a forward launch of `nblocks` workgroups with row blocks of
// `block_m` rows in kp.p.work_counter and sets kp.work_items, when the batch qualifies and the caller lent
// enough words (fa_work_list_words); otherwise leaves kp.work_items NULL.
int prepare_work_list(KParams& kp, int block_m, int64_t nblocks, hipStream_t stream);
int64_t work_list_words(const fa_fwd_params& p);    // words behind work_counter that make every packed launch qualify

#define FA_DECL_BWD(name) int name(const BwdKParams& kp, hipStream_t stream);
FA_DECL_BWD(launch_bwd_bf16_64)
FA_DECL_BWD(launch_bwd_bf16_128)
FA_DECL_BWD(launch_bwd_bf16_256)
FA_DECL_BWD(launch_bwd_fp16_64)
FA_DECL_BWD(launch_bwd_fp16_128)
FA_DECL_BWD(launch_bwd_fp16_256)
FA_DECL_BWD(launch_bwd_dot_bf16)    // rowsum(dO o O) -> softmax_d
FA_DECL_BWD(launch_bwd_dot_fp16)
#undef FA_DECL_BWD
}  // namespace fa
