// C ABI of libfa_mi355x.so: argument checks, mask normalisation, split planning and kernel
// dispatch.  Host-side counterpart of the reference's mha_fwd / mha_varlen_fwd / mha_fwd_kvcache
// bodies after tensor unpacking (csrc/flash_attn/flash_api.cpp:248-424, 426-585, 1038-1279) and of
// run_mha_fwd's dtype x head-dim dispatch (:194-204).
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>
#include <algorithm>
#include <mutex>
#include "fa_prefill.h"
#include "fa_bwd.h"
#include "fa_launch.h"

namespace fa {

static thread_local std::string g_err;
thread_local int32_t g_last_kernel = FA_KERNEL_NONE;
static int fail(const char* msg) { g_err = msg; return 1; }
static int fail_hip(int e, const char* where) {
    g_err = std::string(where) + ": " + hipGetErrorString((hipError_t)e);
    return 2;
}

int prefill_block_n(int db) { return db == 64 ? PrefillTile<64>::BN : db == 128 ? PrefillTile<128>::BN : PrefillTile<256>::BN; }
int prefill_block_m(int db) { return 128 * (db == 64 ? PrefillTile<64>::RB : db == 128 ? PrefillTile<128>::RB : PrefillTile<256>::RB); }
static int bucket(int d) { return d <= 64 ? 64 : d <= 128 ? 128 : 256; }

static const int kNumCU = 256;   // MI355X
#ifndef FA_DEC_SLOTS
#define FA_DEC_SLOTS 8192       // chunk slots per launch, one workgroup per chunk
#endif
#ifndef FA_DEC_SLOTS_P
#define FA_DEC_SLOTS_P 4096     // same for the persistent, ticket-scheduled kernel
#endif
#ifndef FA_DEC_SB
#define FA_DEC_SB 8
#endif
#ifndef FA_SPLIT_BELOW
#define FA_SPLIT_BELOW 256      // row blocks x heads x batch below which the tiled kernel's keys are split
#endif
#ifndef FA_TILE_SLOTS
#define FA_TILE_SLOTS 4096      // chunk slots per launch of the ticket-scheduled tiled kernel
#endif
#ifndef FA_TILE_MINLEN
#define FA_TILE_MINLEN 2048     // its shortest chunk (keys)
#endif
#ifndef FA_DEC_MINLEN
#define FA_DEC_MINLEN 512       // shortest chunk of the decode kernel (keys) once the launch fills the CUs
#endif

// The small-q streaming kernel packs seqlen_q x (h / h_k) rows into 16 MFMA columns.
static bool use_decode_kernel(const fa_fwd_params& p) {
    return p.cu_seqlens_q == nullptr && (int64_t)p.seqlen_q * (p.h / p.h_k) <= 16 && p.p_dropout == 0.f;
}

// One query position with more grouped q heads per kv head than the decode kernel packs into its 16 columns:
// the grouped heads of a kv head take the place of the query positions (the reference's
// seqlenq_ngroups_swapped, csrc/flash_attn/flash_api.cpp:1096-1104 for mha_fwd and :1265 for the kv-cache call).
// q and out are read as (batch, G rows, h_k heads, d) through their strides, so one workgroup per kv head
// serves all of its q heads and every K/V row is fetched once instead of G times (batch 16 x 64k keys, 32 q
// heads on 1 kv head: 1.6 ms -> 0.1 ms).  A single query row at the end of the keys sees all of them under a
// causal mask or a right window bound, so those are dropped; a left bound is not, and keeps the plain form.
// softmax_lse and the split accumulators need no change: (b, h, 1) and (b, h_k, G) index the same words.
static bool groups_as_rows(fa_fwd_params& q) {
    const int G = q.h_k > 0 ? q.h / q.h_k : 0;
    if (q.seqlen_q != 1 || G <= 16 || q.cu_seqlens_q || q.p_dropout != 0.f || q.s_dmask || q.window_left >= 0) return false;
    q.seqlen_q = G;
    q.h = q.h_k;
    q.q_row_stride = q.q_head_stride;
    q.q_head_stride *= G;
    q.o_row_stride = q.o_head_stride;
    q.o_head_stride *= G;
    q.is_causal = 0;
    q.window_right = -1;
    return true;
}

// A few query positions (speculative or chunked decoding) with grouped q heads: seqlen_q x G rows would be
// G separate row blocks of the tiled kernel, each streaming the kv head's K/V for a handful of rows.  Here the
// (position, grouped head) pairs of a kv head become the rows of one problem with h_k heads (KParams::pack_g):
// row = position * G + head within the group, so a workgroup serves up to 128 of them and K/V are fetched once
// (batch 64 x 16k keys, 64 q heads on 8 kv heads, 4 positions: 4.0 -> 0.8 ms).  Up to 16 rows the decode kernel
// packs them itself; from 128 positions on a row block is full without packing.  Returns G when it applies.
static int positions_and_groups_as_rows(fa_fwd_params& q, int64_t* q_head_stride, int64_t* o_head_stride) {
    const int G = q.h_k > 0 ? q.h / q.h_k : 0;
    if (q.seqlen_q <= 1 || q.seqlen_q >= 128 || G < 2 || (int64_t)q.seqlen_q * G <= 16 || q.cu_seqlens_q || q.p_dropout != 0.f || q.s_dmask)
        return 0;
    if (q_head_stride) *q_head_stride = q.q_head_stride;
    if (o_head_stride) *o_head_stride = q.o_head_stride;
    q.seqlen_q *= G;
    q.h = q.h_k;
    q.q_head_stride *= G;
    q.o_head_stride *= G;
    return G;
}

static int check_common(const fa_fwd_params* p) {
    if (!p) return fail("params is NULL");
    if (!p->q || !p->k || !p->v || !p->o || !p->softmax_lse) return fail("q, k, v, o and softmax_lse must be set");
    if (p->dtype != FA_DTYPE_FP16 && p->dtype != FA_DTYPE_BF16) return fail("FlashAttention only support fp16 and bf16 data type");
    if (p->b <= 0) return fail("batch size must be positive");
    if (p->d <= 0 || p->d > 256) return fail("FlashAttention forward only supports head dimension at most 256");
    if (p->d % 8 != 0) return fail("head dimension must be a multiple of 8 at the C boundary (pad on the host)");
    if (p->h <= 0 || p->h_k <= 0 || p->h % p->h_k != 0) return fail("Number of heads in key/value must divide number of heads in query");
    if (p->seqlen_q < 0 || p->seqlen_k < 0) return fail("sequence lengths must be non-negative");
    if (p->num_splits < 0 || p->num_splits > FA_MAX_SPLITS) return fail("num_splits > 128 not supported");
    // every global access is a 16-byte piece of a row
    const void* ptrs[] = {p->q, p->k, p->v, p->o, p->k_new, p->v_new};
    for (const void* q : ptrs) if ((uintptr_t)q % 16 != 0) return fail("q, k, v, o, k_new and v_new must be 16-byte aligned");
    const int64_t strides[] = {p->q_batch_stride, p->q_row_stride, p->q_head_stride, p->k_batch_stride, p->k_row_stride,
                               p->k_head_stride, p->v_batch_stride, p->v_row_stride, p->v_head_stride, p->o_batch_stride,
                               p->o_row_stride, p->o_head_stride, p->knew_batch_stride, p->knew_row_stride,
                               p->knew_head_stride, p->vnew_batch_stride, p->vnew_row_stride, p->vnew_head_stride};
    for (int64_t st : strides) if (st % 8 != 0) return fail("strides must be multiples of 8 elements (16-byte rows)");
    // the long-sequence kernels add a 32-bit lane byte offset (up to 64 rows) to a 64-bit tile base
    if (p->k_row_stride < 0 || p->k_row_stride >= ((int64_t)1 << 23) || p->v_row_stride < 0 || p->v_row_stride >= ((int64_t)1 << 23))
        return fail("k and v row strides must be below 2^23 elements");
    if (!(p->p_dropout >= 0.f && p->p_dropout < 1.f)) return fail("p_dropout must be in [0, 1)");
    if (p->p_dropout > 0.f && !p->rng_state) return fail("rng_state is required when p_dropout > 0");
    if (p->s_dmask && (p->sdm_rows < p->seqlen_q || p->sdm_cols < p->seqlen_k)) return fail("s_dmask is smaller than (seqlen_q, seqlen_k)");
    return 0;
}

// elements from the first to one past the last element of a (b, s, h, d) tensor with non-negative strides
static int64_t span_elems(int64_t b, int64_t s, int64_t h, int64_t d, int64_t bs, int64_t rs, int64_t hs) {
    return (b - 1) * bs + (s - 1) * rs + (h - 1) * hs + d;
}
static bool spans_overlap(const void* a, int64_t a_elems, const void* b, int64_t b_elems) {
    const uintptr_t a0 = (uintptr_t)a, a1 = a0 + (uintptr_t)a_elems * 2, b0 = (uintptr_t)b, b1 = b0 + (uintptr_t)b_elems * 2;
    return a0 < b1 && b0 < a1;
}

// the caller lent enough zeroed words for the persistent decode kernel
static bool counters_ok(const fa_fwd_params& p) {
    return p.work_counter != nullptr && p.work_counter_len >= FA_WORK_COUNTER_WORDS && (uintptr_t)p.work_counter % 8 == 0;
}
// epoch of the next launch's ticket counters (epoch_counter_next, fa_common.h): never zero, never the same twice
// in a row within a process
static uint32_t next_epoch() {
    static std::atomic<uint32_t> g_epoch{0};
    uint32_t e = g_epoch.fetch_add(1, std::memory_order_relaxed) + 1;
    if (e == 0) e = g_epoch.fetch_add(1, std::memory_order_relaxed) + 1;
    return e;
}

// Split planning for 256 CUs.
struct SplitPlan {
    int splits = 1;        // partial slots (what the caller allocates)
    int len = 0;           // keys per chunk
    int persistent = 0;    // ticket-scheduled decode kernel
    int sa = 0, sb = 0, sub = 0;
};

static SplitPlan plan(const fa_fwd_params& p_in, bool allow_split) {
    SplitPlan r;
    fa_fwd_params p = p_in;
    // what runs is the problem with the grouped heads as rows (no change when it already is)
    const bool packed = !groups_as_rows(p) && positions_and_groups_as_rows(p, nullptr, nullptr) > 0;
    const int sk = p.seqlen_k;
    const int db = bucket(p.d);
    const bool dec = use_decode_kernel(p);
    // The tiled kernel under the persistent schedule of the decode kernel (prefill_persistent_kernel): one row
    // block per (batch, kv head) with every q head of the kv head in it, over a cache whose lengths are on the
    // device.  Chunks of FA_TILE_MINLEN keys or more (about FA_TILE_SLOTS per launch; down to 512 keys in launches too
    // small to fill the CUs otherwise), their remainders in halves, quarters or eighths of a chunk (see sb below).
    const int64_t wgs = (int64_t)((p.seqlen_q + prefill_block_m(db) - 1) / prefill_block_m(db)) * p.h * p.b;
    int64_t tile_chunk = 0;
    if (!dec && allow_split && p.num_splits == 0 && p.p_dropout == 0.f && counters_ok(p) && !p.cu_seqlens_q && p.cu_seqlens_k &&
        !p.is_seqlens_k_cumulative && p.seqlen_q <= prefill_block_m(db) && p.h == p.h_k) {
        // (launches too small to give every resident workgroup a chunk of FA_TILE_MINLEN keys take shorter ones,
        // down to 512: one sequence of 16k keys on 8 kv heads is 64 chunks of 2048 keys, a quarter of the CUs)
        const int64_t fill = ((int64_t)sk * wgs / (2 * kNumCU) + 511) / 512 * 512;
        const int64_t minlen = std::min<int64_t>(FA_TILE_MINLEN, std::max<int64_t>(512, fill));
        const int64_t len = (std::max<int64_t>(minlen, (int64_t)sk * wgs / FA_TILE_SLOTS) + 511) / 512 * 512;
        // (launches that fill the CUs without a split keep the plain form up to 8192 keys: two or three chunks per
        // sequence do not pay for the merge)
        // (Rows that are plain query positions, enough of them for the pipelined kernels, in a launch that fills the
        // CUs: left whole, on those kernels -- 96-128 rows, 256-2048 row blocks, caches of 8k-32k: +5-57 % at head
        // dims 64 / 128 and +30-85 % at 256 on equal and on short lengths, -6..-11 % on lengths drawn from the
        // whole range at 512 row blocks; with 64 row blocks the ticket schedule is 2-4 x as fast.)
        const bool whole_is_fast = !packed && p.seqlen_q >= prefill_long_rows(db) && wgs >= kNumCU;
        if (sk >= 2 * len && (wgs < kNumCU || sk >= 8192) && !whole_is_fast) tile_chunk = len;
    }
    const int gran = dec ? 128 : tile_chunk ? 512 : prefill_block_n(db);
    auto rup = [](int64_t x, int64_t m) { return (int)((x + m - 1) / m * m); };
    int splits = 1;
    bool automatic = false;
    if (p.p_dropout > 0.f) allow_split = false;      // as the reference (flash_api.cpp:380)
    if (allow_split && sk > 0) {
        if (p.num_splits > 1) {
            splits = p.num_splits;
        } else if (p.num_splits == 0) {
            automatic = true;
            if (dec) {
                // ~8k chunk slots over the whole launch (16 per resident workgroup), chunks of at
                // least 256 to 512 keys: measured best trade between per-workgroup start-up cost and
                // the tail left by ragged cache lengths on 256 CUs x 2 resident groups.
                // With the caller's scratch word the kernel is persistent and takes longer chunks
                // (4096 keys at batch 64 x 8 kv heads x 32k), their ragged remainders in pieces of 512+ keys.
                const int64_t streams = (int64_t)p.b * p.h_k;
                // Chunks shorter than 512 keys are mostly start-up and merge (batch 4 x 32k: +22 % with
                // 512 over 256); 256 only while 512-key chunks would leave resident slots empty.
                const int64_t minlen = streams * ((sk + FA_DEC_MINLEN - 1) / FA_DEC_MINLEN) < 2 * kNumCU ? 256 : FA_DEC_MINLEN;
                int64_t len = rup(std::max<int64_t>(minlen, (int64_t)sk * streams / FA_DEC_SLOTS), 128);
                if (counters_ok(p)) {
                    const int64_t lp = rup(std::max<int64_t>(256, (int64_t)sk * streams / FA_DEC_SLOTS_P), 128);
                    // (at least 2048 keys once persistent: batch 4 x 128k keys x 8 kv heads +9 % over 1024-key chunks)
                    if (lp >= 1024) len = std::max<int64_t>(lp, 2048);
                }
                splits = (int)((sk + len - 1) / len);
            } else if (tile_chunk) {
                splits = (int)((sk + tile_chunk - 1) / tile_chunk);
            } else {
                // Launches that take the pipelined / ping-pong kernels when left whole (fa_prefill_inst.hip) are split
                // later than the others: those kernels are 1.3-1.5 x (head dim 256: 2 x) as fast per workgroup as
                // the general kernel the split form runs, and the split adds the merge.  Measured, 128-511 rows,
                // 16-192 row blocks, 512-32768 keys: whole wins from 64 row blocks on up to 1024 keys (2048 at head dim 64; +17-58 %),
                // from 96 up to 2048 (+26-63 %), from 192 on longer keys (+2-150 %; at 128: -17..-36 %); head dim
                // 256 from 64 up to 2048 keys and from 96 beyond (+7-28 %; at 64: -28..-43 %).
                int64_t split_below = FA_SPLIT_BELOW;
                if (!packed && p.seqlen_q >= prefill_long_rows(db)) {     // (with q rotary too: see fa_fwd_kvcache)
                    if (db > 128) split_below = sk <= 2048 ? 64 : 96;
                    else split_below = sk <= (db <= 64 ? 2048 : 1024) ? 64 : sk <= 2048 ? 96 : 192;
                }
                if (wgs < split_below) {
                    const int64_t want = (2 * kNumCU + wgs - 1) / wgs;
                    splits = (int)std::min<int64_t>(want, (sk + 255) / 256);
                }
                // From 256 row blocks on nothing is split here, also where every (batch, head) is one row block
                // over long keys: the plan sees the capacity of a cache, not the lengths in it, and chunks cut for
                // the capacity are mostly empty workgroups when the sequences are short (batch 64, 4096 keys in
                // caches of 32768, 4 positions on 8 kv heads: 0.28 ms split against 0.19).
            }
        }
        splits = std::max(1, std::min(splits, FA_MAX_SPLITS));
        splits = std::min(splits, (sk + gran - 1) / gran);   // never more chunks than tiles
        splits = std::max(1, splits);
    }
    int len = rup((sk + splits - 1) / std::max(1, splits), gran);
    if (len <= 0) len = gran;
    splits = std::max(1, (sk + len - 1) / len);               // drop chunks the rounding emptied
    r.splits = splits;
    r.len = len;
    // Persistent two-pass schedule: complete chunks first, then each sequence's ragged remainder in
    // up to eight pieces of a chunk, drawn from a ticket counter.  Needs the caller's scratch word.
    // The pieces of a remainder stay at 512 keys or more (halves of a 1024-key chunk, quarters of a
    // 2048-key one, eighths from 4096 on): shorter pieces are mostly start-up and merge (measured
    // +6 % at batch 256 x 4k and at batch 64 x 8k with 16 grouped heads, nothing lost at config 5).
    // (The tiled kernel pays more per item -- its Q rows, a first tile nothing overlaps, up to 128 partial rows to
    // write: about what 160 keys take -- so its chunks below 4096 keys are only halved: pieces of 1024 keys or more for
    // chunks of FA_TILE_MINLEN, 256 at the least for the 512-key chunks of a launch that would not fill the CUs.)
    // Halves, quarters or eighths of a multiple of 512: whole tiles.
    const int sb = tile_chunk ? (len < 4096 ? 2 : len < 8192 ? 4 : FA_DEC_SB) : len < 2048 ? 2 : len < 4096 ? 4 : FA_DEC_SB;
    if ((dec || tile_chunk) && automatic && splits > 1 && counters_ok(p) && len >= (dec ? 1024 : 512) && splits + sb <= FA_MAX_SPLITS) {
        r.persistent = 1;
        r.sa = splits;
        r.sb = sb;
        r.sub = len / sb;
        r.splits = r.sa + r.sb;
    }
    return r;
}

static void fill_kparams(KParams& kp, const fa_fwd_params& p) {
    kp.p = p;
    fa_fwd_params& q = kp.p;
    // mask normalisation (flash_api.cpp:111-114, 296-297)
    if (q.is_causal) q.window_right = 0;
    kp.has_left = q.window_left >= 0;
    kp.has_right = q.window_right >= 0;
    kp.scale_log2 = q.softmax_scale * (float)M_LOG2E;
    kp.d_rounded = (q.d + 31) / 32 * 32;
    kp.num_splits = 1;
    kp.split_len = 0;
    kp.num_m_blocks = 0;
    kp.rotary_q = 0;
    kp.dec_persistent = kp.dec_sa = kp.dec_sb = kp.dec_sub = kp.dec_append = kp.dec_compact = 0;
    kp.work_counter = q.work_counter;
    kp.epoch = next_epoch();
    kp.work_items = nullptr;
    kp.pack_g = 0;
    kp.pack_q_hs = kp.pack_o_hs = 0;
    // K + V, 16-bit elements; seqlen_k is the cache capacity (or the longest packed sequence): an upper bound
    kp.stream_kv = (int64_t)4 * q.b * q.seqlen_k * q.h_k * q.d >= kStreamKvBytes;
}

static int run_attention(KParams& kp, hipStream_t stream) {
    const fa_fwd_params& p = kp.p;
    int e;
    if (use_decode_kernel(p)) {
        e = launch_decode(kp, stream);
        if (e) return fail_hip(e, "decode kernel launch");
    } else {
        const bool bf = p.dtype == FA_DTYPE_BF16;
        switch (bucket(p.d)) {
            case 64: e = bf ? launch_prefill_bf16_64(kp, stream) : launch_prefill_fp16_64(kp, stream); break;
            case 128: e = bf ? launch_prefill_bf16_128(kp, stream) : launch_prefill_fp16_128(kp, stream); break;
            default: e = bf ? launch_prefill_bf16_256(kp, stream) : launch_prefill_fp16_256(kp, stream); break;
        }
        if (e) return fail_hip(e, "prefill kernel launch");
    }
    if (kp.num_splits > 1) {
        e = launch_combine(kp, stream);
        if (e) return fail_hip(e, "combine kernel launch");
    }
    if (p.s_dmask) {
        e = launch_attn_probs(kp, stream);
        if (e) return fail_hip(e, "attention probability kernel launch");
    }
    return 0;
}

// `p` is the problem as the caller described it (before grouped heads become rows): plan() applies those
// transforms itself, so what it answers here is what fa_plan_splits answered for the same params.
static int resolve_splits(KParams& kp, const fa_fwd_params& p, bool allow_split) {
    const SplitPlan r = plan(p, allow_split);
    const int s = r.splits;
    kp.num_splits = s;
    kp.split_len = r.len;
    kp.dec_persistent = r.persistent;
    kp.dec_sa = r.sa; kp.dec_sb = r.sb; kp.dec_sub = r.sub;
    kp.dec_compact = r.persistent && !kp.has_left && p.b <= kDecCompactMaxBatch;
    if (s > 1 && (!p.o_accum || !p.lse_accum)) return fail("o_accum and lse_accum are required when the key range is split (see fa_plan_splits)");
    return 0;
}

// Backward: host-side counterpart of mha_bwd / mha_varlen_bwd after tensor unpacking
// (flash_api.cpp:609-832, 834-1036) and of run_mha_bwd's dispatch (:587-607).
static int run_bwd(const fa_bwd_params* p, bool varlen, hipStream_t stream) {
    if (!p) return fail("params is NULL");
    if (!p->dout || !p->q || !p->k || !p->v || !p->out || !p->softmax_lse || !p->dq || !p->dk || !p->dv || !p->softmax_d)
        return fail("dout, q, k, v, out, softmax_lse, dq, dk, dv and softmax_d must be set");
    if (p->dtype != FA_DTYPE_FP16 && p->dtype != FA_DTYPE_BF16) return fail("FlashAttention only support fp16 and bf16 data type");
    if (p->b <= 0) return fail("batch size must be positive");
    if (p->d <= 0 || p->d > 256) return fail("FlashAttention backward only supports head dimension at most 256");
    if (p->d % 8 != 0) return fail("head_size should be a multiple of 8");
    if (p->h <= 0 || p->h_k <= 0 || p->h % p->h_k != 0) return fail("Number of heads in key/value must divide number of heads in query");
    if (p->seqlen_q < 0 || p->seqlen_k < 0) return fail("sequence lengths must be non-negative");
    if (p->seqlen_q_rounded < p->seqlen_q) return fail("seqlen_q_rounded must be at least seqlen_q");
    if (varlen && (!p->cu_seqlens_q || !p->cu_seqlens_k)) return fail("fa_varlen_bwd needs cu_seqlens_q and cu_seqlens_k");
    if (!varlen && (p->cu_seqlens_q || p->cu_seqlens_k)) return fail("fa_bwd takes dense batches; use fa_varlen_bwd");
    if (!(p->p_dropout >= 0.f && p->p_dropout < 1.f)) return fail("p_dropout must be in [0, 1)");
    if (p->p_dropout > 0.f && !p->rng_state) return fail("rng_state is required when p_dropout > 0");
    const int64_t strides[] = {p->q_row_stride, p->q_head_stride, p->k_row_stride, p->k_head_stride, p->v_row_stride,
                               p->v_head_stride, p->o_row_stride, p->o_head_stride, p->do_row_stride, p->do_head_stride,
                               p->dq_row_stride, p->dq_head_stride, p->dk_row_stride, p->dk_head_stride,
                               p->dv_row_stride, p->dv_head_stride, p->q_batch_stride, p->k_batch_stride, p->v_batch_stride,
                               p->o_batch_stride, p->do_batch_stride, p->dq_batch_stride, p->dk_batch_stride, p->dv_batch_stride};
    for (int64_t st : strides) if (st % 8 != 0) return fail("strides must be multiples of 8 elements (16-byte rows)");

    const void* ptrs[] = {p->dout, p->q, p->k, p->v, p->out, p->dq, p->dk, p->dv};
    for (const void* q : ptrs) if ((uintptr_t)q % 16 != 0) return fail("dout, q, k, v, out, dq, dk and dv must be 16-byte aligned");
    // the tile movers add a 32-bit lane byte offset (up to 128 rows) to a 64-bit tile base
    const int64_t row_strides[] = {p->q_row_stride, p->k_row_stride, p->v_row_stride, p->do_row_stride};
    for (int64_t st : row_strides) if (st < 0 || st >= ((int64_t)1 << 23)) return fail("row strides must be below 2^23 elements");

    BwdKParams kp;
    kp.p = *p;
    if (kp.p.is_causal) kp.p.window_right = 0;     // flash_api.cpp:627
    kp.has_left = kp.p.window_left >= 0;
    kp.has_right = kp.p.window_right >= 0;
    kp.scale_log2 = p->softmax_scale * (float)M_LOG2E;
    const bool bf = p->dtype == FA_DTYPE_BF16;
    int e = bf ? launch_bwd_dot_bf16(kp, stream) : launch_bwd_dot_fp16(kp, stream);
    if (e) return fail_hip(e, "backward preprocess kernel launch");
    switch (bucket(p->d)) {
        case 64: e = bf ? launch_bwd_bf16_64(kp, stream) : launch_bwd_fp16_64(kp, stream); break;
        case 128: e = bf ? launch_bwd_bf16_128(kp, stream) : launch_bwd_fp16_128(kp, stream); break;
        default: e = bf ? launch_bwd_bf16_256(kp, stream) : launch_bwd_fp16_256(kp, stream); break;
    }
    if (e) return fail_hip(e, "backward kernel launch");
    return 0;
}

}  // namespace fa

using namespace fa;

// ------------------------------------------------------------------------------------------------
// Device memory owned by the library, for the one entry point that must not allocate
// (fa_fwd_kvcache_noalloc): the ticket word, lse_accum and o_accum of a split launch live in this array
// instead of caller-provided buffers.  Every GPU the library runs on holds its own copy at its own
// address until the process ends; `scratch` itself is only the host-side name of the symbol, the
// address kernels may use is looked up once per device.
// ------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[FA_NOALLOC_SCRATCH_BYTES];

static const int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];          // device address of `scratch`, per device (0: not looked up yet)
static std::mutex g_scratch_mutex;

// address of the current device's copy of `scratch`, or nullptr (g_err says why)
static unsigned char* scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { fail_hip((int)e, "hipGetDevice"); return nullptr; }
    if (dev < 0 || dev >= kMaxDevices) { fail("device index out of range for the no-allocation entry point"); return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));      // resolves the symbol on the CURRENT device
        if (e != hipSuccess || !ptr) { fail_hip((int)e, "hipGetSymbolAddress(scratch)"); return nullptr; }
        g_scratch_ptr[dev] = ptr;
    }
    return static_cast<unsigned char*>(g_scratch_ptr[dev]);
}

static __global__ void set_rng_state_kernel(uint64_t* dst, uint64_t seed, uint64_t offset) {
    if (threadIdx.x == 0) { dst[0] = seed; dst[1] = offset; }
}

extern "C" {

const char* fa_last_error(void) { return g_err.c_str(); }
int32_t fa_version(void) { return (0 << 16) | 1; }
int32_t fa_last_kernel(void) { return g_last_kernel; }
int32_t fa_sizeof_params(void) { return (int32_t)sizeof(fa_fwd_params); }

int fa_num_splits_heuristic_reference(int32_t batch_nheads_mblocks, int32_t num_sms, int32_t num_n_blocks, int32_t max_splits) {
    if (batch_nheads_mblocks >= 0.8f * num_sms) return 1;
    max_splits = std::min({max_splits, num_sms, num_n_blocks});
    auto cdiv = [](int a, int b) { return (a + b - 1) / b; };
    auto eligible = [&](int s) { return s == 1 || cdiv(num_n_blocks, s) != cdiv(num_n_blocks, s - 1); };
    std::vector<float> eff(std::max(max_splits, 0) + 1, 0.f);
    float best = 0.f;
    for (int s = 1; s <= max_splits; s++) {
        if (!eligible(s)) continue;
        const float waves = float(batch_nheads_mblocks * s) / num_sms;
        eff[s] = waves / std::ceil(waves);
        best = std::max(best, eff[s]);
    }
    for (int s = 1; s <= max_splits; s++)
        if (eligible(s) && eff[s] >= 0.85f * best) return s;
    return 1;
}

int fa_plan_splits(const fa_fwd_params* p, int32_t api, int32_t* num_splits) {
    g_err.clear();
    if (int r = check_common(p)) return r;
    if (!num_splits) return fail("num_splits is NULL");
    if (api != 0 && api != 2) return fail("api must be 0 (fa_fwd) or 2 (fa_fwd_kvcache)");
    *num_splits = plan(*p, true).splits;
    return 0;
}

int64_t fa_work_list_words(const fa_fwd_params* p) {
    if (!p || p->h_k <= 0 || p->h <= 0 || p->h % p->h_k != 0) return FA_WORK_COUNTER_WORDS;
    const int64_t w = work_list_words(*p);
    return w > FA_WORK_COUNTER_WORDS ? w : FA_WORK_COUNTER_WORDS;
}

int fa_fwd(const fa_fwd_params* p, void* hip_stream) {
    g_err.clear();
    if (int r = check_common(p)) return r;
    if (p->cu_seqlens_q || p->cu_seqlens_k) return fail("fa_fwd takes dense batches; use fa_varlen_fwd or fa_fwd_kvcache");
    if (p->k_new || p->v_new || p->rotary_cos || p->cache_batch_idx) return fail("fa_fwd does not append or rotate; use fa_fwd_kvcache");
    if (p->seqlen_q == 0) return 0;
    KParams kp;
    fill_kparams(kp, *p);
    kp.p.seqlen_knew = 0;
    kp.p.rotary_dim = 0;
    if (groups_as_rows(kp.p)) kp.has_right = 0;
    else kp.pack_g = positions_and_groups_as_rows(kp.p, &kp.pack_q_hs, &kp.pack_o_hs);
    if (int r = resolve_splits(kp, *p, true)) return r;
    return run_attention(kp, (hipStream_t)hip_stream);
}

int fa_varlen_fwd(const fa_fwd_params* p, void* hip_stream) {
    g_err.clear();
    if (int r = check_common(p)) return r;
    if (!p->cu_seqlens_q || !p->cu_seqlens_k) return fail("cu_seqlens_q and cu_seqlens_k are required");
    if (!p->is_seqlens_k_cumulative) return fail("cu_seqlens_k must be cumulative for fa_varlen_fwd");
    if (p->k_new || p->v_new || p->rotary_cos || p->cache_batch_idx) return fail("fa_varlen_fwd does not append or rotate");
    if (p->seqlen_q == 0) return 0;
    KParams kp;
    fill_kparams(kp, *p);
    kp.p.seqlen_knew = 0;
    kp.p.rotary_dim = 0;
    kp.p.num_splits = 1;
    if (int r = resolve_splits(kp, kp.p, false)) return r;
    return run_attention(kp, (hipStream_t)hip_stream);
}

int fa_fwd_kvcache(const fa_fwd_params* p, void* hip_stream) {
    g_err.clear();
    if (int r = check_common(p)) return r;
    if (p->cu_seqlens_q) return fail("fa_fwd_kvcache takes a dense q batch");
    if (p->p_dropout != 0.f || p->s_dmask) return fail("fa_fwd_kvcache has no dropout");
    if (p->cu_seqlens_k && p->is_seqlens_k_cumulative) return fail("cache_seqlens must be per-batch lengths, not prefix sums");
    const bool has_new = p->k_new != nullptr;
    if (has_new) {
        if (!p->v_new) return fail("If key is supplied, value must also be passed in");
        if (!p->cu_seqlens_k) return fail("If key is supplied, seqlens_k must also be passed in");
        if (p->seqlen_knew <= 0) return fail("seqlen_knew must be positive when k_new is given");
        if (p->seqlen_q > p->seqlen_k) return fail("If key is supplied, it must have seqlen <= the seqlen of the KV cache");
    } else if (p->v_new) {
        return fail("If value is supplied, key must also be passed in");
    }
    if (p->rotary_cos || p->rotary_sin) {
        if (!has_new) return fail("If rotary cos/sin are provided, new key / value to be appended to KV cache must also be provided");
        if (!p->rotary_cos || !p->rotary_sin) return fail("If rotary cos is provided, rotary sin must also be provided");
        if (p->rotary_dim <= 0 || p->rotary_dim > p->d) return fail("rotary_dim must be <= headdim");
        if (p->rotary_dim % 16 != 0) return fail("Only rotary dimensions divisible by 16 are currently supported");
    }
    if (p->seqlen_q == 0) return 0;
    KParams kp;
    fill_kparams(kp, *p);
    if (!has_new) kp.p.seqlen_knew = 0;
    if (!p->rotary_cos) kp.p.rotary_dim = 0;
    kp.rotary_q = kp.p.rotary_dim > 0;
    // (q rotary: without a mask every row is rotated to the position of the first new token, as the one row was)
    if (groups_as_rows(kp.p)) kp.has_right = 0;
    else kp.pack_g = positions_and_groups_as_rows(kp.p, &kp.pack_q_hs, &kp.pack_o_hs);
    if (int r = resolve_splits(kp, *p, true)) return r;
    hipStream_t stream = (hipStream_t)hip_stream;
    // The persistent decode kernel appends the new rows itself: the item that reaches them writes them.
    // With a left window bound some new rows may lie outside every query's window and would not be
    // visited, so there the append stays a launch of its own, as for every other kernel.
    kp.dec_append = has_new && kp.dec_persistent && use_decode_kernel(kp.p) && !kp.has_left;
    if (has_new && !kp.dec_append) {
        if (int e = launch_append_kv(kp, stream)) return fail_hip(e, "append_kv kernel launch");
    }
    // A whole (unsplit) launch of 96+ query rows with q rotary: the rows are rotated into the output tensor by a
    // pass of their own and the attention kernel reads them from there, so that the launch takes the pipelined /
    // ping-pong kernels like one without rotary (a chunk of 512 tokens appended to caches of 16k, batch 64:
    // 8.7 -> 6.0 ms; the general kernel, which rotates while it loads Q, runs at two thirds of their rate).
    // (o holds the rotated q rows before the results land in it, so o must not share memory with q: when their
    // address ranges meet -- the same tensor, or views of one tensor -- the general kernel runs, which rotates
    // while it loads and writes nothing but results)
    const bool disjoint = !spans_overlap(
        kp.p.q, span_elems(kp.p.b, kp.p.seqlen_q, kp.p.h, kp.p.d, kp.p.q_batch_stride, kp.p.q_row_stride, kp.p.q_head_stride),
        kp.p.o, span_elems(kp.p.b, kp.p.seqlen_q, kp.p.h, kp.p.d, kp.p.o_batch_stride, kp.p.o_row_stride, kp.p.o_head_stride));
    if (kp.rotary_q && kp.num_splits <= 1 && kp.pack_g <= 1 && !use_decode_kernel(kp.p) && disjoint &&
        kp.p.seqlen_q >= prefill_long_rows(bucket(kp.p.d))) {
        if (int e = launch_rotate_q(kp, stream)) return fail_hip(e, "q rotary kernel launch");
        kp.p.q = kp.p.o;
        kp.p.q_batch_stride = kp.p.o_batch_stride;
        kp.p.q_row_stride = kp.p.o_row_stride;
        kp.p.q_head_stride = kp.p.o_head_stride;
        kp.rotary_q = 0;
    }
    return run_attention(kp, stream);
}

int fa_fwd_kvcache_noalloc(const fa_fwd_params* p, void* hip_stream) {
    g_err.clear();
    if (!p) return fail("params is NULL");
    unsigned char* base = scratch_of_current_device();
    if (!base) return 2;
    // layout inside the array: [0, kCounterBytes) the persistent decode kernel's counters (zero when the
    // library is loaded, left zero by every launch), then lse_accum, then o_accum (256-byte aligned)
    constexpr size_t kCounterBytes = 64u << 10;
    fa_fwd_params q = *p;
    q.work_counter = reinterpret_cast<int32_t*>(base);
    q.work_counter_len = (int32_t)(kCounterBytes / sizeof(int32_t));
    q.o_accum = nullptr;
    q.lse_accum = nullptr;
    if (int r = check_common(&q)) return r;
    const int splits = plan(q, q.p_dropout == 0.f).splits;
    if (splits > 1) {
        auto up256 = [](size_t x) { return (x + 255) / 256 * 256; };
        const size_t rows = (size_t)q.b * q.h * q.seqlen_q;
        const size_t lse_bytes = up256((size_t)splits * rows * sizeof(float));
        const size_t o_bytes = (size_t)splits * rows * (size_t)((q.d + 31) / 32 * 32) * sizeof(float);
        if (kCounterBytes + lse_bytes + o_bytes > (size_t)FA_NOALLOC_SCRATCH_BYTES)
            return fail("fa_fwd_kvcache_noalloc: the split accumulators of this problem exceed FA_NOALLOC_SCRATCH_BYTES; "
                        "use fa_fwd_kvcache with caller-provided o_accum / lse_accum, or request num_splits = 1");
        q.lse_accum = reinterpret_cast<float*>(base + kCounterBytes);
        q.o_accum = reinterpret_cast<float*>(base + kCounterBytes + lse_bytes);
    }
    return fa_fwd_kvcache(&q, hip_stream);
}

int fa_set_rng_state(uint64_t* rng_state, uint64_t seed, uint64_t offset, void* hip_stream) {
    g_err.clear();
    if (!rng_state) return fail("rng_state is NULL");
    hipLaunchKernelGGL(set_rng_state_kernel, dim3(1), dim3(64), 0, (hipStream_t)hip_stream, rng_state, seed, offset);
    if (int e = (int)hipGetLastError()) return fail_hip(e, "rng state launch");
    return 0;
}

int32_t fa_sizeof_rotary_params(void) { return (int32_t)sizeof(fa_rotary_params); }

int fa_rotary(const fa_rotary_params* p, void* hip_stream) {
    g_err.clear();
    if (!p) return fail("null parameters");
    if (!p->x || !p->out || !p->cos || !p->sin) return fail("x, out, cos and sin are required");
    if (p->dtype != FA_DTYPE_FP16 && p->dtype != FA_DTYPE_BF16) return fail("rotary only supports fp16 and bf16 data");
    if (p->cs_dtype != FA_DTYPE_FP16 && p->cs_dtype != FA_DTYPE_BF16 && p->cs_dtype != FA_DTYPE_FP32) return fail("cos/sin must be fp16, bf16 or fp32");
    if (p->b < 0 || p->seqlen < 0 || p->h < 0 || p->d <= 0) return fail("negative size");
    if (p->rotary_dim <= 0 || p->rotary_dim > p->d) return fail("rotary_dim must be <= headdim");
    if (p->rotary_dim % 2 != 0) return fail("rotary_dim must be even");
    if (p->seqlen_ro < 0) return fail("negative table length");
    // (16-byte granules when rotary_dim is a multiple of 16, the head dim and all strides multiples of 8 elements
    // and the pointers 16-byte aligned; anything else takes the element-wise kernel)
    if (int e = launch_rotary(*p, (hipStream_t)hip_stream)) return fail_hip(e, "rotary kernel launch");
    return 0;
}

int32_t fa_sizeof_bwd_params(void) { return (int32_t)sizeof(fa_bwd_params); }

int fa_bwd(const fa_bwd_params* p, void* hip_stream) {
    g_err.clear();
    return run_bwd(p, false, (hipStream_t)hip_stream);
}

int fa_varlen_bwd(const fa_bwd_params* p, void* hip_stream) {
    g_err.clear();
    return run_bwd(p, true, (hipStream_t)hip_stream);
}

}  // extern "C"
