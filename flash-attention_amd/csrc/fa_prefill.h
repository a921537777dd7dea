// Tiled online-softmax forward kernel for gfx950 (multi-row query tiles: prefill, training
// forward, chunked prefill against a KV cache).  Counterpart of the reference's
// compute_attn_1rowblock / compute_attn_1rowblock_splitkv
// (csrc/flash_attn/src/flash_fwd_kernel.h:74-580, 584-1130), designed for CDNA4:
//
//  * A workgroup is 4 wave64s; each wave owns RB blocks of 32 query rows and keeps its Q
//    fragments in registers for the whole kernel.
//  * Scores are computed TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16: the accumulator
//    layout then gives every lane 16 keys of ONE query row (row = lane % 32), so row max / row sum
//    are in-lane reductions plus one v_permlane32_swap, and the probabilities are already in the
//    B-operand layout of the second product O^T = V^T P^T -- P never leaves registers.
//  * O^T accumulators likewise hold one query row per lane: the online-softmax rescale is a
//    per-lane scalar multiply, no broadcast.
//  * K and V tiles are double-buffered in LDS with a 16-byte-chunk XOR swizzle under which both the
//    K fragment reads (ds_read_b128) and the transposing V reads (ds_read_b64_tr_b16) are
//    bank-conflict free; global loads are 128-bit, issued one tile ahead; LDS operands are read one
//    group of MFMAs ahead (product_rows / product_cols in fa_common.h).
//  * Key tiles that a wave's rows cannot see (causal / sliding window) are skipped per wave.
#pragma once
#include "fa_common.h"
#include "fa_launch.h"

namespace fa {

template <typename T, int D, int RB, int BN>
struct PrefillCfg {
    static constexpr int kThreads = 256;
    static constexpr int kWaves = 4;
    static constexpr int BM = kWaves * 32 * RB;   // query rows per workgroup
    static constexpr int NB = BN / 32;            // 32-key blocks per key tile
    static constexpr int KS = D / 16;             // k-steps of S^T = K Q^T
    static constexpr int DB = D / 32;             // 32-row blocks of O^T
    static constexpr int PT = BN / 16;            // k-steps of O^T = V^T P^T
    static constexpr int CPR = D / 8;             // 16-byte chunks per tile row
    static constexpr int ROWB = D * 2;            // bytes per tile row
    static constexpr int TILE_BYTES = BN * ROWB;
    static constexpr int LOADS = BN * CPR / kThreads;  // 16 B loads per thread, per tensor, per tile
    static constexpr int SMEM = 4 * TILE_BYTES;   // {K,V} x 2 stages
    static_assert(BN % 32 == 0 && D % 32 == 0 && (BN * CPR) % kThreads == 0, "tile shape");
    static_assert(RB == 1, "one 32-row block per wave");
};

// One work item: the row block mb of q head hk * G + g of batch entry b over a key range -- all visible keys
// (SPLIT = false), or those of item (mode, idx) of the split schedule, written as partial `split` (item_key_range).
template <typename T, int D, int RB, int BN, bool SPLIT, bool DROPOUT, bool STREAM>
FA_DEV void prefill_item(const KParams& kp, char* smem, const int tid, const int hk, const int b, const int g, const int mb,
                         const int split, const int mode, const int idx) {
    typedef PrefillCfg<T, D, RB, BN> C;
    typedef typename Elem<T>::v8 v8;
    const fa_fwd_params& p = kp.p;

    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int l32 = lane & 31, hh = lane >> 5;
    const int G = p.h / p.h_k;
    const int head = hk * G + g;

    const SeqInfo si = seq_info(p, b);
    const int m0 = mb * C::BM;
    if (m0 >= si.sq) return;

    // rows may stand for (query position, grouped head) pairs (KParams::pack_g): the position of row r is r / pg
    const int pg = kp.pack_g > 1 ? kp.pack_g : 1;
    const int shift = si.sk - si.sq / pg;
    const int wl = p.window_left, wr = p.window_right;
    const bool has_left = kp.has_left, has_right = kp.has_right;
    int n_hi = si.sk;
    if (has_right) n_hi = min(n_hi, (min(m0 + C::BM, si.sq) - 1) / pg + 1 + shift + wr);
    int n_lo = 0;
    if (has_left) n_lo = max(0, m0 / pg + shift - wl);
    int t_lo = n_lo / BN;
    int t_hi = n_hi > 0 ? (n_hi + BN - 1) / BN : 0;
    if (SPLIT) {
        int c_lo, c_hi;      // multiples of BN (the planner's chunk and piece lengths are)
        item_key_range(kp, mode, idx, si.sk, c_lo, c_hi);
        t_lo = max(t_lo, c_lo / BN);
        t_hi = min(t_hi, c_hi / BN);
    }

    const T* __restrict__ qg = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)head * p.q_head_stride;
    const T* __restrict__ kg = reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)hk * p.k_head_stride;
    const T* __restrict__ vg = reinterpret_cast<const T*>(p.v) + si.v_off + (int64_t)hk * p.v_head_stride;

    // ---- Q fragments (B operand of S^T = K Q^T): lane (l32, hh) holds Q[row l32][16*dk + 8*hh ..+7]
    v8 qf[RB][C::KS];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int row = m0 + (wave * RB + rb) * 32 + l32;
        const bool valid = row < si.sq;
        const int qi = row / pg;
        const T* qrow = qg + (int64_t)qi * p.q_row_stride + (pg > 1 ? (int64_t)(row - qi * pg) * kp.pack_q_hs : (int64_t)0);
#pragma unroll
        for (int dk = 0; dk < C::KS; dk++) {
            const int d0 = dk * 16 + 8 * hh;
            u32x4 raw = {0, 0, 0, 0};
            if (valid && d0 < p.d) {
                raw = ld_global16(qrow + d0);
                if (kp.rotary_q && d0 < p.rotary_dim) {
                    // (a full cache puts cache length + row past the cache: the table is only known to cover the
                    // cache capacity, so the position stops at its last row)
                    const int pos = min(si.sk_cache + ((p.is_causal || has_left || has_right) ? qi : 0), p.seqlen_k - 1);
                    const T* cr = reinterpret_cast<const T*>(p.rotary_cos) + (int64_t)pos * (p.rotary_dim / 2);
                    const T* sr = reinterpret_cast<const T*>(p.rotary_sin) + (int64_t)pos * (p.rotary_dim / 2);
                    float x[8];
                    unpack8<T>(raw, x);
                    rotary8<T>(x, qrow, cr, sr, d0, p.rotary_dim, p.is_rotary_interleaved != 0);
                    raw = pack8<T>(x);
                }
            }
            qf[rb][dk] = __builtin_bit_cast(v8, raw);
        }
    }

    wait_resident_loads();
    f32x16 o_acc[RB][C::DB];
    float m_run[RB], l_run[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        m_run[rb] = -INFINITY;
        l_run[rb] = 0.f;
#pragma unroll
        for (int db = 0; db < C::DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o_acc[rb][db][r] = 0.f;
    }

    // ---- tile movers
    u32x4 kr[C::LOADS], vr[C::LOADS];
    // Loads are unconditional (row / column clamped into range) so that they stay in flight across
    // the tile's compute; out-of-range rows and columns are zeroed when the tile is written to LDS.
    const int d_last_chunk = p.d / 8 - 1;
    auto load_tile = [&](int t) {
        const int n0 = t * BN;
#pragma unroll
        for (int i = 0; i < C::LOADS; i++) {
            const int f = tid + i * C::kThreads;
            const int row = f / C::CPR, c = min(f % C::CPR, d_last_chunk);
            const int n = min(n0 + row, si.sk - 1);
            if constexpr (STREAM) {
                kr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kg + (int64_t)n * p.k_row_stride + c * 8));
                vr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vg + (int64_t)n * p.v_row_stride + c * 8));
            } else {
                kr[i] = ld_global16(kg + (int64_t)n * p.k_row_stride + c * 8);
                vr[i] = ld_global16(vg + (int64_t)n * p.v_row_stride + c * 8);
            }
        }
    };
    auto store_tile = [&](int buf, int t) {
        char* kb = smem + buf * 2 * C::TILE_BYTES;
        char* vb = kb + C::TILE_BYTES;
        const int n0 = t * BN;
#pragma unroll
        for (int i = 0; i < C::LOADS; i++) {
            const int f = tid + i * C::kThreads;
            const int row = f / C::CPR, c = f % C::CPR;
            const bool ok = (n0 + row < si.sk) && (c <= d_last_chunk);
            const u32x4 z = {0, 0, 0, 0};
            const int off = row * C::ROWB + swz_u<D>(c, row) * 16;
            *reinterpret_cast<u32x4*>(kb + off) = ok ? kr[i] : z;
            *reinterpret_cast<u32x4*>(vb + off) = ok ? vr[i] : z;
        }
    };

    LdsOffs<D, C::KS, C::DB> lo;
    lo.init(lane);

    const float sl2 = kp.scale_log2;
    Drop drop = {0, 0, 256, 1.f};
    if constexpr (DROPOUT) drop = drop_init(p.rng_state, p.p_dropout, b, head, p.h);

    if (t_hi > t_lo) {
        load_tile(t_hi - 1);
        store_tile(0, t_hi - 1);
    }
    __syncthreads();
    int buf = 0;
    for (int t = t_hi - 1; t >= t_lo; --t) {
        const bool has_next = t > t_lo;
        if (has_next) load_tile(t - 1);

        const int n0 = t * BN;
        const char* kb = smem + buf * 2 * C::TILE_BYTES;
        const char* vb = kb + C::TILE_BYTES;

        bool skip[RB];
        bool any_work = false;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const int r0 = m0 + (wave * RB + rb) * 32;
            skip[rb] = (has_right && n0 > (r0 + 31) / pg + shift + wr) ||
                       (has_left && n0 + BN - 1 < r0 / pg + shift - wl) || (r0 >= si.sq);
            any_work |= !skip[rb];
        }

        if (any_work) {
            // ---- S^T = K Q^T
            f32x16 s_acc[RB][C::NB];
            product_rows<T, D, C::NB, C::KS, 4>(s_acc[0], kb, lo.r, qf[0]);

            // ---- mask, online softmax, pack P
            v8 pf[RB][C::PT];
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                if (skip[rb]) continue;
                const int r0 = m0 + (wave * RB + rb) * 32;
                const bool need_mask = (n0 + BN > si.sk) || (has_right && n0 + BN - 1 > r0 / pg + shift + wr) ||
                                       (has_left && n0 < (r0 + 31) / pg + shift - wl);
                if (need_mask) {
                    const int row = (r0 + l32) / pg;       // the query position the masks follow
                    int lim_hi = si.sk - 1;
                    if (has_right) lim_hi = min(lim_hi, row + shift + wr);
                    const int lim_lo = has_left ? row + shift - wl : 0;
#pragma unroll
                    for (int nb = 0; nb < C::NB; nb++) mask_acc16(s_acc[rb][nb], n0 + nb * 32 + 4 * hh, lim_lo, lim_hi);
                }
                float mx = -INFINITY;
#pragma unroll
                for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) mx = fmaxf(mx, s_acc[rb][nb][r]);
                mx = xhalf_max(mx);
                const float m_old = m_run[rb];
                const float m_new = fmaxf(m_old, mx);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                const float corr = fast_exp2((m_old - m_use) * sl2);
                const float msc = m_use * sl2;
                float sum = 0.f;
#pragma unroll
                for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const float pv = fast_exp2(s_acc[rb][nb][r] * sl2 - msc);
                        s_acc[rb][nb][r] = pv;
                        sum += pv;
                    }
                l_run[rb] = l_run[rb] * corr + sum;
                m_run[rb] = m_new;
                // the row sum above is of the undropped probabilities; dropped entries leave the
                // second product only (masked after packing), and 1 / (1 - p) is applied once in the epilogue
                uint32_t keep[C::NB][8];
                if constexpr (DROPOUT) {
#pragma unroll
                    for (int nb = 0; nb < C::NB; nb++) drop_pairs_row(drop, r0 + l32, n0 + nb * 32, hh, keep[nb]);
                }
                if (__builtin_amdgcn_ballot_w64(m_new != m_old) != 0) {
#pragma unroll
                    for (int db = 0; db < C::DB; db++)
#pragma unroll
                        for (int r = 0; r < 16; r++) o_acc[rb][db][r] *= corr;
                }
#pragma unroll
                for (int t16 = 0; t16 < C::PT; t16++) {
                    const int nb = t16 >> 1, r8 = (t16 & 1) * 8;
                    u32x4 pk;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        pk[e] = pack2<T>(s_acc[rb][nb][r8 + 2 * e], s_acc[rb][nb][r8 + 2 * e + 1]);
                        if constexpr (DROPOUT) pk[e] &= keep[nb][r8 / 2 + e];
                    }
                    pf[rb][t16] = __builtin_bit_cast(v8, pk);
                }
            }

            // ---- O^T += V^T P^T
            product_cols<T, D, C::PT, C::DB, 4>(o_acc[0], vb, lo.c, pf[0]);
        }

        if (has_next) store_tile(buf ^ 1, t - 1);
        __syncthreads();
        buf ^= 1;
    }

    // ---- epilogue: normalise, write O (and log-sum-exp).  A row that saw no key gives 0 / +inf
    // (reference: flash_fwd_kernel.h:509-516), a split that saw no key gives 0 / -inf (:623-662).
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int row = m0 + (wave * RB + rb) * 32 + l32;
        const float l_tot = xhalf_sum(l_run[rb]);
        const bool dead = (l_tot == 0.f) || (l_tot != l_tot);
        const float inv = dead ? 1.f : drop.rp / l_tot;
        const float lse = dead ? (SPLIT ? -INFINITY : INFINITY) : m_run[rb] * p.softmax_scale + __logf(l_tot);
        if (row >= si.sq) continue;
        const int qi = row / pg, gg = row - qi * pg;
        if (SPLIT) {
            const int64_t ridx = (((int64_t)split * p.b + b) * p.h + head) * p.seqlen_q + row;
            if (hh == 0) p.lse_accum[ridx] = lse;
            float* orow = p.o_accum + ridx * kp.d_rounded;
#pragma unroll
            for (int db = 0; db < C::DB; db++)
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const int d0 = db * 32 + 8 * q4 + 4 * hh;
                    if (d0 < kp.d_rounded) {
                        f32x4 v = {o_acc[rb][db][4 * q4] * inv, o_acc[rb][db][4 * q4 + 1] * inv,
                                   o_acc[rb][db][4 * q4 + 2] * inv, o_acc[rb][db][4 * q4 + 3] * inv};
                        *reinterpret_cast<f32x4*>(orow + d0) = v;
                    }
                }
        } else {
            if (hh == 0) p.softmax_lse[(((int64_t)b * p.h + head) * pg + gg) * (p.seqlen_q / pg) + qi] = lse;
            T* orow = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)qi * p.o_row_stride + (int64_t)head * p.o_head_stride +
                      (pg > 1 ? (int64_t)gg * kp.pack_o_hs : (int64_t)0);
#pragma unroll
            for (int db = 0; db < C::DB; db++)
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const int d0 = db * 32 + 8 * q4 + 4 * hh;
                    if (d0 < p.d) {
                        u32x2 v = {pack2<T>(o_acc[rb][db][4 * q4] * inv, o_acc[rb][db][4 * q4 + 1] * inv),
                                   pack2<T>(o_acc[rb][db][4 * q4 + 2] * inv, o_acc[rb][db][4 * q4 + 3] * inv)};
                        st_global8(orow + d0, v);
                    }
                }
        }
    }
}

// STREAM: K and V tiles are fetched with non-temporal loads -- for launches in which every K/V row is read by
// exactly one workgroup (one row block per kv head, all of its q heads in it) and the caches are too large to
// stay in the memory-side cache anyway (+5-8 % there; see decode_item in fa_decode.hip).
template <typename T, int D, int RB, int BN, int MINW, bool SPLIT, bool DROPOUT = false, bool STREAM = false>
__global__ void __launch_bounds__(256, MINW) prefill_kernel(const KParams kp) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const fa_fwd_params& p = kp.p;
    // ---- work decode: whole (batch, kv head) streams go to one XCD (block ids are dealt round-robin
    // over the 8 XCDs), so that workgroups sharing a K/V stream share an L2; see xcd_stream_unit.
    const int G = p.h / p.h_k;
    const int S = SPLIT ? kp.num_splits : 1;
    uint32_t unit;
    int hk, b;
    if (!xcd_stream_unit(xcd_strided(p.cu_seqlens_q != nullptr, p.b, p.h_k), (uint32_t)p.b, (uint32_t)p.h_k,
                         (uint32_t)(S * G * kp.num_m_blocks), (kp.has_left || kp.has_right) ? 32u * MINW : 0u, (uint32_t)(S * G), unit, hk, b)) return;
    const int split = (int)(unit % (uint32_t)S); unit /= (uint32_t)S;
    const int g = (int)(unit % (uint32_t)G);
    const int mb = kp.num_m_blocks - 1 - (int)(unit / (uint32_t)G);
    prefill_item<T, D, RB, BN, SPLIT, DROPOUT, STREAM>(kp, smem, (int)threadIdx.x, hk, b, g, mb, split, kChunk, split);
}

// One row block per (batch, kv head) -- a few query positions, the grouped q heads of a kv head as rows -- over
// a cache whose lengths only the device knows: the persistent two-pass schedule of the decode kernel
// (for_each_ticket), here with this kernel's tiles.  A plan cut for the capacity of the cache leaves the
// workgroups of short sequences empty and those of the longest ones alone at the end; the tickets hand out
// only chunks that hold keys, the ragged remainders last and in small pieces.
// (PrefillTicketItem: what for_each_ticket calls per ticket)
template <typename T, int D, int RB, int BN, bool STREAM>
struct PrefillTicketItem {
    static FA_DEV void run(const KParams& kp, char* smem, int hk, int b, int slot, int mode, int idx) {
        // The lane index is made opaque per item: what an item derives from it (row and column offsets of the
        // tile movers, LDS offsets, Q row addresses) would otherwise be computed once before the ticket loop and
        // kept in registers across it, which do not exist: the spills landed between the loads of the Q rows,
        // each reload waiting for every load before it (15 us per item).
        int tid = (int)threadIdx.x;
        asm volatile("" : "+v"(tid));
        prefill_item<T, D, RB, BN, true, false, STREAM>(kp, smem, tid, hk, b, 0, 0, slot, mode, idx);
    }
};
template <typename T, int D, int RB, int BN, int MINW, bool STREAM>
__global__ void __launch_bounds__(256, MINW) prefill_persistent_kernel(const KParams kp) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    for_each_ticket<PrefillTicketItem<T, D, RB, BN, STREAM>>(kp, smem);
}

template <typename T, int D, int RB, int BN, int MINW>
int launch_prefill(KParams kp, hipStream_t stream) {
    typedef PrefillCfg<T, D, RB, BN> C;
    kp.num_m_blocks = (kp.p.seqlen_q + C::BM - 1) / C::BM;
    const bool split = kp.num_splits > 1;
    const int64_t total = (int64_t)kp.num_m_blocks * kp.p.h * kp.p.b * (split ? kp.num_splits : 1);
    if (total <= 0) return 0;
    const int64_t nblocks = xcd_grid(xcd_strided(kp.p.cu_seqlens_q != nullptr, kp.p.b, kp.p.h_k), kp.p.b, kp.p.h_k,
                                     (int64_t)kp.num_m_blocks * (kp.p.h / kp.p.h_k) * (split ? kp.num_splits : 1));
    if (nblocks == 0) return -2;
    dim3 grid((unsigned)nblocks), block(C::kThreads);
    hipError_t e;
    if (kp.dec_persistent) {
        // (the planner asks for this only with one row block per kv head, no grouped heads left and no dropout)
        if (kp.num_m_blocks != 1 || kp.p.h != kp.p.h_k || !split || kp.p.p_dropout > 0.f) return -3;
        const int64_t items = (int64_t)kp.p.b * (kp.dec_sa + kp.dec_sb) * kp.p.h_k;
        const int64_t resident = 256 * MINW;                     // workgroups the 256 CUs hold at once
        const dim3 pgrid((unsigned)std::min(items, resident));
        if (kp.stream_kv) {
            auto kern = prefill_persistent_kernel<T, D, RB, BN, MINW, true>;
            e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
            if (e != hipSuccess) return (int)e;
            hipLaunchKernelGGL(kern, pgrid, block, C::SMEM, stream, kp);
        } else {
            auto kern = prefill_persistent_kernel<T, D, RB, BN, MINW, false>;
            e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
            if (e != hipSuccess) return (int)e;
            hipLaunchKernelGGL(kern, pgrid, block, C::SMEM, stream, kp);
        }
        return note_kernel((int)hipGetLastError(), FA_KERNEL_TILED_TICKETS, false, true, D);
    }
    const bool one_reader = kp.stream_kv && kp.num_m_blocks == 1 && kp.p.h == kp.p.h_k && !(kp.p.p_dropout > 0.f);
    if (split && one_reader) {
        auto kern = prefill_kernel<T, D, RB, BN, MINW, true, false, true>;
        e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    } else if (one_reader) {
        auto kern = prefill_kernel<T, D, RB, BN, MINW, false, false, true>;
        e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    } else if (split) {
        auto kern = prefill_kernel<T, D, RB, BN, MINW, true>;
        e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    } else if (kp.p.p_dropout > 0.f) {
        auto kern = prefill_kernel<T, D, RB, BN, MINW, false, true>;
        e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    } else {
        auto kern = prefill_kernel<T, D, RB, BN, MINW, false>;
        e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
        if (e != hipSuccess) return (int)e;
        hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    }
    return note_kernel((int)hipGetLastError(), FA_KERNEL_TILED, kp.p.p_dropout > 0.f, split, D);
}

// key-tile length used by launch_prefill for a head-dim bucket (the split planner needs it)
template <int D> struct PrefillTile;
template <> struct PrefillTile<64> { static constexpr int RB = 1, BN = 64, MINW = 2; };
template <> struct PrefillTile<128> { static constexpr int RB = 1, BN = 64, MINW = 2; };
template <> struct PrefillTile<256> { static constexpr int RB = 1, BN = 32, MINW = 1; };

}  // namespace fa
