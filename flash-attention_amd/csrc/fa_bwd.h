// Backward kernels for gfx950: dQ by one pass over query tiles, dK / dV by one pass over key tiles.
// Counterpart of the reference's compute_dq_dk_dv_1colblock (csrc/flash_attn/src/flash_bwd_kernel.h:
// 79-780) and its dot_do_o / convert_dQ passes (flash_bwd_preprocess_kernel.h), re-designed so that
// nothing is accumulated through global atomics and no fp32 dq buffer exists:
//
//   D_i   = sum_d dO[i,d] O[i,d]                                   (bwd_dot_kernel)
//   P     = exp(scale * Q K^T - lse),   dP = dO V^T,   dS = P o (dP - D)
//   dQ    = scale * dS K                                           (bwd_dq_kernel: per query tile)
//   dV    = P^T dO,   dK = scale * dS^T Q                          (bwd_dkv3_kernel: per key tile)
//
// Both kernels keep the forward kernels' register geometry: every product is computed TRANSPOSED with
// v_mfma_f32_32x32x16 so that the accumulator gives each lane ONE row of the resident operand (a
// query row in the dQ kernel, a key row in the dK/dV kernel) and 16 rows of the streamed tile; the
// accumulator layout is then already the B-operand layout of the next product, so P and dS never
// leave registers.  Streamed tiles are read from LDS twice, row-wise (ds_read_b128) as the A operand
// of the score-shaped products and transposed (ds_read_b64_tr_b16) as the A operand of the
// gradient-shaped ones; one swizzle (swz_u) keeps both conflict free.  The sum of dK / dV over the
// query heads of a GQA group is a loop inside the key-tile kernel.
#pragma once
#include "fa_common.h"

namespace fa {

struct BwdKParams {
    fa_bwd_params p;
    float scale_log2;             // softmax_scale * log2(e)
    int32_t has_left, has_right;  // window bounds active (after causal normalisation)
};

struct BwdSeq {
    int sq, sk;
    int64_t q_off, k_off, v_off, o_off, do_off, dq_off, dk_off, dv_off;   // element offsets of (row 0, head 0)
};
FA_DEV BwdSeq bwd_seq(const fa_bwd_params& p, int b) {
    BwdSeq s;
    if (p.cu_seqlens_q) {
        const int64_t r0 = p.cu_seqlens_q[b];
        s.sq = p.cu_seqlens_q[b + 1] - (int)r0;
        s.q_off = r0 * p.q_row_stride; s.o_off = r0 * p.o_row_stride;
        s.do_off = r0 * p.do_row_stride; s.dq_off = r0 * p.dq_row_stride;
    } else {
        s.sq = p.seqlen_q;
        s.q_off = (int64_t)b * p.q_batch_stride; s.o_off = (int64_t)b * p.o_batch_stride;
        s.do_off = (int64_t)b * p.do_batch_stride; s.dq_off = (int64_t)b * p.dq_batch_stride;
    }
    if (p.cu_seqlens_k) {
        const int64_t r0 = p.cu_seqlens_k[b];
        s.sk = p.cu_seqlens_k[b + 1] - (int)r0;
        s.k_off = r0 * p.k_row_stride; s.v_off = r0 * p.v_row_stride;
        s.dk_off = r0 * p.dk_row_stride; s.dv_off = r0 * p.dv_row_stride;
    } else {
        s.sk = p.seqlen_k;
        s.k_off = (int64_t)b * p.k_batch_stride; s.v_off = (int64_t)b * p.v_batch_stride;
        s.dk_off = (int64_t)b * p.dk_batch_stride; s.dv_off = (int64_t)b * p.dv_batch_stride;
    }
    return s;
}

// ------------------------------------------------------------------------------------------------
// D_i = rowsum(dO o O).  16 lanes per (row, head); HBM-bound, reads dO and O once.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) bwd_dot_kernel(const BwdKParams kp) {
    const fa_bwd_params& p = kp.p;
    const int b = blockIdx.z, head = blockIdx.y;
    const int row = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int sub = threadIdx.x & 15;
    const BwdSeq si = bwd_seq(p, b);
    float acc = 0.f;
    if (row < si.sq) {
        const T* o = reinterpret_cast<const T*>(p.out) + si.o_off + (int64_t)row * p.o_row_stride + (int64_t)head * p.o_head_stride;
        const T* g = reinterpret_cast<const T*>(p.dout) + si.do_off + (int64_t)row * p.do_row_stride + (int64_t)head * p.do_head_stride;
        for (int c = sub; c * 8 < p.d; c += 16) {
            float a[8], bb[8];
            unpack8<T>(ld_global16(o + c * 8), a);
            unpack8<T>(ld_global16(g + c * 8), bb);
#pragma unroll
            for (int e = 0; e < 8; e++) acc += a[e] * bb[e];
        }
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 16);
    if (sub == 0 && row < p.seqlen_q_rounded)
        p.softmax_d[((int64_t)b * p.h + head) * p.seqlen_q_rounded + row] = row < si.sq ? acc : 0.f;
}

// ------------------------------------------------------------------------------------------------
// dQ: a workgroup owns 128 query rows of one (batch, head) and streams K / V tiles of BN keys.
// ------------------------------------------------------------------------------------------------
// DV: head dims the products run over (a multiple of 32, d <= DV <= D); tiles keep the LDS layout of the bucket D
template <typename T, int D, int BN, int DV = D>
struct BwdDqCfg {
    static constexpr int kThreads = 256, kWaves = 4, BM = 128;
    static constexpr int NB = BN / 32, KS = DV / 16, DB = DV / 32, PT = BN / 16, CPR = D / 8, ROWB = D * 2;
    static constexpr int TILE_BYTES = BN * ROWB;
    static constexpr int LOADS = BN * CPR / kThreads;
    static constexpr int STAGE_BYTES = stage_tile_bytes<DB>();   // a wave's dQ rows on their way out
    static constexpr int GRP = 4;      // tile operands are read this many matrix instructions ahead
    static constexpr int SMEM = 4 * TILE_BYTES > kWaves * STAGE_BYTES ? 4 * TILE_BYTES : kWaves * STAGE_BYTES;   // {K, V} x 2 stages
    static_assert(BN % 32 == 0 && D % 32 == 0 && (BN * CPR) % kThreads == 0, "tile shape");
    static_assert(TILE_BYTES % (kWaves * 1024) == 0 && TILE_BYTES / (kWaves * 1024) == LOADS, "one fill = 1 KB per wave");
};

template <typename T, int D, int BN, int MINW, bool DROPOUT, int DV = D>
__global__ void __launch_bounds__(256, MINW) bwd_dq_kernel(const BwdKParams kp) {
    typedef BwdDqCfg<T, D, BN, DV> C;
    typedef typename Elem<T>::v8 v8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const fa_bwd_params& p = kp.p;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, hh = lane >> 5;

    // logical order: heads of one group adjacent, then query tiles, then kv heads, then batch; whole
    // (batch, kv head) streams go to one XCD so that workgroups streaming the same K / V share an L2
    // (xcd_stream_unit: contiguous eighths for dense batches, every 8th stream for packed ones)
    const int G = p.h / p.h_k;
    const int num_m_blocks = (p.seqlen_q + C::BM - 1) / C::BM;
    int g, mb, hk, b;
    if (!xcd_rows_item(false, p.cu_seqlens_q != nullptr, (uint32_t)p.b, (uint32_t)p.h_k, (uint32_t)G, (uint32_t)num_m_blocks,
                       (kp.has_left || kp.has_right) ? 32u * MINW : 0u, g, mb, hk, b)) return;
    const int head = hk * G + g;

    const BwdSeq si = bwd_seq(p, b);
    const int m0 = mb * C::BM;
    if (m0 >= si.sq) return;
    const int shift = si.sk - si.sq;
    const int wl = p.window_left, wr = p.window_right;
    const bool has_left = kp.has_left, has_right = kp.has_right;
    int n_hi = si.sk;
    if (has_right) n_hi = min(n_hi, min(m0 + C::BM, si.sq) + shift + wr);
    const int n_lo = has_left ? max(0, m0 + shift - wl) : 0;
    const int t_lo = n_lo / BN;
    const int t_hi = n_hi > 0 ? (n_hi + BN - 1) / BN : 0;

    const T* __restrict__ kg = reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)hk * p.k_head_stride;
    const T* __restrict__ vg = reinterpret_cast<const T*>(p.v) + si.v_off + (int64_t)hk * p.v_head_stride;

    // resident operands: this lane's query row of Q and dO, its log-sum-exp and D
    const int r0w = m0 + wave * 32;
    const int row = r0w + l32;
    const bool row_ok = row < si.sq;
    v8 qf[C::KS], gf[C::KS];
    {
        const T* qrow = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)row * p.q_row_stride + (int64_t)head * p.q_head_stride;
        const T* grow = reinterpret_cast<const T*>(p.dout) + si.do_off + (int64_t)row * p.do_row_stride + (int64_t)head * p.do_head_stride;
#pragma unroll
        for (int dk = 0; dk < C::KS; dk++) {
            const int d0 = dk * 16 + 8 * hh;
            u32x4 a = {0, 0, 0, 0}, c = {0, 0, 0, 0};
            if (row_ok && d0 < p.d) { a = ld_global16(qrow + d0); c = ld_global16(grow + d0); }
            qf[dk] = __builtin_bit_cast(v8, a);
            gf[dk] = __builtin_bit_cast(v8, c);
        }
    }
    // a row beyond the sequence, or one that saw no key (lse = +inf), gets P = exp2(-inf) = 0
    const float lse2 = row_ok ? p.softmax_lse[((int64_t)b * p.h + head) * p.seqlen_q + row] * kLog2e : INFINITY;
    const float dsum = row_ok ? p.softmax_d[((int64_t)b * p.h + head) * p.seqlen_q_rounded + row] : 0.f;

    wait_resident_loads();
    f32x16 dq_acc[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) dq_acc[db][r] = 0.f;

    // Tile movers: K and V go from global memory straight into LDS (global_load_lds, 1 KB per wave
    // instruction); the swizzle is applied on the global side.  No zero fill: keys past the sequence
    // repeat its last key and are masked, columns past d repeat the last chunk and meet the zero
    // columns of the resident Q / dO rows or land in dQ columns that are never written.
    const int d_last_chunk = p.d / 8 - 1;
    const uint32_t lds0 = (uint32_t)(size_t)((FA_LDS_PTR(char))smem);
    const uint32_t fill0 = __builtin_amdgcn_readfirstlane((int)(lds0 + (uint32_t)(wave * C::LOADS * 1024)));
    // fill j of this lane: row f_row(j), chunk f_col(j) of the tile (recomputed where the last tile needs them)
    auto f_row = [&](int j) { return ((wave * C::LOADS + j) * 1024 + lane * 16) / C::ROWB; };
    auto f_col = [&](int j) { return min(swz_u<D>((((wave * C::LOADS + j) * 1024 + lane * 16) % C::ROWB) / 16, f_row(j)), d_last_chunk); };
    uint32_t f_koff[C::LOADS], f_voff[C::LOADS];
#pragma unroll
    for (int j = 0; j < C::LOADS; j++) {
        f_koff[j] = (uint32_t)((f_row(j) * (int)p.k_row_stride + f_col(j) * 8) * 2);
        f_voff[j] = (uint32_t)((f_row(j) * (int)p.v_row_stride + f_col(j) * 8) * 2);
    }
    auto load_tile = [&](int buf, int t) {
        const int n0 = t * BN;
        const T* kt = kg + (int64_t)n0 * p.k_row_stride;
        const T* vt = vg + (int64_t)n0 * p.v_row_stride;
        const uint32_t dk_ = fill0 + (uint32_t)(buf * 2 * C::TILE_BYTES);
        const uint32_t dv_ = dk_ + (uint32_t)C::TILE_BYTES;
        if (n0 + BN <= si.sk) {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) {
                async_fill16(kt, f_koff[j], dk_ + j * 1024);
                async_fill16(vt, f_voff[j], dv_ + j * 1024);
            }
        } else {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) {
                const int r = min(f_row(j), si.sk - 1 - n0);
                async_fill16(kt, (uint32_t)((r * (int)p.k_row_stride + f_col(j) * 8) * 2), dk_ + j * 1024);
                async_fill16(vt, (uint32_t)((r * (int)p.v_row_stride + f_col(j) * 8) * 2), dv_ + j * 1024);
            }
        }
    };

    const float sl2 = kp.scale_log2;
    Drop drop = {0, 0, 256, 1.f};
    if constexpr (DROPOUT) drop = drop_init(p.rng_state, p.p_dropout, b, head, p.h);
    LdsOffs<D, C::KS, C::DB> lo;
    lo.init(lane);
    if (t_hi > t_lo) { load_tile(0, t_lo); wait_vmcnt<0>(); }
    __syncthreads();
    int buf = 0;
    for (int t = t_lo; t < t_hi; ++t) {
        const bool has_next = t + 1 < t_hi;
        if (has_next) load_tile(buf ^ 1, t + 1);     // the other stage was last read before the previous barrier
        const int n0 = t * BN;
        const char* kb = smem + buf * 2 * C::TILE_BYTES;
        const char* vb = kb + C::TILE_BYTES;
        const bool skip = (has_right && n0 > r0w + 31 + shift + wr) || (has_left && n0 + BN - 1 < r0w + shift - wl) ||
                          (r0w >= si.sq);
        if (!skip) {
            // one 32-key block at a time, so that only one block's S and dP are live
            const bool need_mask = (n0 + BN > si.sk) || (has_right && n0 + BN - 1 > r0w + shift + wr) ||
                                   (has_left && n0 < r0w + 31 + shift - wl);
            int lim_hi = si.sk - 1;
            if (has_right) lim_hi = min(lim_hi, row + shift + wr);
            const int lim_lo = has_left ? row + shift - wl : 0;
            v8 dsf[C::PT];
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++) {
                f32x16 s_acc[1], dp_acc[1];
                product_rows<T, D, 1, C::KS, C::GRP>(s_acc, kb + nb * 32 * C::ROWB, lo.r, qf);
                product_rows<T, D, 1, C::KS, C::GRP>(dp_acc, vb + nb * 32 * C::ROWB, lo.r, gf);
                if (need_mask) mask_acc16(s_acc[0], n0 + nb * 32 + 4 * hh, lim_lo, lim_hi);
                uint32_t keep[8];
                if constexpr (DROPOUT) drop_pairs_row(drop, row, n0 + nb * 32, hh, keep);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float pv = fast_exp2(s_acc[0][r] * sl2 - lse2);
                    float dpv = dp_acc[0][r];
                    if constexpr (DROPOUT) dpv = drop_gate_half(dpv * drop.rp, keep[r >> 1], r & 1);   // gradient through the dropped P
                    s_acc[0][r] = pv * (dpv - dsum);
                }
                dsf[2 * nb] = pack_acc8<T>(s_acc[0], 0);
                dsf[2 * nb + 1] = pack_acc8<T>(s_acc[0], 8);
            }
            // dQ^T += K^T dS^T
            product_cols<T, D, C::PT, C::DB, C::GRP>(dq_acc, kb, lo.c, dsf);
        }
        wait_vmcnt<0>();       // this wave's fills of the next tile have landed; the barrier publishes them
        __syncthreads();
        buf ^= 1;
    }

    // every tile read is behind the loop's last barrier: the ring is free to stage the gradient rows
    T* obase = reinterpret_cast<T*>(p.dq) + si.dq_off + (int64_t)r0w * p.dq_row_stride + (int64_t)head * p.dq_head_stride;
    store_tile_rows<T, C::DB>(dq_acc, p.softmax_scale, smem + wave * C::STAGE_BYTES, lane, obase, p.dq_row_stride, si.sq - r0w, p.d);
}

// ------------------------------------------------------------------------------------------------
// dK, dV: a workgroup owns 128 keys of one (batch, kv head) and streams the Q / dO tiles (BM query rows)
// of every query head of the group; no product is repeated.  8 waves; wave w < 4 ("P wave") owns key
// block w for S = Q K^T, P = exp(S - lse) and dV^T += dO^T P; wave w + 4 ("dS wave") owns the same keys
// for dP = dO V^T, dS = P o (dP - D) and dK^T += Q^T dS.  P goes from the first to the second through
// LDS in accumulator layout (both waves map lanes to keys and registers to query rows identically,
// so the hand-over is lane to same lane, 16 bytes at a time, sign bit = dropped by dropout).  P is
// handed over in fp16 whatever the tensor type: it lies in [0, 1], and its rounding (2^-11 relative)
// is no coarser than the rounding dS = P o (dP - D) gets anyway as an operand of the dK product.
// The dS wave runs ONE TILE BEHIND: in step t it forms dP of tile t (matrix pipe) and dS, dK of tile
// t - 1 (P of that tile was published before the barrier that ended step t - 1), so no barrier is
// added and its exp-free vector work overlaps its own products.  The Q ring therefore has three
// stages (tile t + 1 arriving, t read by the P wave, t - 1 read transposed by the dS wave); dO has two.
// With DPARTS = 2 (head dims 193-256, or 129-256 with dropout) two workgroups share a key block and each
// accumulates half of the head dimension of dK / dV (both form S and dP in full): the accumulators of all
// 256 columns do not fit next to the resident K / V row in 256 registers (128 + 64 + operand sets, offsets
// and the score block: 55 registers spilled, twice the time).  Up to head dim 192 they do (96 + 48).
// ------------------------------------------------------------------------------------------------
template <typename T, int D, int BM, int DPARTS, int DV = D>
struct BwdDkv3Cfg {
    static constexpr int kThreads = 512, kWaves = 8, BNW = 128;
    static constexpr int MBK = BM / 32, KS = DV / 16, DB = DV / 32 / DPARTS, PT = BM / 16, CPR = D / 8, ROWB = D * 2;
    static constexpr int TILE_BYTES = BM * ROWB;
    static constexpr int LOADS = BM * CPR / kThreads;
    static constexpr int Q_OFF = 0;                                  // 3 stages
    static constexpr int G_OFF = 3 * TILE_BYTES;                     // dO: 2 stages
    static constexpr int AUX_OFF = 5 * TILE_BYTES;                   // 3 stages x {lse (log2 units), D} x BM floats
    static constexpr int X_OFF = AUX_OFF + 3 * 2 * BM * 4;           // P hand-over: 2 buffers x 4 key blocks
    static constexpr int XBLK = BM * 32 * 2;                         // one key block's P tile, fp16
    static constexpr int RING_END = X_OFF + 2 * 4 * XBLK;
    static constexpr int OUT_BYTES = kWaves * stage_tile_bytes<DB>();   // the gradient rows, staged over the ring after the loop
    static constexpr int SMEM = RING_END > OUT_BYTES ? RING_END : OUT_BYTES;
    // the resident K / V rows come in through LDS where the idle ring stages and the hand-over hold them
    static constexpr bool STAGED_ROWS = 4 * 32 * ROWB <= 2 * TILE_BYTES && 4 * 32 * ROWB <= 2 * 4 * XBLK;
    static_assert(BM % 32 == 0 && DV % (32 * DPARTS) == 0 && DV <= D && (BM * CPR) % kThreads == 0 && 2 * BM <= kThreads, "tile shape");
    static_assert(SMEM <= 160 * 1024, "LDS budget");
    static_assert(TILE_BYTES % (kWaves * 1024) == 0 && TILE_BYTES / (kWaves * 1024) == LOADS, "one fill = 1 KB per wave");
};

template <typename T, int D, int BM, int DPARTS, bool DROPOUT, int DV = D>
__global__ void __launch_bounds__(512, 1) bwd_dkv3_kernel(const BwdKParams kp) {
    typedef BwdDkv3Cfg<T, D, BM, DPARTS, DV> C;
    typedef typename Elem<T>::v8 v8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const fa_bwd_params& p = kp.p;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
    const bool role_ds = wave >= 4;         // wave-uniform
    const int kblk = wave & 3;

    const int G = p.h / p.h_k;
    const int num_n_blocks = (p.seqlen_k + C::BNW - 1) / C::BNW;
    uint32_t unit;
    int hk, b;
    if (!xcd_stream_unit(xcd_strided(p.cu_seqlens_q != nullptr, p.b, p.h_k), (uint32_t)p.b, (uint32_t)p.h_k,
                         (uint32_t)(num_n_blocks * DPARTS), (kp.has_left || kp.has_right) ? 32u : 0u, (uint32_t)DPARTS, unit, hk, b)) return;
    const int dpart = (int)(unit % DPARTS);      // with DPARTS = 2 a workgroup accumulates half of the head dim
    const int nblk = (int)(unit / DPARTS);

    const BwdSeq si = bwd_seq(p, b);
    const int n0 = nblk * C::BNW;
    if (n0 >= si.sk) return;
    const int shift = si.sk - si.sq;
    const int wl = p.window_left, wr = p.window_right;
    const bool has_left = kp.has_left, has_right = kp.has_right;
    int i_lo = 0, i_hi = si.sq;
    if (has_right) i_lo = max(0, n0 - shift - wr);
    if (has_left) i_hi = min(si.sq, min(n0 + C::BNW, si.sk) - shift + wl);
    const int t_lo = i_lo / BM;
    const int t_hi = i_hi > i_lo ? (i_hi + BM - 1) / BM : t_lo;
    const int nt = t_hi - t_lo;
    const int iters = nt * G;

    const int j0w = n0 + kblk * 32;
    const int key = j0w + l32;
    const bool key_ok = key < si.sk;

    f32x16 acc[C::DB];      // dV^T (P wave) or dK^T (dS wave) of this wave's keys
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] = 0.f;

    // Tile movers.  Q and dO go from global memory straight into their ring slots (global_load_lds,
    // 1 KB per wave instruction, no staging registers and no LDS store pass): LDS bytes are laid down
    // in lane order, so the swizzle is applied on the global side -- the lane that fills physical chunk
    // pc of row r fetches logical chunk swz_u(pc, r).  There is no zero fill on this path: rows past
    // the sequence repeat its last row and are neutralised by lse = +inf (P = 0), columns past d repeat
    // the last chunk and meet the zero columns of the resident K / V rows, or land in gradient
    // columns that are never written.  lse and D take the register path (one float per lane).
    float aux = 0.f;
    const int d_last_chunk = p.d / 8 - 1;
    const uint32_t lds0 = (uint32_t)(size_t)((FA_LDS_PTR(char))smem);
    // Only the P waves request tiles (FL fills each per tensor): a CU accepts 64 bytes of vector loads
    // per cycle, so a tile keeps the requesting waves at the top of the step for several hundred
    // cycles; meanwhile the dS waves, which request nothing, have the matrix pipe to themselves.
    constexpr int FL = 2 * C::LOADS;
    const uint32_t fill0 = __builtin_amdgcn_readfirstlane((int)(lds0 + (uint32_t)(kblk * FL * 1024)));
    int f_row[FL], f_col[FL];
    uint32_t f_qoff[FL], f_goff[FL];
#pragma unroll
    for (int j = 0; j < FL; j++) {
        const int pos = (kblk * FL + j) * 1024 + lane * 16;
        f_row[j] = pos / C::ROWB;
        f_col[j] = min(swz_u<D>((pos % C::ROWB) / 16, f_row[j]), d_last_chunk);
        f_qoff[j] = (uint32_t)((f_row[j] * (int)p.q_row_stride + f_col[j] * 8) * 2);
        f_goff[j] = (uint32_t)((f_row[j] * (int)p.do_row_stride + f_col[j] * 8) * 2);
    }
    const int aux_row = tid < BM ? tid : tid - BM;
    auto load_tile = [&](int g, int t, int q3, int g2) {
        const int head = hk * G + g;
        const int i0 = t * BM;
        const T* qt = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)head * p.q_head_stride + (int64_t)i0 * p.q_row_stride;
        const T* gt = reinterpret_cast<const T*>(p.dout) + si.do_off + (int64_t)head * p.do_head_stride + (int64_t)i0 * p.do_row_stride;
        const uint32_t dq_ = fill0 + (uint32_t)(C::Q_OFF + q3 * C::TILE_BYTES);
        const uint32_t dg_ = fill0 + (uint32_t)(C::G_OFF + g2 * C::TILE_BYTES);
        if (role_ds) {
            // nothing to request
        } else if (i0 + BM <= si.sq) {
#pragma unroll
            for (int j = 0; j < FL; j++) {
                async_fill16(qt, f_qoff[j], dq_ + j * 1024);
                async_fill16(gt, f_goff[j], dg_ + j * 1024);
            }
        } else {
#pragma unroll
            for (int j = 0; j < FL; j++) {
                const int r = min(f_row[j], si.sq - 1 - i0);
                async_fill16(qt, (uint32_t)((r * (int)p.q_row_stride + f_col[j] * 8) * 2), dq_ + j * 1024);
                async_fill16(gt, (uint32_t)((r * (int)p.do_row_stride + f_col[j] * 8) * 2), dg_ + j * 1024);
            }
        }
        if (tid < 2 * BM) {
            // raw value only: anything computed from it here would make the wave wait for the load
            const float* src = tid < BM ? p.softmax_lse + ((int64_t)b * p.h + head) * p.seqlen_q
                                        : p.softmax_d + ((int64_t)b * p.h + head) * p.seqlen_q_rounded;
            aux = src[min(i0 + aux_row, si.sq - 1)];
        }
    };
    // end of a step: the wave's own fills have landed (the barrier that follows publishes them), lse / D go to LDS
    auto finish_tile = [&](int q3, int t) {
        wait_vmcnt<0>();
        if (tid < 2 * BM) {
            const bool in_range = t * BM + aux_row < si.sq;   // rows past the end: lse = +inf => P = 0
            // D goes in negated where the dS wave starts dP from it (dS = P o (dP - D) without a subtraction)
            const float dval = DROPOUT ? aux : -aux;
            reinterpret_cast<float*>(smem + C::AUX_OFF + q3 * 2 * BM * 4)[tid] = tid < BM ? (in_range ? aux * kLog2e : INFINITY) : (in_range ? dval : 0.f);
        }
    };
    auto skip_tile = [&](int i0) {   // keys of this wave against the rows of a tile: nothing visible
        return (has_right && j0w > i0 + BM - 1 + shift + wr) || (has_left && j0w + 31 < i0 + shift - wl) || (j0w >= si.sk);
    };

    // Prologue: the first tile's requests go out first, then the resident operand -- this lane's key
    // row of K (P wave) or of V (dS wave) -- so that the two latencies overlap.
    if (iters > 0) load_tile(0, t_lo, 0, 0);
    v8 rf[C::KS];
    {
        const T* blk = role_ds
            ? reinterpret_cast<const T*>(p.v) + si.v_off + (int64_t)n0 * p.v_row_stride + (int64_t)hk * p.v_head_stride
            : reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)n0 * p.k_row_stride + (int64_t)hk * p.k_head_stride;
        const int rs = (int)(role_ds ? p.v_row_stride : p.k_row_stride);
        if constexpr (C::STAGED_ROWS) {
            // through a wave-private piece of LDS that the ring does not use before the first barrier
            // (K rows: Q stages 1 and 2, V rows: the P hand-over); keys past the sequence repeat its
            // last key: whatever a lane computes for such a key stays in that lane and is never written
            const int region = (role_ds ? C::X_OFF : C::Q_OFF + C::TILE_BYTES) + kblk * 32 * C::ROWB;
            const int last = si.sk - 1 - n0;
            stage_rows_issue<T, D>(blk, [&](int r) { return min(kblk * 32 + r, last) * rs; }, p.d,
                                   (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + (uint32_t)region)), lane);
            wait_vmcnt<0>();
            stage_rows_read<T, D, C::KS>(rf, smem + region, p.d, lane);
        } else {
            const T* row = blk + (int64_t)(kblk * 32 + l32) * rs;
#pragma unroll
            for (int dk = 0; dk < C::KS; dk++) {
                const int d0 = dk * 16 + 8 * hh;
                u32x4 a = {0, 0, 0, 0};
                if (key_ok && d0 < p.d) a = ld_global16(row + d0);
                rf[dk] = __builtin_bit_cast(v8, a);
            }
        }
    }
    wait_resident_loads();
    if (iters > 0) finish_tile(0, t_lo);
    __syncthreads();

    const float sl2 = kp.scale_log2;
    const int rel_hi = has_right ? shift + wr : 0x3fffffff;
    const int rel_lo = has_left ? shift - wl : -0x3fffffff;
    LdsOffs<D, C::KS, C::DB> lo;
    lo.init(lane, dpart * C::DB);

    // The tile walk shared by both kinds of wave; `body(it, i0, g, live, prev_live, q3, q3_prev)` is the
    // wave's own work of one step.  iters + 1 steps: the last one drains the dS wave's final tile.
    auto walk = [&](auto&& body) {
        int q3 = 0, q3_prev = 0;                     // Q / aux ring slots of the current and the previous tile
        int cur_t = t_lo, cur_g = 0, nxt_g = 0, nxt_t = t_lo;
        bool prev_live = false;                      // the previous tile was not skipped (its P is in the hand-over)
        for (int it = 0; it <= iters; ++it) {
            const bool has_next = it + 1 < iters;
            const int q3_next = q3 == 2 ? 0 : q3 + 1;
            if (has_next) {
                if (++nxt_t == t_hi) { nxt_t = t_lo; ++nxt_g; }
                // slots free since the barrier that ended the previous step: Q[q3_next] held tile it - 2
                // (last read transposed by the dS wave in step it - 1), dO[(it + 1) & 1] held tile it - 1
                load_tile(nxt_g, nxt_t, q3_next, (it + 1) & 1);
            }
            const int i0 = cur_t * BM;
            const bool live = it < iters && !skip_tile(i0);
            body(it, i0, cur_g, live, prev_live, q3, q3_prev);
            prev_live = live;
            if (has_next) finish_tile(q3_next, nxt_t);
            __syncthreads();
            q3_prev = q3;
            q3 = q3_next;
            cur_t = nxt_t;
            cur_g = nxt_g;
        }
    };

    if (!role_ds) {
        walk([&](int it, int i0, int g, bool live, bool, int q3, int) {
            if (live) {
            const char* qb = smem + C::Q_OFF + q3 * C::TILE_BYTES;
            const char* gb = smem + C::G_OFF + (it & 1) * C::TILE_BYTES;
            const float* lse_s = reinterpret_cast<const float*>(smem + C::AUX_OFF + q3 * 2 * BM * 4);
            char* xw = smem + C::X_OFF + ((it & 1) * 4 + kblk) * C::XBLK;
            Drop drop = {0, 0, 256, 1.f};
            if constexpr (DROPOUT) drop = drop_init(p.rng_state, p.p_dropout, b, hk * G + g, p.h);
            f32x16 s_acc[C::MBK];
            product_rows<T, D, C::MBK, C::KS, 4>(s_acc, qb, lo.r, rf);
            v8 pf[C::PT];
#pragma unroll
            for (int mb = 0; mb < C::MBK; mb++) {
                const int ib = i0 + mb * 32;
                const bool need_mask = (has_right && j0w + 31 > ib + shift + wr) || (has_left && j0w < ib + 31 + shift - wl);
                if (need_mask) {
                    // entry r is query row ib + 4 hh + c_r, visible iff rel_lo + c_r <= key - ib - 4 hh <= rel_hi + c_r
                    const int rel = key - ib - 4 * hh;
                    mask_acc16(s_acc[mb], 0, rel - rel_hi, rel - rel_lo);
                }
                uint32_t keep[8];
                if constexpr (DROPOUT) drop_pairs_key(drop, key, ib, hh, keep);
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_s + mb * 32 + 8 * q4 + 4 * hh);
#pragma unroll
                    for (int e = 0; e < 4; e++) s_acc[mb][4 * q4 + e] = fast_exp2(s_acc[mb][4 * q4 + e] * sl2 - l4[e]);
                }
                // hand-over copy in fp16 with the sign bit set where dropped (P >= 0), own copy with zeros there:
                // both masked as packed pairs
#pragma unroll
                for (int h8 = 0; h8 < 2; h8++) {
                    u32x4 xo = __builtin_bit_cast(u32x4, pack_acc8<_Float16>(s_acc[mb], 8 * h8));
                    u32x4 pk = __builtin_bit_cast(u32x4, pack_acc8<T>(s_acc[mb], 8 * h8));
                    if constexpr (DROPOUT) {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            xo[e] |= ~keep[4 * h8 + e] & 0x80008000u;
                            pk[e] &= keep[4 * h8 + e];
                        }
                    }
                    *reinterpret_cast<u32x4*>(xw + ((mb * 2 + h8) * 64 + lane) * 16) = xo;
                    pf[2 * mb + h8] = __builtin_bit_cast(v8, pk);
                }
            }
            product_cols<T, D, C::PT, C::DB, 4>(acc, gb, lo.c, pf);
            }
        });
    } else {
        f32x16 dp[C::MBK];      // dP of the tile of the previous step, carried over the loop
#pragma unroll
        for (int mb = 0; mb < C::MBK; mb++)
#pragma unroll
            for (int r = 0; r < 16; r++) dp[mb][r] = 0.f;
        walk([&](int it, int, int, bool live, bool prev_live, int q3, int q3_prev) {
            // first the previous tile (consumes dp), then dP of this tile into the same registers
            if (prev_live) {
                const char* qp = smem + C::Q_OFF + q3_prev * C::TILE_BYTES;
                const float* dsum_s = reinterpret_cast<const float*>(smem + C::AUX_OFF + q3_prev * 2 * BM * 4) + BM;
                const char* xr = smem + C::X_OFF + (((it - 1) & 1) * 4 + kblk) * C::XBLK;
                const float rp = DROPOUT ? 1.f / (1.f - p.p_dropout) : 1.f;
                v8 dsf[C::PT];
#pragma unroll
                for (int mb = 0; mb < C::MBK; mb++) {
                    const f16x8 ph[2] = {*reinterpret_cast<const f16x8*>(xr + ((mb * 2) * 64 + lane) * 16),
                                         *reinterpret_cast<const f16x8*>(xr + ((mb * 2 + 1) * 64 + lane) * 16)};
                    if constexpr (DROPOUT) {
#pragma unroll
                        for (int q4 = 0; q4 < 4; q4++) {
                            const f32x4 d4 = *reinterpret_cast<const f32x4*>(dsum_s + mb * 32 + 8 * q4 + 4 * hh);
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                const int r = 4 * q4 + e;
                                const float pv = (float)ph[r >> 3][r & 7];
                                const float dpv = __builtin_signbit(pv) ? 0.f : dp[mb][r] * rp;
                                dp[mb][r] = fabsf(pv) * (dpv - d4[e]);
                            }
                        }
                    } else {
                        // dp already holds dP - D: the product below started from -D
#pragma unroll
                        for (int r = 0; r < 16; r++) dp[mb][r] *= (float)ph[r >> 3][r & 7];
                    }
                    dsf[2 * mb] = pack_acc8<T>(dp[mb], 0);
                    dsf[2 * mb + 1] = pack_acc8<T>(dp[mb], 8);
                }
                product_cols<T, D, C::PT, C::DB, 4>(acc, qp, lo.c, dsf);
            }
            if (live) {
                const char* gb = smem + C::G_OFF + (it & 1) * C::TILE_BYTES;
                if constexpr (DROPOUT) {
                    product_rows<T, D, C::MBK, C::KS, 4>(dp, gb, lo.r, rf);
                } else {
                    // dP - D in one go: the accumulators start from -D of their rows (entry r of a lane
                    // is row 8 (r >> 2) + 4 hh + (r & 3) of its block)
                    const float* nd = reinterpret_cast<const float*>(smem + C::AUX_OFF + q3 * 2 * BM * 4) + BM;
#pragma unroll
                    for (int mb = 0; mb < C::MBK; mb++)
#pragma unroll
                        for (int q4 = 0; q4 < 4; q4++) {
                            const f32x4 d4 = *reinterpret_cast<const f32x4*>(nd + mb * 32 + 8 * q4 + 4 * hh);
                            dp[mb][4 * q4] = d4[0]; dp[mb][4 * q4 + 1] = d4[1]; dp[mb][4 * q4 + 2] = d4[2]; dp[mb][4 * q4 + 3] = d4[3];
                        }
                    product_rows<T, D, C::MBK, C::KS, 4, false>(dp, gb, lo.r, rf);
                }
            }
        });
    }
    // every tile read is behind the loop's last barrier: the ring is free to stage the gradient rows
    T* obase = role_ds ? reinterpret_cast<T*>(p.dk) + si.dk_off + (int64_t)j0w * p.dk_row_stride + (int64_t)hk * p.dk_head_stride
                       : reinterpret_cast<T*>(p.dv) + si.dv_off + (int64_t)j0w * p.dv_row_stride + (int64_t)hk * p.dv_head_stride;
    const float sc = role_ds ? p.softmax_scale : (DROPOUT ? 1.f / (1.f - p.p_dropout) : 1.f);
    const int col0 = dpart * C::DB * 32;
    store_tile_rows<T, C::DB>(acc, sc, smem + wave * stage_tile_bytes<C::DB>(), lane, obase + col0,
                              role_ds ? p.dk_row_stride : p.dv_row_stride, si.sk - j0w, p.d - col0);
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
template <typename T, int D, int BN, int MINW, bool DROPOUT, int DV = D>
int launch_bwd_dq(const BwdKParams& kp, hipStream_t stream) {
    typedef BwdDqCfg<T, D, BN, DV> C;
    const int64_t nmb = (kp.p.seqlen_q + C::BM - 1) / C::BM;
    if (nmb * kp.p.h * kp.p.b <= 0) return 0;
    const int64_t nblocks = xcd_rows_grid(false, kp.p.cu_seqlens_q != nullptr, kp.p.b, kp.p.h_k, kp.p.h / kp.p.h_k, nmb);
    if (nblocks == 0) return -2;
    auto kern = bwd_dq_kernel<T, D, BN, MINW, DROPOUT, DV>;
    if (int e = (int)FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM)) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(C::kThreads), C::SMEM, stream, kp);
    return (int)hipGetLastError();
}

template <typename T, int D, int BM, int DPARTS, bool DROPOUT, int DV = D>
int launch_bwd_dkv3(const BwdKParams& kp, hipStream_t stream) {
    typedef BwdDkv3Cfg<T, D, BM, DPARTS, DV> C;
    const int64_t per_stream = (int64_t)((kp.p.seqlen_k + C::BNW - 1) / C::BNW) * DPARTS;
    if (per_stream * kp.p.h_k * kp.p.b <= 0) return 0;
    const int64_t nblocks = xcd_grid(xcd_strided(kp.p.cu_seqlens_q != nullptr, kp.p.b, kp.p.h_k), kp.p.b, kp.p.h_k, per_stream);
    if (nblocks == 0) return -2;
    auto kern = bwd_dkv3_kernel<T, D, BM, DPARTS, DROPOUT, DV>;
    if (int e = (int)FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM)) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(C::kThreads), C::SMEM, stream, kp);
    return (int)hipGetLastError();
}

template <typename T>
int launch_bwd_dot(const BwdKParams& kp, hipStream_t stream) {
    const fa_bwd_params& p = kp.p;
    if (p.b <= 0 || p.h <= 0 || p.seqlen_q_rounded <= 0) return 0;
    dim3 grid((unsigned)((p.seqlen_q_rounded + 15) / 16), (unsigned)p.h, (unsigned)p.b);
    hipLaunchKernelGGL(bwd_dot_kernel<T>, grid, dim3(256), 0, stream, kp);
    return (int)hipGetLastError();
}

}  // namespace fa
