// "Ping-pong" variant of the tiled forward kernel for long query sequences on gfx950.
//
// Same mathematics and register layouts as prefill_kernel (fa_prefill.h): S^T = K Q^T and
// O^T = V^T P^T on v_mfma_f32_32x32x16 with one query row per lane.  What changes is how the
// execution pipes of a SIMD are kept busy.  A CDNA4 SIMD issues matrix (MFMA) and vector (VALU)
// instructions from different waves at the same time, and for head dim 128 the exp2/max/sum work
// of a key tile costs about as many cycles as its two matrix products.  So:
//
//  * a workgroup is 8 waves = two groups of 4; waves w and w+4 sit on the same SIMD;
//  * every wave alternates a VALU phase Y(i) (mask + online softmax of tile i) and an MFMA phase
//    X(i) (O += P_i V_i, then S = K_{i+1} Q), separated by workgroup barriers;
//  * group 1 runs one phase behind group 0 (it takes one extra barrier up front, group 0 one extra
//    at the end), so at any time one wave of each SIMD is in its MFMA phase and the other in its
//    VALU phase.
//
// K and V tiles are shared by all 8 waves (256 query rows per workgroup) and move from global
// memory straight into LDS with global_load_lds_dwordx4 (no staging registers, no ds_write):
// each wave instruction deposits 64 x 16 B contiguously in LDS, so the bank-conflict-avoiding XOR
// swizzle is applied on the global side (lane -> which 16 B chunk of which row it fetches).  A ring
// of 4 tile slots per tensor is filled 3 tiles ahead; the barrier pattern guarantees that a slot is
// refilled only after both groups have passed the phase that read it, and each wave waits for its
// own outstanding fills (vmcnt) before the barrier that publishes them.
//
// The running max is updated lazily: a row's reference max moves only when the new max exceeds it
// by more than 2^8 in the exp2 domain, which makes the O rescale rare after the first tiles while
// keeping every probability <= 256 (exact in the final normalisation, safe in fp16/bf16).
#pragma once
#include "fa_common.h"
#include "fa_launch.h"

namespace fa {

#ifndef FA_PP_LA
#define FA_PP_LA 4
#endif

template <typename T, int D, int BN>
struct PPCfg {
    static constexpr int kThreads = 512;
    static constexpr int kWaves = 8;
    static constexpr int BM = kWaves * 32;
    static constexpr int NB = BN / 32;
    static constexpr int KS = D / 16;
    static constexpr int DB = D / 32;
    static constexpr int PT = BN / 16;
    static constexpr int CPR = D / 8;                       // 16 B chunks per tile row
    static constexpr int ROWB = D * 2;
    static constexpr int TILE = BN * ROWB;                  // bytes of one K or V tile
    static constexpr int NS = 4;                            // ring slots per tensor
    static constexpr int PF = NS - 1;                       // tiles of look-ahead
    static constexpr int LOADS = BN * CPR / kThreads;       // 16 B fills per thread per tile
    static constexpr int ROWS_PER_PASS = kThreads / CPR;
    static constexpr int SMEM = 2 * NS * TILE;              // K ring, then V ring
    static_assert((BN * CPR) % kThreads == 0 && 64 % CPR == 0, "tile shape");
};

// DV: head dims the products run over (a multiple of 32, p.d <= DV <= D).  Tiles keep the LDS layout of the
// bucket D; with DV < D the k-steps and output column blocks past DV are not computed (head dim 96 on the
// 128 bucket: 6 of 8 k-steps of S, 3 of 4 column blocks of O).
template <typename T, int D, int BN, bool DROPOUT = false, int DV = D>
__global__ void __launch_bounds__(512, 2) prefill_pp_kernel(const KParams kp) {
    typedef PPCfg<T, D, BN> C;
    static_assert(DV % 32 == 0 && DV <= D, "computed head dims");
    constexpr int KSV = DV / 16, DBV = DV / 32;
    typedef typename Elem<T>::v8 v8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const fa_fwd_params& p = kp.p;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int l32 = lane & 31, hh = lane >> 5;
    const int group = wave >> 2;

    // work item of this block (32-bit arithmetic: the launcher bounds the grid by 2^31)
    const uint32_t G = (uint32_t)(p.h / p.h_k);
    int g, mb, hk, b;
    if (!xcd_work_item(kp, (uint32_t)kp.num_m_blocks, (kp.has_left || kp.has_right) ? 32u : 0u, g, mb, hk, b)) return;
    const int head = hk * (int)G + g;

    const SeqInfo si = seq_info(p, b);
    const int m0 = mb * C::BM;
    if (m0 >= si.sq) return;

    const int shift = si.sk - si.sq;
    const int wl = p.window_left, wr = p.window_right;
    const bool has_left = kp.has_left, has_right = kp.has_right;
    int n_hi = si.sk;
    if (has_right) n_hi = min(n_hi, min(m0 + C::BM, si.sq) + shift + wr);
    int n_lo = 0;
    if (has_left) n_lo = max(0, m0 + shift - wl);
    const int t_lo = n_lo / BN;
    const int t_hi = n_hi > 0 ? (n_hi + BN - 1) / BN : 0;
    const int nt = max(0, t_hi - t_lo);           // tiles visited, the same for all 8 waves

    const T* __restrict__ qg = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)head * p.q_head_stride;
    const T* __restrict__ kg = reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)hk * p.k_head_stride;
    const T* __restrict__ vg = reinterpret_cast<const T*>(p.v) + si.v_off + (int64_t)hk * p.v_head_stride;

    const int r0 = m0 + wave * 32;                // first query row of this wave
    const int row = r0 + l32;

    // visit i of the key loop handles key tile tile_of(i) and uses ring slot i % NS
    // (from the last tile down: the masked tiles of a causal row block come first)
    auto tile_of = [&](int i) { return t_hi - 1 - i; };

    // ---- asynchronous tile fills.  Pass j of wave w fills LDS positions [(w + 8j) * 64, +64) of the
    // tile (16 B each); position p is tile row p / CPR, stored chunk p % CPR, and holds global chunk
    // (p % CPR) ^ swizzle(row).
    const int frow = (wave * 64 + lane) / C::CPR;              // tile row of pass 0
    const int fch = lane % C::CPR;
    const int kch = min(swz_k<D>(fch, frow), p.d / 8 - 1);     // clamped: columns >= d are never used
    const int vch = min(swz_v<D>(fch, frow), p.d / 8 - 1);
    const uint32_t lds0 = (uint32_t)(size_t)((FA_LDS_PTR(char))smem);
    const uint32_t fill_base = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(wave * 1024));
    // The address of a fill is a scalar base (start of the tile, uniform over the workgroup) plus a
    // 32-bit per-lane byte offset, so stepping to the next tile is scalar arithmetic.
    const int64_t kstep = (int64_t)BN * p.k_row_stride, vstep = (int64_t)BN * p.v_row_stride;
    const int64_t kpass = (int64_t)C::ROWS_PER_PASS * p.k_row_stride, vpass = (int64_t)C::ROWS_PER_PASS * p.v_row_stride;
    const int t_first = t_hi - 1;
    const T* ktile = kg + (int64_t)t_first * BN * p.k_row_stride;       // tile next to be requested
    const T* vtile = vg + (int64_t)t_first * BN * p.v_row_stride;
    const uint32_t koff = (uint32_t)(((int64_t)frow * p.k_row_stride + kch * 8) * 2);
    const uint32_t voff = (uint32_t)(((int64_t)frow * p.v_row_stride + vch * 8) * 2);
    // only key tile t_hi - 1 can reach past seqlen_k: its rows are clamped
    const int i_tail = (t_hi * BN > si.sk) ? 0 : -1;
    auto fill_k = [&](int i) {
        const uint32_t dst = fill_base + (uint32_t)((i & (C::NS - 1)) * C::TILE);
        if (i == i_tail) {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) {
                const int n = min(frow + j * C::ROWS_PER_PASS, si.sk - 1 - (t_hi - 1) * BN);
                async_fill16(ktile, (uint32_t)(((int64_t)n * p.k_row_stride + kch * 8) * 2), dst + j * 8192);
            }
        } else {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) async_fill16(ktile + j * kpass, koff, dst + j * 8192);
        }
        ktile -= kstep;
    };
    auto fill_v = [&](int i) {
        const uint32_t dst = fill_base + (uint32_t)((C::NS + (i & (C::NS - 1))) * C::TILE);
        if (i == i_tail) {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) {
                const int n = min(frow + j * C::ROWS_PER_PASS, si.sk - 1 - (t_hi - 1) * BN);
                async_fill16(vtile, (uint32_t)(((int64_t)n * p.v_row_stride + vch * 8) * 2), dst + j * 8192);
            }
        } else {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) async_fill16(vtile + j * vpass, voff, dst + j * 8192);
        }
        vtile -= vstep;
    };

    // The first tiles are requested before anything else is set up: the q rows, the accumulators and the
    // per-lane LDS offsets below are all prepared while these requests are in flight.
    if (nt > 0) {
        fill_k(0);
        fill_v(0);
        if (nt > 1) { fill_k(1); fill_v(1); }
        if (nt > 2) fill_k(2);
    }

    v8 qf[KSV];
    {
        const bool valid = row < si.sq;
        const T* qrow = qg + (int64_t)row * p.q_row_stride;
#pragma unroll
        for (int dk = 0; dk < KSV; dk++) {
            const int d0 = dk * 16 + 8 * hh;
            u32x4 raw = {0, 0, 0, 0};
            if (valid && d0 < p.d) raw = ld_global16(qrow + d0);
            qf[dk] = __builtin_bit_cast(v8, raw);
        }
    }
    f32x16 o_acc[DBV];
#pragma unroll
    for (int db = 0; db < DBV; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[db][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const float sl2 = kp.scale_log2;
    Drop drop = {0, 0, 256, 1.f};
    if constexpr (DROPOUT) drop = drop_init(p.rng_state, p.p_dropout, b, head, p.h);


    // Per-wave tile classes, as ranges of the absolute key-tile index t: the wave has visible keys
    // in tiles [ta_lo, ta_hi]; tiles in [tf_lo, tf_hi] are fully visible to all 32 rows (no masking).
    int ta_lo = t_lo, ta_hi = t_hi - 1, tf_lo = 0, tf_hi = si.sk / BN - 1;
    if (has_right) {
        const int c = r0 + shift + wr;            // last visible key of the wave's first row
        ta_hi = min(ta_hi, (c + 31 >= 0) ? (c + 31) / BN : -1);
        tf_hi = min(tf_hi, (c + 1 >= BN) ? (c + 1) / BN - 1 : -1);
    }
    if (has_left) {
        const int c = r0 + shift - wl;            // first visible key of the wave's first row
        ta_lo = max(ta_lo, (c > 0) ? c / BN : 0);
        tf_lo = (c + 31 > 0) ? (c + 31 + BN - 1) / BN : 0;
    }
    if (r0 >= si.sq) ta_hi = ta_lo - 1;
    auto active = [&](int i) -> bool { const int t = tile_of(i); return t >= ta_lo && t <= ta_hi; };

    // ---- S^T = K Q^T.  Fragment reads run LA matrix instructions ahead of their use and are
    // interleaved one-for-one with the MFMAs.
    int kofs[KSV];
#pragma unroll
    for (int dk = 0; dk < KSV; dk++) kofs[dk] = l32 * C::ROWB + swz_k<D>(dk * 2 + hh, l32) * 16;
    f32x16 s_acc[C::NB];
    auto qk = [&](int i) {
        // one address register per k-step, advanced to the tile's ring slot once; every other
        // displacement is an instruction immediate
        const int slot = (i & (C::NS - 1)) * C::TILE;
        const char* kb[KSV];
#pragma unroll
        for (int dk = 0; dk < KSV; dk++) kb[dk] = smem + (slot + kofs[dk]);
        constexpr int NF = C::NB * KSV;          // fragments in (nb, dk) order
        constexpr int LA = FA_PP_LA;
        auto frag_ptr = [&](int f) { return kb[f % KSV] + (f / KSV) * 32 * C::ROWB; };
        u32x4 fr[LA];
#pragma unroll
        for (int e = 0; e < LA; e++) fr[e] = *reinterpret_cast<const u32x4*>(frag_ptr(e));
#pragma unroll
        for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) s_acc[nb][r] = 0.f;
#pragma unroll
        for (int f = 0; f < NF; f++) {
            s_acc[f / KSV] = Elem<T>::mfma32(__builtin_bit_cast(v8, fr[f % LA]), qf[f % KSV], s_acc[f / KSV]);
            if (f + LA < NF) fr[f % LA] = *reinterpret_cast<const u32x4*>(frag_ptr(f + LA));
        }
        __builtin_amdgcn_sched_group_barrier(0x100, LA, 0);      // look-ahead reads
#pragma unroll
        for (int f = 0; f < NF; f++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
            if (f + LA < NF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 DS read
        }
    };

    // ---- O^T += V^T P^T, same interleave with two transposing reads per MFMA
    const int tj = (lane & 15) >> 2, tq = lane & 3, dhalf = (lane >> 4) & 1;
    int vofs[DBV];
#pragma unroll
    for (int db = 0; db < DBV; db++)
        vofs[db] = (4 * hh + tj) * C::ROWB + swz_v<D>(db * 4 + dhalf * 2 + (tq >> 1), 4 * hh + tj) * 16 + (tq & 1) * 8;
    v8 pf[C::PT];
    auto pv = [&](int i) {
        const int slot = (C::NS + (i & (C::NS - 1))) * C::TILE;
        const char* vb[DBV];
#pragma unroll
        for (int db = 0; db < DBV; db++) vb[db] = smem + (slot + vofs[db]);
        constexpr int NF = C::PT * DBV;          // fragments in (t16, db) order
        constexpr int LA = FA_PP_LA;
        auto fetch = [&](int f) {
            const int t16 = f / DBV, db = f % DBV;
            const u32x2 lo = lds_read_tr16(vb[db] + t16 * 16 * C::ROWB);
            const u32x2 hi = lds_read_tr16(vb[db] + (t16 * 16 + 8) * C::ROWB);
            return (u32x4){lo[0], lo[1], hi[0], hi[1]};
        };
        u32x4 fr[LA];
#pragma unroll
        for (int e = 0; e < LA; e++) fr[e] = fetch(e);
#pragma unroll
        for (int f = 0; f < NF; f++) {
            o_acc[f % DBV] = Elem<T>::mfma32(__builtin_bit_cast(v8, fr[f % LA]), pf[f / DBV], o_acc[f % DBV]);
            if (f + LA < NF) fr[f % LA] = fetch(f + LA);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * LA, 0);  // look-ahead reads
#pragma unroll
        for (int f = 0; f < NF; f++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
            if (f + LA < NF) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // 2 DS reads
        }
    };

    auto softmax = [&](int i) {
        const int tt = tile_of(i);
        if (tt < tf_lo || tt > tf_hi) {
            const int n0 = tt * BN;
            int lim_hi = si.sk - 1;
            if (has_right) lim_hi = min(lim_hi, row + shift + wr);
            const int lim_lo = has_left ? row + shift - wl : 0;
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++) mask_acc16(s_acc[nb], n0 + nb * 32 + 4 * hh, lim_lo, lim_hi);
        }
        {
            // The tile is exponentiated against the reference max the row already has, and only the
            // tile's row sum is looked at afterwards: at most 2^14 means no probability above 2^14 (safe
            // in fp16 / bf16 and in the fp32 sums), so the reference stays and no row max is formed.
            // A larger or non-finite sum in any row of the wave (always the case while a row has no
            // reference: -inf makes every exponent +inf or NaN) takes the rare branch, which forms the
            // exact row max from the untouched scores, moves the reference under the usual rule and
            // exponentiates again.
            uint32_t keep[C::NB][8];
            if constexpr (DROPOUT) {
#pragma unroll
                for (int nb = 0; nb < C::NB; nb++) drop_pairs_row(drop, row, tt * BN + nb * 32, hh, keep[nb]);
            }
            auto exp_tile = [&](float msc) -> float {
                float suma = 0.f, sumb = 0.f;
#pragma unroll
                for (int t16 = 0; t16 < C::PT; t16++) {
                    const int nb = t16 >> 1, r8 = (t16 & 1) * 8;
                    u32x4 pk;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float e0 = fast_exp2(s_acc[nb][r8 + 2 * e] * sl2 - msc);
                        const float e1 = fast_exp2(s_acc[nb][r8 + 2 * e + 1] * sl2 - msc);
                        suma += e0;
                        sumb += e1;
                        // the row sum is of the undropped probabilities; dropped entries leave the second
                        // product only, and 1 / (1 - p) is applied once in the epilogue
                        pk[e] = pack2<T>(e0, e1);
                        if constexpr (DROPOUT) pk[e] &= keep[nb][r8 / 2 + e];
                    }
                    pf[t16] = __builtin_bit_cast(v8, pk);
                }
                return suma + sumb;
            };
            float tsum = exp_tile(m_run * sl2);
            float corr = 1.f;
            if (__builtin_amdgcn_ballot_w64(!(tsum <= 16384.f)) != 0) {
                float mx = -INFINITY;
#pragma unroll
                for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) mx = fmaxf(mx, s_acc[nb][r]);
                mx = xhalf_max(mx);
                // lazy reference max: move it only when the tile max exceeds it by more than 2^8 (exp2 domain)
                const bool move = (mx - m_run) * sl2 > 8.f;       // false for NaN (-inf - -inf)
                const float m_new = move ? mx : m_run;
                corr = move ? fast_exp2((m_run - m_new) * sl2) : 1.f;   // m_run = -inf -> 0
                l_run *= corr;
                m_run = m_new;
                tsum = exp_tile((m_run == -INFINITY) ? 0.f : m_run * sl2);
            }
            l_run += tsum;
            // (tested on corr itself, not on a flag set in the branch above: with a flag the compiler
            // merges this block into that branch and copies all of o_acc around it on every tile)
            if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
                for (int db = 0; db < DBV; db++)
#pragma unroll
                    for (int r = 0; r < 16; r++) o_acc[db][r] *= corr;
            }
        }
    };

    if (nt > 0) {
        // ---- prologue: K(0), V(0), K(1), V(1), K(2) were requested above; S = K(0) Q
        wait_vmcnt<0>();
        __syncthreads();
        if (active(0)) qk(0);
        if (group == 1) __syncthreads();   // group 1 runs one phase behind group 0

        for (int i = 0; i < nt; i++) {
            // ---- Y(i): VALU phase (and requests for the tiles needed 3 iterations ahead)
            if (i + C::PF < nt) fill_k(i + C::PF);
            if (i + C::PF - 1 < nt) fill_v(i + C::PF - 1);
            const bool act = active(i);
            if (act) softmax(i);
            __syncthreads();
            // ---- X(i): MFMA phase
            __builtin_amdgcn_s_setprio(1);
            if (act) pv(i);
            if (i + 1 < nt && active(i + 1)) qk(i + 1);
            __builtin_amdgcn_s_setprio(0);
            // this wave's fills of K(i+2), V(i+1) must have landed before the barrier publishes them;
            // the 2 * LOADS requests of Y(i) may stay in flight
            if (i + C::PF < nt) wait_vmcnt<2 * C::LOADS>(); else wait_vmcnt<0>();
            __syncthreads();
        }
        if (group == 0) __syncthreads();
    }

    // ---- epilogue
    const float l_tot = xhalf_sum(l_run);
    const bool dead = (l_tot == 0.f) || (l_tot != l_tot);
    const float inv = dead ? 1.f : drop.rp / l_tot;
    const float lse = dead ? INFINITY : m_run * p.softmax_scale + __logf(l_tot);
    if (hh == 0 && row < si.sq) p.softmax_lse[((int64_t)b * p.h + head) * p.seqlen_q + row] = lse;
    // The output tile of the wave (32 rows x D) goes through LDS so that every store instruction
    // writes whole rows (16 B per lane, 64 / (D/8) rows per instruction) instead of 8-byte pieces
    // of 32 rows.  All tile reads of the ring are behind the last barrier and each wave uses its
    // own region, so no barrier is needed.
    {
        constexpr int PITCH = C::ROWB + 16;
        char* stage = smem + wave * (32 * PITCH);
#pragma unroll
        for (int db = 0; db < DBV; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int d0 = db * 32 + 8 * q4 + 4 * hh;
                const u32x2 v = {pack2<T>(o_acc[db][4 * q4] * inv, o_acc[db][4 * q4 + 1] * inv),
                                 pack2<T>(o_acc[db][4 * q4 + 2] * inv, o_acc[db][4 * q4 + 3] * inv)};
                *reinterpret_cast<u32x2*>(stage + l32 * PITCH + d0 * 2) = v;
            }
        constexpr int RPP = 64 / C::CPR;                // rows per store instruction
        const int srow = lane / C::CPR, sch = lane % C::CPR;
        T* obase = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)head * p.o_head_stride + sch * 8;
#pragma unroll
        for (int j = 0; j < 32 / RPP; j++) {
            const int rr = j * RPP + srow;
            const u32x4 v = *reinterpret_cast<const u32x4*>(stage + rr * PITCH + sch * 16);
            if (r0 + rr < si.sq && sch * 8 < p.d) st_global16(obase + (int64_t)(r0 + rr) * p.o_row_stride, v);
        }
    }
}

template <typename T, int D, int BN, bool DROPOUT, int DV = D>
int launch_prefill_pp_one(KParams kp, hipStream_t stream) {
    typedef PPCfg<T, D, BN> C;
    kp.num_m_blocks = (kp.p.seqlen_q + C::BM - 1) / C::BM;
    const int64_t total = (int64_t)kp.num_m_blocks * kp.p.h * kp.p.b;
    if (total <= 0) return 0;
    const int64_t nblocks = xcd_grid(kp.p, kp.num_m_blocks);
    if (nblocks == 0) return -2;
    dim3 grid((unsigned)nblocks), block(C::kThreads);
    if (int e = prepare_work_list(kp, C::BM, nblocks, stream)) return e;
    auto kern = prefill_pp_kernel<T, D, BN, DROPOUT, DV>;
    hipError_t e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    return note_kernel((int)hipGetLastError(), FA_KERNEL_PINGPONG, DROPOUT, false, DV);
}
}  // namespace fa
