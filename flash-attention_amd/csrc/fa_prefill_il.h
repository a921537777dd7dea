// Software-pipelined forward kernel for gfx950: 4 waves x 32 query rows, two workgroups per CU.
//
// Same mathematics, register layouts and LDS tile format as prefill_pp_kernel (fa_prefill_pp.h):
// S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16 with one query row per lane, K/V tiles of 64
// keys moved global -> LDS by global_load_lds_dwordx4.  What differs is the schedule.  Every wave
// runs the three independent pieces of work of one loop step in ONE instruction stream:
//
//     step i:   O += P(i-1) V(i-1)      (16 MFMA for head dim 128)
//               S(i+1) = K(i+1) Q       (16 MFMA)
//               P(i) = softmax(S(i))    (vector/transcendental work)
//
// written as one chunk per matrix instruction (the MFMA, the LDS fragment read a few chunks ahead,
// a slice of the softmax) with scheduling barriers between chunks, so the matrix pipe of a SIMD is
// fed by whichever of its two resident waves is ready.  Those two waves belong to DIFFERENT
// workgroups (128 query rows and a 64 KB two-slot K/V ring each), so they never wait for each other,
// and the start-up and output phases of one workgroup overlap the steady state of the other.  The
// price is that each K/V tile is fetched from L2 once per 128 rows instead of once per 256: the
// ping-pong kernel stays ahead for long non-causal sequences at head dim 128, this one wins for
// shorter sequences and for head dim 64.  S and P are double-buffered in registers (the loop is
// unrolled by two so that the buffers alternate without copies).
//
// Steps whose tile needs masking, and the first and last steps, run the same three pieces one
// after the other ("plain" step).  The running max is lazy as in the ping-pong kernel; the rescale
// of O that a moved max needs is applied after the step's matrix instructions.
#pragma once
#include "fa_common.h"
#include "fa_launch.h"
#include "fa_prefill_pp.h"

namespace fa {

#ifndef FA_IL_LA
#define FA_IL_LA 4
#endif

// One query-row group of 32 rows per wave, the whole head dimension in that wave.  Up to head dim 128 two
// (three at 64) workgroups share a CU; at head dim 256 O (128 accumulator registers) and the Q fragments (64)
// leave room for one wave per SIMD only, which then has all 512 registers and 160 KB of LDS to itself.
// DV_: head dims the products run over (a multiple of 32, d <= DV_ <= D_); tiles keep the LDS layout of the
// bucket D_ (head dim 96 runs on the 128 bucket with 6 of 8 k-steps and 3 of 4 output column blocks).
template <typename T, int D_, int BN_, int DV_ = D_>
struct ILCfg {
    static constexpr int D = D_, BN = BN_;
    static constexpr bool kPair = false;
    static constexpr int kKernelId = D_ > 128 ? FA_KERNEL_WIDE : FA_KERNEL_PIPELINED, kHeadDims = DV_;   // for fa_last_kernel
    static constexpr int kThreads = 256;
    static constexpr int kWaves = 4;
    static constexpr int BM = kWaves * 32;
    static constexpr int DH = DV_;                          // head-dim slice of one wave
    static constexpr int NB = BN / 32;
    static constexpr int KS = DH / 16;
    static constexpr int DB = DH / 32;
    static constexpr int PT = BN / 16;
    static constexpr int CPR = D / 8;                       // 16 B chunks per tile row
    static constexpr int ROWB = D * 2;
    static constexpr int TILE = BN * ROWB;                  // bytes of one K or V tile
    static constexpr int NS = 2;                            // ring slots per tensor
    static constexpr int LOADS = BN * CPR / kThreads;       // 16 B fills per thread per tile
    static constexpr int ROWS_PER_PASS = kThreads / CPR;
    static constexpr int PASSB = kThreads * 16;             // LDS bytes filled by one pass of the workgroup
    static constexpr int XCH = 0;
    static constexpr int OUT_LANES = DH / 8 <= 8 ? 8 : DH / 8 <= 16 ? 16 : 32;      // lanes per output row in the epilogue
    static constexpr int STAGE = kWaves * 32 * (OUT_LANES * 16 + 16);              // output staging of the epilogue
    static constexpr int SMEM = 2 * NS * TILE > STAGE ? 2 * NS * TILE : STAGE;      // K ring, then V ring
    static_assert((BN * CPR) % kThreads == 0 && 64 % CPR == 0, "tile shape");
};

// Head dim 256 with two waves per SIMD (the form that runs with dropout, whose mask arithmetic needs a second
// wave to hide behind): two waves share each group of 32 query rows and split the head
// dimension between them.  Each computes the partial scores over its 128 columns of Q and K,
// the two partial S tiles are exchanged through LDS and added (both waves then hold the same S
// and run the same softmax), and each accumulates its own 128 columns of O.  8 waves, 128 rows
// per workgroup, 32-key tiles, one workgroup per CU.
template <typename T, int DV_ = 256>
struct ILCfgPair {
    static constexpr int D = 256, BN = 32;
    static constexpr bool kPair = true;
    static constexpr int kKernelId = FA_KERNEL_WIDE_PAIR, kHeadDims = DV_;
    static constexpr int kThreads = 512;
    static constexpr int kWaves = 8;
    static constexpr int BM = (kWaves / 2) * 32;
    static constexpr int DH = DV_ / 2;                      // 128, or 96 for head dims up to 192
    static constexpr int NB = BN / 32;
    static constexpr int KS = DH / 16;
    static constexpr int DB = DH / 32;
    static constexpr int PT = BN / 16;
    static constexpr int CPR = D / 8;
    static constexpr int ROWB = D * 2;
    static constexpr int TILE = BN * ROWB;
    static constexpr int NS = 2;
    static constexpr int LOADS = BN * CPR / kThreads;
    static constexpr int ROWS_PER_PASS = kThreads / CPR;
    static constexpr int PASSB = kThreads * 16;
    static constexpr int XCH = NB * 16 * 64 * 4;            // one partial S tile of a wave, fp32
    static constexpr int SMEM = 2 * NS * TILE + kWaves * 2 * XCH;   // rings, then two exchange tiles per wave
    static_assert((BN * CPR) % kThreads == 0, "tile shape");
};

// Occupancy: two workgroups per CU at head dim 128 (about 250 registers); at head dim 64, where the
// vector work per matrix instruction doubles and a third wave per SIMD adds the issue slots it needs,
// three workgroups in 168 registers each (measured +3..10 %); the dropout variant, whose mask arithmetic
// does not fit 168 registers without spilling, stays at two; one wave per SIMD (all 512 registers) for the
// whole-head-dim form at 256.
template <typename T, typename C, bool DROPOUT = false>
__global__ void __launch_bounds__(C::kThreads, (!C::kPair && C::D == 256) ? 1 : (!C::kPair && C::D == 64 && !DROPOUT) ? 3 : 2) prefill_il_kernel(const KParams kp) {
    constexpr int D = C::D, BN = C::BN;
    typedef typename Elem<T>::v8 v8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const fa_fwd_params& p = kp.p;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int l32 = lane & 31, hh = lane >> 5;

    const int G = p.h / p.h_k;
    int g, mb, hk, b;
    if (!xcd_work_item(kp, (uint32_t)kp.num_m_blocks,
                       !(kp.has_left || kp.has_right) ? 0u : (C::kPair || C::D == 256) ? 32u : ((C::D == 64 && !DROPOUT) ? 96u : 64u), g, mb, hk, b)) return;
    const int head = hk * G + g;

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

    // first query row of this wave, and the first head-dim column it owns
    const int r0 = m0 + (C::kPair ? (wave >> 1) : wave) * 32;
    const int row = r0 + l32;
    const int dcol0 = C::kPair ? (wave & 1) * C::DH : 0;

    v8 qf[C::KS];
    {
        const bool valid = row < si.sq;
        const T* qrow = qg + (int64_t)row * p.q_row_stride;
#pragma unroll
        for (int dk = 0; dk < C::KS; dk++) {
            const int d0 = dcol0 + dk * 16 + 8 * hh;
            u32x4 raw = {0, 0, 0, 0};
            if (valid && d0 < p.d) raw = ld_global16(qrow + d0);
            qf[dk] = __builtin_bit_cast(v8, raw);
        }
    }

    f32x16 o_acc[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[db][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    // dropout: the row sums are of the undropped probabilities; dropped entries leave the second
    // product only, and 1 / (1 - p) is applied once in the epilogue
    Drop drop = {0, 0, 256, 1.f};
    if constexpr (DROPOUT) drop = drop_init(p.rng_state, p.p_dropout, b, head, p.h);
    const float sl2 = kp.scale_log2;

    // visit i of the key loop handles key tile t_hi - 1 - i and uses ring slot i % NS
    auto tile_of = [&](int i) { return t_hi - 1 - i; };

    // ---- asynchronous tile fills (layout as in prefill_pp_kernel)
    const int frow = (wave * 64 + lane) / C::CPR;
    const int fch = lane % C::CPR;
    const int kch = min(swz_k<D>(fch, frow), p.d / 8 - 1);
    // (a pass of fewer than 16 rows -- 256 lanes at head dim 256 cover 8 -- alternates between two row
    // phases of the K swizzle: odd passes take their own chunk)
    constexpr bool kTwoPhases = (C::ROWS_PER_PASS % 16) != 0;
    static_assert(!kTwoPhases || C::ROWS_PER_PASS == 8, "K swizzle phase per pass");
    const int kch1 = kTwoPhases ? min(swz_k<D>(fch, frow + C::ROWS_PER_PASS), p.d / 8 - 1) : kch;
    const int vch = min(swz_v<D>(fch, frow), p.d / 8 - 1);
    const uint32_t lds0 = (uint32_t)(size_t)((FA_LDS_PTR(char))smem);
    const uint32_t fill_base = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(wave * 1024));
    // Scalar base of the tile (uniform over the workgroup) + a 32-bit per-lane byte offset: the
    // fill instruction takes its address as SGPR pair + VGPR offset, and moving on to the next tile
    // is scalar arithmetic.
    const int64_t kstep = (int64_t)BN * p.k_row_stride, vstep = (int64_t)BN * p.v_row_stride;
    const int64_t kpass = (int64_t)C::ROWS_PER_PASS * p.k_row_stride, vpass = (int64_t)C::ROWS_PER_PASS * p.v_row_stride;
    const T* ktile = scalar_ptr(kg + (int64_t)(t_hi - 1) * BN * p.k_row_stride);     // uniform
    const T* vtile = scalar_ptr(vg + (int64_t)(t_hi - 1) * BN * p.v_row_stride);
    const uint32_t koff = (uint32_t)(((int64_t)frow * p.k_row_stride + kch * 8) * 2);
    const uint32_t koff1 = (uint32_t)(((int64_t)frow * p.k_row_stride + kch1 * 8) * 2);
    const uint32_t voff = (uint32_t)(((int64_t)frow * p.v_row_stride + vch * 8) * 2);
    const bool tail_clamp = t_hi * BN > si.sk;    // only visit 0 can reach past seqlen_k
    auto fill_s = [&](const T* base, uint32_t off, uint32_t dst) { async_fill16(base, off, dst); };
    auto fill_k = [&](int i) {
        const uint32_t dst = fill_base + (uint32_t)((i & (C::NS - 1)) * C::TILE);
        if (i == 0 && tail_clamp) {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) {
                const int n = min(frow + j * C::ROWS_PER_PASS, si.sk - 1 - (t_hi - 1) * BN);
                fill_s(ktile, (uint32_t)(((int64_t)n * p.k_row_stride + ((j & 1) ? kch1 : kch) * 8) * 2), dst + j * C::PASSB);
            }
        } else {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) fill_s(ktile + j * kpass, (j & 1) ? koff1 : koff, dst + j * C::PASSB);
        }
        ktile -= kstep;
    };
    auto fill_v = [&](int i) {
        const uint32_t dst = fill_base + (uint32_t)((C::NS + (i & (C::NS - 1))) * C::TILE);
        if (i == 0 && tail_clamp) {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) {
                const int n = min(frow + j * C::ROWS_PER_PASS, si.sk - 1 - (t_hi - 1) * BN);
                fill_s(vtile, (uint32_t)(((int64_t)n * p.v_row_stride + vch * 8) * 2), dst + j * C::PASSB);
            }
        } else {
#pragma unroll
            for (int j = 0; j < C::LOADS; j++) fill_s(vtile + j * vpass, voff, dst + j * C::PASSB);
        }
        vtile -= vstep;
    };

    // Tiles in [tf_lo, tf_hi] (absolute key-tile index) are fully visible to all 32 rows of the wave.
    int tf_lo = 0, tf_hi = si.sk / BN - 1;
    if (has_right) {
        const int c = r0 + shift + wr;            // last visible key of the wave's first row
        tf_hi = min(tf_hi, (c + 1 >= BN) ? (c + 1) / BN - 1 : -1);
    }
    if (has_left) {
        const int c = r0 + shift - wl;            // first visible key of the wave's first row
        tf_lo = (c + 31 > 0) ? (c + 31 + BN - 1) / BN : 0;
    }

    // ---- LDS fragment addressing
    int kofs[C::KS];
#pragma unroll
    for (int dk = 0; dk < C::KS; dk++) kofs[dk] = l32 * C::ROWB + swz_k<D>(dcol0 / 8 + dk * 2 + hh, l32) * 16;
    const int tj = (lane & 15) >> 2, tq = lane & 3, dhalf = (lane >> 4) & 1;
    int vofs[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++)
        vofs[db] = (4 * hh + tj) * C::ROWB + swz_v<D>(dcol0 / 8 + db * 4 + dhalf * 2 + (tq >> 1), 4 * hh + tj) * 16 + (tq & 1) * 8;

    constexpr int LA = FA_IL_LA;
    constexpr int NFV = C::PT * C::DB;             // V fragments in (t16, db) order
    constexpr int NFK = C::NB * C::KS;             // K fragments in (nb, dk) order
    static_assert(LA <= NFV && LA <= NFK, "look-ahead depth");

    // The matrix stream of one step: O += P(iv) V(iv) when PV, then s_out = K(ik) Q when QK.
    // Fragment reads run LA matrix instructions ahead.
    auto mma = [&](auto with_pv, auto with_qk, int iv, int ik, const v8 (&pf)[C::PT],
                   f32x16 (&s_out)[C::NB]) __attribute__((always_inline)) {
        constexpr bool PV = decltype(with_pv)::value, QK = decltype(with_qk)::value;
        constexpr int F0 = PV ? 0 : NFV, F1 = QK ? NFV + NFK : NFV;
        const int vslot = (C::NS + (iv & (C::NS - 1))) * C::TILE;
        const int kslot = (ik & (C::NS - 1)) * C::TILE;
        const char* vb[C::DB];
        const char* kb[C::KS];
        if (PV) {
#pragma unroll
            for (int db = 0; db < C::DB; db++) vb[db] = smem + (vslot + vofs[db]);
        }
        if (QK) {
#pragma unroll
            for (int dk = 0; dk < C::KS; dk++) kb[dk] = smem + (kslot + kofs[dk]);
        }
        auto fetch = [&](int f) {
            if (f < NFV) {
                const int t16 = f / C::DB, db = f % C::DB;
                const u32x2 lo = lds_read_tr16(vb[db] + t16 * 16 * C::ROWB);
                const u32x2 hi = lds_read_tr16(vb[db] + (t16 * 16 + 8) * C::ROWB);
                return (u32x4){lo[0], lo[1], hi[0], hi[1]};
            }
            const int gk = f - NFV;
            return *reinterpret_cast<const u32x4*>(kb[gk % C::KS] + (gk / C::KS) * 32 * C::ROWB);
        };
        u32x4 fr[LA];
#pragma unroll
        for (int e = 0; e < LA; e++) fr[e] = fetch(F0 + e);
#pragma unroll
        for (int f = F0; f < F1; f++) {
            const v8 a = __builtin_bit_cast(v8, fr[(f - F0) % LA]);
            if (f < NFV) {
                o_acc[f % C::DB] = Elem<T>::mfma32(a, pf[f / C::DB], o_acc[f % C::DB]);
            } else {
                const int gk = f - NFV, nb = gk / C::KS, dk = gk % C::KS;
                if (dk == 0) {
                    f32x16 z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0.f;
                    s_out[nb] = Elem<T>::mfma32(a, qf[dk], z);
                } else {
                    s_out[nb] = Elem<T>::mfma32(a, qf[dk], s_out[nb]);
                }
            }
            if (f + LA < F1) fr[(f - F0) % LA] = fetch(f + LA);
        }
        // look-ahead reads first
        __builtin_amdgcn_sched_group_barrier(0x100, PV ? 2 * LA : LA, 0);
#pragma unroll
        for (int f = F0; f < F1; f++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                            // 1 MFMA
            if (f + LA < NFV) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);          // V fragment
            else if (f + LA < F1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // K fragment
        }
    };

    // ---- softmax pieces.  decide(): tile max, lazy reference-max update; returns the factor the
    // old O and row sum must be scaled by (1 when the reference max did not move).
    auto mask_tile = [&](int i, f32x16 (&s)[C::NB]) __attribute__((always_inline)) {
        const int tt = tile_of(i);
        if (tt < tf_lo || tt > tf_hi) {
            const int n0 = tt * BN;
            int lim_hi = si.sk - 1;
            if (has_right) lim_hi = min(lim_hi, row + shift + wr);
            const int lim_lo = has_left ? row + shift - wl : 0;
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++) mask_acc16(s[nb], n0 + nb * 32 + 4 * hh, lim_lo, lim_hi);
        }
    };
    auto probs = [&](int i, const f32x16 (&s)[C::NB], v8 (&pf)[C::PT], float& corr_out, bool& move_out, float sl2) __attribute__((always_inline)) {
        uint32_t keep[C::NB][8];      // per pair of registers: 0xffff in the half of a kept element
        if constexpr (DROPOUT) {
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++) drop_pairs_row(drop, row, tile_of(i) * C::BN + nb * 32, hh, keep[nb]);
        }
        float mx = -INFINITY;
#pragma unroll
        for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[nb][r]);
        mx = xhalf_max(mx);
        // lazy reference max: move it only when the tile max exceeds it by more than 2^8 (exp2 domain)
        const bool move = (mx - m_run) * sl2 > 8.f;       // false for NaN (-inf - -inf)
        const float m_new = move ? mx : m_run;
        const float corr = move ? fast_exp2((m_run - m_new) * sl2) : 1.f;   // m_run = -inf -> 0
        m_run = m_new;
        const float msc = (m_new == -INFINITY) ? 0.f : m_new * sl2;
        float suma = 0.f, sumb = 0.f;
#pragma unroll
        for (int t16 = 0; t16 < C::PT; t16++) {
            const int nb = t16 >> 1, r8 = (t16 & 1) * 8;
            u32x4 pk;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float e0 = fast_exp2(s[nb][r8 + 2 * e] * sl2 - msc);
                const float e1 = fast_exp2(s[nb][r8 + 2 * e + 1] * sl2 - msc);
                suma += e0;
                sumb += e1;
                pk[e] = pack2<T>(e0, e1);
                if constexpr (DROPOUT) pk[e] &= keep[nb][r8 / 2 + e];
            }
            pf[t16] = __builtin_bit_cast(v8, pk);
        }
        l_run = l_run * corr + (suma + sumb);
        corr_out = corr;
        move_out = move;
    };
    auto rescale = [&](float corr, bool move) __attribute__((always_inline)) {
        if (__builtin_amdgcn_ballot_w64(move) != 0) {
#pragma unroll
            for (int db = 0; db < C::DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o_acc[db][r] *= corr;
        }
    };

    // Pair mode: the partial S tile of step i lives in exchange slot i & 1 of the wave that made it
    // (same lane, same register order on both sides, so writer and reader use identical addresses).
    // A slot written at the end of step i-1 is read by the partner at the start of step i and
    // rewritten at the end of step i+1; the barriers closing steps i-1 and i order the three.
    auto xch_ptr = [&](int w, int i) { return smem + 2 * C::NS * C::TILE + (w * 2 + (i & 1)) * C::XCH + lane * 16; };
    auto xch_write = [&](int i, const f32x16 (&s)[C::NB]) __attribute__((always_inline)) {
        if constexpr (C::kPair) {
            char* base = xch_ptr(wave, i);
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    const f32x4 v = {s[nb][4 * r4], s[nb][4 * r4 + 1], s[nb][4 * r4 + 2], s[nb][4 * r4 + 3]};
                    *reinterpret_cast<f32x4*>(base + (nb * 4 + r4) * 1024) = v;
                }
        }
    };
    auto xch_read_add = [&](int i, f32x16 (&s)[C::NB]) __attribute__((always_inline)) {
        if constexpr (C::kPair) {
            const char* base = xch_ptr(wave ^ 1, i);
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(base + (nb * 4 + r4) * 1024);
                    s[nb][4 * r4] += v[0]; s[nb][4 * r4 + 1] += v[1]; s[nb][4 * r4 + 2] += v[2]; s[nb][4 * r4 + 3] += v[3];
                }
        }
    };

    f32x16 sA[C::NB], sB[C::NB];
    v8 pA[C::PT], pB[C::PT];
#pragma unroll
    for (int t = 0; t < C::PT; t++)
#pragma unroll
        for (int e = 0; e < 8; e++) { pA[t][e] = (T)0.f; pB[t][e] = (T)0.f; }

    // Two-slot rings.  Step i reads V(i-1) and K(i+1).  When it opens, every wave of the workgroup
    // has passed the barrier that closed step i-1, so the slots of V(i-2) and K(i) are free: the
    // step requests V(i) and K(i+2) into them, and closes by waiting for those requests before
    // the barrier that publishes them.  The second workgroup resident on the CU (its own rings)
    // keeps the SIMDs busy while this one waits.
    auto open_step = [&](int i) __attribute__((always_inline)) {
        if (i < nt) fill_v(i);
        if (i + 2 < nt) fill_k(i + 2);
    };
    auto advance_ring = [&](int i) __attribute__((always_inline)) {
        wait_vmcnt<0>();
        __syncthreads();
    };
    // Steady-state step: s_cur holds S(i), p_prev holds P(i-1); leaves S(i+1) in s_nxt and P(i) in
    // p_cur.  The step is written as NF chunks, one per matrix instruction: the MFMA, the fragment
    // read LA chunks ahead, and a slice of the softmax of S(i) (running max in the first chunks,
    // then the decision about the reference max, then the exponentials two at a time).  Scheduling
    // barriers between the chunks keep the compiler from regrouping them.
    auto fast_step = [&](int i, f32x16 (&s_cur)[C::NB], f32x16 (&s_nxt)[C::NB], const v8 (&p_prev)[C::PT],
                         v8 (&p_cur)[C::PT]) __attribute__((always_inline)) {
        constexpr int NF = NFV + NFK;
        constexpr int NE = C::NB * 16;             // S elements per lane
        constexpr int NP = NE / 2;                 // pairs
        constexpr int CM = 3;                      // chunks that take the running max
        constexpr int CD = CM;                     // chunk of the decision
        constexpr int CE = CD + 1;                 // first chunk with exponentials
        static_assert(NF > CE + 1, "tile too small for the chunked step");
        open_step(i);
        xch_read_add(i, s_cur);
        if constexpr (!C::kPair) mask_tile(i, s_cur);
        // an opaque copy of the scale keeps the vector work in this block (behind the barrier)
        float sc = sl2;
        asm volatile("" : "+v"(sc));
        const int vslot = (C::NS + ((i - 1) & (C::NS - 1))) * C::TILE;
        const int kslot = ((i + 1) & (C::NS - 1)) * C::TILE;
        const char* vb[C::DB];
        const char* kb[C::KS];
#pragma unroll
        for (int db = 0; db < C::DB; db++) vb[db] = smem + (vslot + vofs[db]);
#pragma unroll
        for (int dk = 0; dk < C::KS; dk++) kb[dk] = smem + (kslot + kofs[dk]);
        auto fetch = [&](int f) {
            if (f < NFV) {
                const int t16 = f / C::DB, db = f % C::DB;
                const u32x2 lo = lds_read_tr16(vb[db] + t16 * 16 * C::ROWB);
                const u32x2 hi = lds_read_tr16(vb[db] + (t16 * 16 + 8) * C::ROWB);
                return (u32x4){lo[0], lo[1], hi[0], hi[1]};
            }
            const int gk = f - NFV;
            return *reinterpret_cast<const u32x4*>(kb[gk % C::KS] + (gk / C::KS) * 32 * C::ROWB);
        };
        u32x4 fr[LA];
#pragma unroll
        for (int e = 0; e < LA; e++) fr[e] = fetch(e);
        __builtin_amdgcn_sched_barrier(0);

        float mx = -INFINITY, msc = 0.f, corr = 1.f, suma = 0.f, sumb = 0.f;
        bool move = false;
        uint32_t pk[NP];
        uint32_t keep[C::NB][8];      // per pair of registers: 0xffff in the half of a kept element
        if constexpr (DROPOUT) {
#pragma unroll
            for (int nb = 0; nb < C::NB; nb++) drop_pairs_row(drop, row, tile_of(i) * C::BN + nb * 32, hh, keep[nb]);
        }
#pragma unroll
        for (int f = 0; f < NF; f++) {
            // ---- matrix instruction f and the read for f + LA
            const v8 a = __builtin_bit_cast(v8, fr[f % LA]);
            if (f < NFV) {
                o_acc[f % C::DB] = Elem<T>::mfma32(a, p_prev[f / C::DB], o_acc[f % C::DB]);
            } else {
                const int gk = f - NFV, nb = gk / C::KS, dk = gk % C::KS;
                if (dk == 0) {
                    f32x16 z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0.f;
                    s_nxt[nb] = Elem<T>::mfma32(a, qf[dk], z);
                } else {
                    s_nxt[nb] = Elem<T>::mfma32(a, qf[dk], s_nxt[nb]);
                }
            }
            if (f + LA < NF) fr[f % LA] = fetch(f + LA);
            // ---- vector slice f
            if (f < CM) {
#pragma unroll
                for (int e = f * NE / CM; e < (f + 1) * NE / CM; e++) mx = fmaxf(mx, s_cur[e / 16][e % 16]);
            }
            if (f == CD) {
                mx = xhalf_max(mx);
                move = (mx - m_run) * sc > 8.f;               // false for NaN (-inf - -inf)
                const float m_new = move ? mx : m_run;
                corr = move ? fast_exp2((m_run - m_new) * sc) : 1.f;
                m_run = m_new;
                msc = (m_new == -INFINITY) ? 0.f : m_new * sc;
            }
            if (f >= CE) {
#pragma unroll
                for (int pr = 0; pr < NP; pr++) {
                    if (CE + (pr * (NF - CE)) / NP == f) {
                        const float e0 = fast_exp2(s_cur[(2 * pr) / 16][(2 * pr) % 16] * sc - msc);
                        const float e1 = fast_exp2(s_cur[(2 * pr + 1) / 16][(2 * pr + 1) % 16] * sc - msc);
                        suma += e0;
                        sumb += e1;
                        pk[pr] = pack2<T>(e0, e1);
                        if constexpr (DROPOUT) pk[pr] &= keep[pr / 8][pr % 8];
                    }
                }
            }
            if (f == NF - 1) l_run = l_run * corr + (suma + sumb);
            __builtin_amdgcn_sched_barrier(0);
        }
        // pin the step's results here, or the compiler sinks the vector work past the branch below,
        // out of the block that holds the matrix instructions
#pragma unroll
        for (int t = 0; t < C::PT; t++) {
            u32x4 u = {pk[4 * t], pk[4 * t + 1], pk[4 * t + 2], pk[4 * t + 3]};
            asm volatile("" : "+v"(u));
            p_cur[t] = __builtin_bit_cast(v8, u);
        }
        asm volatile("" : "+v"(l_run));
        rescale(corr, move);
        xch_write(i + 1, s_nxt);
        advance_ring(i);
    };
    // Plain step (first, last and masked tiles): the same pieces one after the other; S stays in sA
    // and P in pA.
    auto plain_step = [&](int i) __attribute__((always_inline)) {
        open_step(i);
        xch_read_add(i, sA);
        if (i > 0) mma(std::true_type(), std::false_type(), i - 1, 0, pA, sB);
        if (i + 1 < nt) {
            mma(std::false_type(), std::true_type(), 0, i + 1, pA, sB);
            xch_write(i + 1, sB);
        }
        mask_tile(i, sA);
        float corr; bool move;
        probs(i, sA, pA, corr, move, sl2);
        rescale(corr, move);
#pragma unroll
        for (int nb = 0; nb < C::NB; nb++) sA[nb] = sB[nb];
        advance_ring(i);
    };

    if (nt > 0) {
        // ---- prologue: K(0), K(1); S(0) = K(0) Q
        fill_k(0);
        if (nt > 1) fill_k(1);
        wait_vmcnt<0>();
        __syncthreads();
        mma(std::false_type(), std::true_type(), 0, 0, pA, sA);
        xch_write(0, sA);
        __syncthreads();      // K(0)'s ring slot is refilled when step 0 opens

        // Steps [i_fb, i_fe), an even number of them, take the chunked form.  With the whole head
        // dimension in one wave that is every step but the first and the last (the mask is applied on
        // the way in); in pair mode only the tiles that need no masking for this wave (measured: the
        // masked tiles are faster there as plain steps).
        int i_fb = C::kPair ? max(1, t_hi - 1 - tf_hi) : 1;
        int i_fe = C::kPair ? min(nt - 1, t_hi - tf_lo) : nt - 1;
        i_fb = __builtin_amdgcn_readfirstlane(min(i_fb, nt));
        i_fe = __builtin_amdgcn_readfirstlane(i_fe <= i_fb ? i_fb : i_fb + ((i_fe - i_fb) & ~1));
        int i = 0;
        for (; i < i_fb; i++) plain_step(i);
        for (; i < i_fe; i += 2) {
            fast_step(i, sA, sB, pA, pB);
            fast_step(i + 1, sB, sA, pB, pA);
        }
        for (; i < nt; i++) plain_step(i);
        mma(std::true_type(), std::false_type(), nt - 1, 0, pA, sB);
        __syncthreads();      // the output staging below reuses the ring this product has just read
    }

    // ---- epilogue
    const float l_tot = xhalf_sum(l_run);
    const bool dead = (l_tot == 0.f) || (l_tot != l_tot);
    const float inv = dead ? 1.f : drop.rp / l_tot;
    const float lse = dead ? INFINITY : m_run * p.softmax_scale + __logf(l_tot);
    if (hh == 0 && dcol0 == 0 && row < si.sq) p.softmax_lse[((int64_t)b * p.h + head) * p.seqlen_q + row] = lse;
    // output tile of the wave (32 rows x DH columns) through LDS (whole rows per store instruction); all ring reads are
    // behind the barrier that follows the last product and each wave uses its own region
    {
        constexpr int OCPR = C::DH / 8;                 // 16 B chunks per output row of the wave
        constexpr int OCPP = OCPR <= 8 ? 8 : OCPR <= 16 ? 16 : 32;   // lanes per row in a store instruction (a power of two)
        constexpr int PITCH = OCPP * 16 + 16;
        static_assert(C::kWaves * 32 * PITCH <= C::SMEM, "staging region");
        char* stage = smem + wave * (32 * PITCH);
#pragma unroll
        for (int db = 0; db < C::DB; db++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int d0 = db * 32 + 8 * q4 + 4 * hh;
                const u32x2 v = {pack2<T>(o_acc[db][4 * q4] * inv, o_acc[db][4 * q4 + 1] * inv),
                                 pack2<T>(o_acc[db][4 * q4 + 2] * inv, o_acc[db][4 * q4 + 3] * inv)};
                *reinterpret_cast<u32x2*>(stage + l32 * PITCH + d0 * 2) = v;
            }
        constexpr int RPP = 64 / OCPP;
        const int srow = lane / OCPP, sch = lane % OCPP;
        T* obase = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)head * p.o_head_stride + dcol0 + sch * 8;
#pragma unroll
        for (int j = 0; j < 32 / RPP; j++) {
            const int rr = j * RPP + srow;
            const u32x4 v = *reinterpret_cast<const u32x4*>(stage + rr * PITCH + sch * 16);
            if (r0 + rr < si.sq && sch < OCPR && dcol0 + sch * 8 < p.d) st_global16(obase + (int64_t)(r0 + rr) * p.o_row_stride, v);
        }
    }
}

template <typename T, typename C, bool DROPOUT>
int launch_prefill_il_one(KParams kp, hipStream_t stream) {
    kp.num_m_blocks = (kp.p.seqlen_q + C::BM - 1) / C::BM;
    const int64_t total = (int64_t)kp.num_m_blocks * kp.p.h * kp.p.b;
    if (total <= 0) return 0;
    const int64_t nblocks = xcd_grid(kp.p, kp.num_m_blocks);
    if (nblocks == 0) return -2;
    dim3 grid((unsigned)nblocks), block(C::kThreads);
    if (int e = prepare_work_list(kp, C::BM, nblocks, stream)) return e;
    auto kern = prefill_il_kernel<T, C, DROPOUT>;
    hipError_t e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    return note_kernel((int)hipGetLastError(), C::kKernelId, DROPOUT, false, C::kHeadDims);
}

template <typename T, typename C>
int launch_prefill_il_cfg(const KParams& kp, hipStream_t stream) {
    return kp.p.p_dropout > 0.f ? launch_prefill_il_one<T, C, true>(kp, stream) : launch_prefill_il_one<T, C, false>(kp, stream);
}
// The reference's head-dim buckets 32 and 96 (csrc/flash_attn/src/flash_fwd_launch_template.h:141-149, 179-205) run on
// the tiles of the next larger bucket with the k-steps and output column blocks past the head dim left out.
template <typename T, int D, int BN>
int launch_prefill_il(const KParams& kp, hipStream_t stream) {
    if constexpr (D == 128) {
        if (kp.p.d <= 96 && !(kp.p.p_dropout > 0.f)) return launch_prefill_il_one<T, ILCfg<T, D, BN, 96>, false>(kp, stream);
    }
    if constexpr (D == 64) {
        if (kp.p.d <= 32 && !(kp.p.p_dropout > 0.f)) return launch_prefill_il_one<T, ILCfg<T, D, BN, 32>, false>(kp, stream);
    }
    return launch_prefill_il_cfg<T, ILCfg<T, D, BN>>(kp, stream);
}
// Head dims 129..256 with dropout: the pair form (without dropout those head dims run on the 8-wave kernel of
// fa_prefill_pp16.h with 16 query rows per wave, measured 7-18 % ahead of the whole-head-dim form ILCfg<T, 256, 32, DV>
// of this kernel, one wave per SIMD with all 512 registers, which is no longer instantiated).
template <typename T>
int launch_prefill_il_256(const KParams& kp, hipStream_t stream) {
    return launch_prefill_il_one<T, ILCfgPair<T>, true>(kp, stream);
}

}  // namespace fa
