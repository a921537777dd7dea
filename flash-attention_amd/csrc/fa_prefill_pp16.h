// The 8-wave ping-pong forward kernel of fa_prefill_pp.h on v_mfma_f32_16x16x32 instead of v_mfma_f32_32x32x16.
//
// Why the other instruction: on Gaussian operands the part does not hold its clock.  A kernel that only issues matrix
// instructions on random bf16 data sustains 1.85 PFLOP/s with 32x32x16 and 2.12 with 16x16x32 (the clock settles near
// 1.8 against 2.05 GHz): per flop the small shape moves half the accumulator registers (4 registers in and out per 16K
// flops against 16 per 32K).  This kernel runs at 2.05 GHz where its 32x32x16 form ran at 1.69.
//
// What stays: the work order, the tile ring (global_load_lds straight into LDS, 4 slots per tensor, 3 tiles ahead),
// the two wave groups one phase apart, the lazy reference maximum with the max-free fast path, the staged output.
// What changes is the register geometry.  A wave owns 32 query rows (16 at head dims above 192) as blocks of 16 (rb):
//   * lane (m = lane & 15, g = lane >> 4) holds, for each rb, query row 16 rb + m;
//   * S^T = K Q^T per 16-key block kb: A = K rows (lane: key m of the block, head dims 32 c + 8 g .. + 7, one
//     ds_read_b128), B = the resident Q fragment (row m, same head dims); the lane receives keys 4 g .. 4 g + 3 of
//     the block for its row.  One K fragment feeds every row block of the wave;
//   * O^T += V^T P^T per 32 keys: the lane's probabilities of two neighbouring key blocks, packed, are the B operand
//     (k slots 0-3 <-> keys 4 g + j of the first block, 4-7 <-> the second), the A operand is V^T read by two
//     transposing ds_read_b64_tr_b16 of the same keys; the lane accumulates head dims 16 db + 4 g .. + 3 of its row;
//   * a row's keys are spread over the 4 lanes m, m + 16, m + 32, m + 48: row sums stay per lane until the epilogue,
//     the (rare) exact maximum is reduced over those lanes.
#pragma once
#include <type_traits>
#include "fa_prefill_pp.h"

namespace fa {

// mask of one 16-key accumulator block: entry r stands at key pos0 + r, visible iff lo <= key <= hi
FA_DEV void mask_acc4(f32x4& s, int pos0, int lo, int hi) {
    const bool any = hi >= lo;
    const uint32_t span = any ? (uint32_t)(hi - lo) : 0u;
    const int z = any ? pos0 - lo : -64;
#pragma unroll
    for (int r = 0; r < 4; r++) s[r] = (uint32_t)(z + r) > span ? -INFINITY : s[r];
}

// RB: 16-row blocks per wave (2: 256 rows per workgroup; 1: 128, the form for head dims 193-256, where 32 rows of output
// and Q per wave do not fit the 256 registers of two waves per SIMD: there each fragment read from LDS feeds one matrix
// instruction instead of two, and the kernel is bound by its fragment reads; also for launches of few or short row
// blocks at head dims 129-192, see launch_prefill_pp_wide).
template <typename T, int D, int BN, int DV = D, int RB = 2>
__global__ void __launch_bounds__(512, 2) prefill_pp16_kernel(const KParams kp) {
    typedef PPCfg<T, D, BN> C;
    static_assert(DV % 32 == 0 && DV <= D, "computed head dims");
    static_assert(RB == 1 || RB == 2, "row blocks per wave");
    constexpr int WR = 16 * RB;          // query rows of a wave
    constexpr int BM = C::kWaves * WR;   // query rows of a workgroup
    constexpr int KC = DV / 32;          // k-steps of S (32 head dims each)
    constexpr int DB = DV / 16;          // 16-column blocks of O
    constexpr int KB = BN / 16;          // 16-key blocks of a tile
    constexpr int T32 = BN / 32;         // 32-key steps of the second product
    typedef typename Elem<T>::v8 v8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const fa_fwd_params& p = kp.p;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int m16 = lane & 15, g4 = lane >> 4;
    const int group = __builtin_amdgcn_readfirstlane(wave >> 2);

    // work item of this block (32-bit arithmetic: the launcher bounds the grid by 2^31)
    const uint32_t G = (uint32_t)(p.h / p.h_k);
    int g, mb, hk, b;
    if (!xcd_work_item(kp, (uint32_t)kp.num_m_blocks, (kp.has_left || kp.has_right) ? 32u : 0u, g, mb, hk, b)) return;
    const int head = hk * (int)G + g;

    const SeqInfo si = seq_info(p, b);
    // Row blocks are aligned to the END of the sequence: the partial block of a length that is no multiple of BM is
    // the first one, which under a causal mask sees the fewest keys (aligned to the start, the half-empty block is the
    // one that visits the most tiles).  Measured: 64 packed sequences of 2176 tokens -2.4 %, lengths drawn from
    // 128-4096 +-0.3 %.  m0 < 0 in that first block.
    const int nmb_seq = (si.sq + BM - 1) / BM;
    if (mb >= nmb_seq) return;
    const int m0 = si.sq - (nmb_seq - mb) * BM;

    const int shift = si.sk - si.sq;
    const int wl = p.window_left, wr = p.window_right;
    const bool has_left = kp.has_left, has_right = kp.has_right;
    int n_hi = si.sk;
    if (has_right) n_hi = min(n_hi, min(m0 + BM, si.sq) + shift + wr);
    int n_lo = 0;
    if (has_left) n_lo = max(0, max(m0, 0) + shift - wl);
    const int t_lo = n_lo / BN;
    const int t_hi = n_hi > 0 ? (n_hi + BN - 1) / BN : 0;
    const int nt = max(0, t_hi - t_lo);           // tiles visited, the same for all 8 waves

    const T* __restrict__ qg = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)head * p.q_head_stride;
    const T* __restrict__ kg = reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)hk * p.k_head_stride;
    const T* __restrict__ vg = reinterpret_cast<const T*>(p.v) + si.v_off + (int64_t)hk * p.v_head_stride;

    const int r0 = m0 + wave * WR;                // first query row of this wave

    // visit i of the key loop handles key tile tile_of(i) and uses ring slot i % NS
    // (from the last tile down: the masked tiles of a causal row block come first)
    auto tile_of = [&](int i) { return t_hi - 1 - i; };

    // ---- asynchronous tile fills, as in prefill_pp_kernel; V tiles take the swizzle of the 16x16x32 read pattern
    const int frow = (wave * 64 + lane) / C::CPR;              // tile row of pass 0
    const int fch = lane % C::CPR;
    const int kch = min(swz_k<D>(fch, frow), p.d / 8 - 1);     // clamped: columns >= d are never used
    const int vch = min(swz_vd<D>(fch, frow), p.d / 8 - 1);
    const uint32_t lds0 = (uint32_t)(size_t)((FA_LDS_PTR(char))smem);
    const uint32_t fill_base = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(wave * 1024));
    const int64_t kstep = (int64_t)BN * p.k_row_stride, vstep = (int64_t)BN * p.v_row_stride;
    const int64_t kpass = (int64_t)C::ROWS_PER_PASS * p.k_row_stride, vpass = (int64_t)C::ROWS_PER_PASS * p.v_row_stride;
    const int t_first = t_hi - 1;
    const T* ktile = scalar_ptr(kg + (int64_t)t_first * BN * p.k_row_stride);       // tile next to be requested
    const T* vtile = scalar_ptr(vg + (int64_t)t_first * BN * p.v_row_stride);
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

    // The first tiles are requested before anything else is set up.
    if (nt > 0) {
        fill_k(0);
        fill_v(0);
        if (nt > 1) { fill_k(1); fill_v(1); }
        if (nt > 2) fill_k(2);
    }

    // ---- resident Q fragments (B operand of the first product): row 16 rb + m16, head dims 32 c + 8 g4 .. + 7
    v8 qf[RB][KC];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int row = r0 + 16 * rb + m16;
        const bool valid = row >= 0 && row < si.sq;
        const T* qrow = qg + (int64_t)row * p.q_row_stride;
#pragma unroll
        for (int c = 0; c < KC; c++) {
            const int d0 = c * 32 + 8 * g4;
            u32x4 raw = {0, 0, 0, 0};
            if (valid && d0 < p.d) raw = ld_global16(qrow + d0);
            qf[rb][c] = __builtin_bit_cast(v8, raw);
        }
    }

    f32x4 o_acc[RB][DB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int db = 0; db < DB; db++) o_acc[rb][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run[RB], l_run[RB];     // l_run: this lane's share of the row sum
#pragma unroll
    for (int rb = 0; rb < RB; rb++) { m_run[rb] = -INFINITY; l_run[rb] = 0.f; }
    const float sl2 = kp.scale_log2;

    // Per-wave tile classes, as ranges of the absolute key-tile index t: the wave has visible keys
    // in tiles [ta_lo, ta_hi]; tiles in [tf_lo, tf_hi] are fully visible to all its rows (no masking).
    int ta_lo = t_lo, ta_hi = t_hi - 1, tf_lo = 0, tf_hi = si.sk / BN - 1;
    if (has_right) {
        const int c = r0 + shift + wr;            // last visible key of the wave's first row
        ta_hi = min(ta_hi, (c + WR - 1 >= 0) ? (c + WR - 1) / BN : -1);
        tf_hi = min(tf_hi, (c + 1 >= BN) ? (c + 1) / BN - 1 : -1);
    }
    if (has_left) {
        const int c = r0 + shift - wl;            // first visible key of the wave's first row
        ta_lo = max(ta_lo, (c > 0) ? c / BN : 0);
        tf_lo = (c + WR - 1 > 0) ? (c + WR - 1 + BN - 1) / BN : 0;
    }
    if (r0 >= si.sq || r0 + WR <= 0) ta_hi = ta_lo - 1;
    auto active = [&](int i) -> bool { const int t = tile_of(i); return t >= ta_lo && t <= ta_hi; };

    // ---- S^T = K Q^T.  Fragment reads run LA fragments (2 LA matrix instructions) ahead of their use.
    // (the swizzles leave bit 4 of the chunk index alone: 16 chunks = 256 bytes further along a row is a compile-time
    // offset, so the per-lane tables hold the first 4 k-steps and 8 output blocks)
    constexpr int KCT = KC < 4 ? KC : 4, DBT = DB < 8 ? DB : 8;
    int kofs[KCT];
#pragma unroll
    for (int c = 0; c < KCT; c++) kofs[c] = m16 * C::ROWB + swz_k<D>(c * 4 + g4, m16) * 16;
    f32x4 s_acc[RB][KB];
    auto qk = [&](int i, auto slot_c) __attribute__((always_inline)) {
        // the ring slot of visit i is a compile-time constant (the key loop is unrolled by the ring depth), so slot and
        // fragment offsets go into the offset field of the LDS reads instead of a vector add per fragment pointer
        constexpr int slot = decltype(slot_c)::value * C::TILE;
        const char* kb[KC];
#pragma unroll
        for (int c = 0; c < KC; c++) kb[c] = smem + (slot + (c / KCT) * 256 + kofs[c % KCT]);
        constexpr int NF = KC * KB;              // fragments in (c, kb) order: 2 KB matrix instructions between two
        constexpr int LA = FA_PP_LA;             // on the same accumulator
        auto frag_ptr = [&](int f) { return kb[f / KB] + (f % KB) * 16 * C::ROWB; };
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        u32x4 fr[LA];
#pragma unroll
        for (int e = 0; e < LA; e++) fr[e] = *reinterpret_cast<const u32x4*>(frag_ptr(e));
#pragma unroll
        for (int f = 0; f < NF; f++) {
            const int c = f / KB, kbk = f % KB;
            const v8 a = __builtin_bit_cast(v8, fr[f % LA]);
#pragma unroll
            for (int rb = 0; rb < RB; rb++) s_acc[rb][kbk] = Elem<T>::mfma16(a, qf[rb][c], c == 0 ? zero : s_acc[rb][kbk]);
            if (f + LA < NF) fr[f % LA] = *reinterpret_cast<const u32x4*>(frag_ptr(f + LA));
        }
        __builtin_amdgcn_sched_group_barrier(0x100, LA, 0);      // look-ahead reads
#pragma unroll
        for (int f = 0; f < NF; f++) {
            __builtin_amdgcn_sched_group_barrier(0x008, RB, 0);  // RB MFMAs
            if (f + LA < NF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 DS read
        }
    };

    // ---- O^T += V^T P^T, same interleave with two transposing reads per fragment
    const int tj = m16 >> 2, tq = m16 & 3;
    int vofs[DBT];
#pragma unroll
    for (int db = 0; db < DBT; db++)
        vofs[db] = C::NS * C::TILE + (4 * g4 + tj) * C::ROWB + swz_vd<D>(db * 2 + (tq >> 1), 4 * g4 + tj) * 16 + (tq & 1) * 8;
    v8 pf[RB][T32];
    auto pv = [&](int i, auto slot_c) __attribute__((always_inline)) {
        // (vofs already points into the V ring, so that slot and fragment offsets fit the 16-bit offset field)
        constexpr int slot = decltype(slot_c)::value * C::TILE;
        const char* vb[DB];
#pragma unroll
        for (int db = 0; db < DB; db++) vb[db] = smem + (slot + (db / DBT) * 256 + vofs[db % DBT]);
        constexpr int NF = T32 * DB;             // fragments in (t32, db) order
        constexpr int LA = FA_PP_LA;
        auto fetch = [&](int f) {
            const int t32 = f / DB, db = f % DB;
            const u32x2 lo = lds_read_tr16(vb[db] + t32 * 32 * C::ROWB);
            const u32x2 hi = lds_read_tr16(vb[db] + (t32 * 32 + 16) * C::ROWB);
            return (u32x4){lo[0], lo[1], hi[0], hi[1]};
        };
        u32x4 fr[LA];
#pragma unroll
        for (int e = 0; e < LA; e++) fr[e] = fetch(e);
#pragma unroll
        for (int f = 0; f < NF; f++) {
            const int t32 = f / DB, db = f % DB;
            const v8 a = __builtin_bit_cast(v8, fr[f % LA]);
#pragma unroll
            for (int rb = 0; rb < RB; rb++) o_acc[rb][db] = Elem<T>::mfma16(a, pf[rb][t32], o_acc[rb][db]);
            if (f + LA < NF) fr[f % LA] = fetch(f + LA);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * LA, 0);  // look-ahead reads
#pragma unroll
        for (int f = 0; f < NF; f++) {
            __builtin_amdgcn_sched_group_barrier(0x008, RB, 0);  // RB MFMAs
            if (f + LA < NF) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // 2 DS reads
        }
    };

    auto softmax = [&](int i) __attribute__((always_inline)) {
        const int tt = tile_of(i);
        if (tt < tf_lo || tt > tf_hi) {
            const int n0 = tt * BN;
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                const int row = r0 + 16 * rb + m16;
                int lim_hi = si.sk - 1;
                if (has_right) lim_hi = min(lim_hi, row + shift + wr);
                const int lim_lo = has_left ? row + shift - wl : 0;
#pragma unroll
                for (int kbk = 0; kbk < KB; kbk++) mask_acc4(s_acc[rb][kbk], n0 + kbk * 16 + 4 * g4, lim_lo, lim_hi);
            }
        }
        // The tile is exponentiated against the reference maxima its two rows already have and only the lane's
        // shares of the two row sums are looked at afterwards: at most 2^14 each means no probability above 2^14
        // (safe in fp16 / bf16 and in the fp32 sums), so the references stay and no maximum is formed.  A larger or
        // non-finite share anywhere in the wave (always the case while a row has no reference) takes the rare
        // branch, which forms the exact row maxima from the untouched scores (over the row's 4 lanes), moves the
        // references under the usual rule and exponentiates again.
        auto exp_tile = [&](int rb, float msc) -> float {
            float suma = 0.f, sumb = 0.f;
#pragma unroll
            for (int t32 = 0; t32 < T32; t32++) {
                u32x4 pk;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const f32x4& s = s_acc[rb][2 * t32 + h];
                    const float e0 = fast_exp2(s[0] * sl2 - msc), e1 = fast_exp2(s[1] * sl2 - msc);
                    const float e2 = fast_exp2(s[2] * sl2 - msc), e3 = fast_exp2(s[3] * sl2 - msc);
                    suma += e0 + e2;
                    sumb += e1 + e3;
                    pk[2 * h] = pack2<T>(e0, e1);
                    pk[2 * h + 1] = pack2<T>(e2, e3);
                }
                pf[rb][t32] = __builtin_bit_cast(v8, pk);
            }
            return suma + sumb;
        };
        float tsum[RB], corr[RB];
        bool redo = false;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            tsum[rb] = exp_tile(rb, m_run[rb] * sl2);
            corr[rb] = 1.f;
            redo = redo || !(tsum[rb] <= 16384.f);
        }
        if (__builtin_amdgcn_ballot_w64(redo) != 0) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                float mx = -INFINITY;
#pragma unroll
                for (int kbk = 0; kbk < KB; kbk++)
#pragma unroll
                    for (int r = 0; r < 4; r++) mx = fmaxf(mx, s_acc[rb][kbk][r]);
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                // lazy reference max: move it only when the tile max exceeds it by more than 2^8 (exp2 domain)
                const bool move = (mx - m_run[rb]) * sl2 > 8.f;       // false for NaN (-inf - -inf)
                const float m_new = move ? mx : m_run[rb];
                corr[rb] = move ? fast_exp2((m_run[rb] - m_new) * sl2) : 1.f;   // m_run = -inf -> 0
                l_run[rb] *= corr[rb];
                m_run[rb] = m_new;
                tsum[rb] = exp_tile(rb, (m_new == -INFINITY) ? 0.f : m_new * sl2);
            }
        }
        bool moved = false;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            l_run[rb] += tsum[rb];
            moved = moved || corr[rb] != 1.f;
        }
        // (tested on the factors themselves, not on a flag set in the branch above: with a flag the compiler
        // merges this block into that branch and copies all of o_acc around it on every tile)
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int rb = 0; rb < RB; rb++) o_acc[rb][db] *= corr[rb];
        }
    };

    if (nt > 0) {
        // ---- prologue: K(0), V(0), K(1), V(1), K(2) were requested above; S = K(0) Q
        wait_vmcnt<0>();
        __syncthreads();
        if (active(0)) qk(0, std::integral_constant<int, 0>());
        if (group == 1) __syncthreads();   // group 1 runs one phase behind group 0

        // visit i of the key loop with its ring slots as compile-time constants: i % NS == SL (measured +0.5-1 %)
        auto visit = [&](int i, auto sl) __attribute__((always_inline)) {
            constexpr int SL = decltype(sl)::value;
            // ---- Y(i): VALU phase (and requests for the tiles needed 3 iterations ahead)
            if (i + C::PF < nt) fill_k(i + C::PF);
            if (i + C::PF - 1 < nt) fill_v(i + C::PF - 1);
            const bool act = active(i);
            if (act) softmax(i);
            __syncthreads();
            // ---- X(i): MFMA phase
            __builtin_amdgcn_s_setprio(1);
            if (act) pv(i, std::integral_constant<int, SL>());
            if (i + 1 < nt && active(i + 1)) qk(i + 1, std::integral_constant<int, (SL + 1) % C::NS>());
            __builtin_amdgcn_s_setprio(0);
            // this wave's fills of K(i+2), V(i+1) must have landed before the barrier publishes them;
            // the 2 * LOADS requests of Y(i) may stay in flight
            if (i + C::PF < nt) wait_vmcnt<2 * C::LOADS>(); else wait_vmcnt<0>();
            __syncthreads();
        };
        static_assert(C::NS == 4, "the loop is unrolled by the ring depth");
        int i = 0;
        for (; i + 4 <= nt; i += 4) {
            visit(i, std::integral_constant<int, 0>());
            visit(i + 1, std::integral_constant<int, 1>());
            visit(i + 2, std::integral_constant<int, 2>());
            visit(i + 3, std::integral_constant<int, 3>());
        }
        if (i < nt) { visit(i, std::integral_constant<int, 0>()); i++; }
        if (i < nt) { visit(i, std::integral_constant<int, 1>()); i++; }
        if (i < nt) { visit(i, std::integral_constant<int, 2>()); i++; }
        if (group == 0) __syncthreads();
    }

    // ---- epilogue: the row sums of the 4 lanes that share a row, normalisation, log-sum-exp
    float inv[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        float l_tot = l_run[rb];
        l_tot += __shfl_xor(l_tot, 16);
        l_tot += __shfl_xor(l_tot, 32);
        const bool dead = (l_tot == 0.f) || (l_tot != l_tot);
        inv[rb] = dead ? 1.f : 1.f / l_tot;
        const float lse = dead ? INFINITY : m_run[rb] * p.softmax_scale + __logf(l_tot);
        const int row = r0 + 16 * rb + m16;
        if (g4 == 0 && row >= 0 && row < si.sq) p.softmax_lse[((int64_t)b * p.h + head) * p.seqlen_q + row] = lse;
    }
    // The output tile of the wave (its rows x D) goes through LDS so that every store instruction writes whole
    // rows (16 B per lane).  All tile reads of the ring are behind the last barrier and each wave uses its own
    // region, so no barrier is needed.
    {
        constexpr int PITCH = DV * 2 + 16;             // the computed head dims of a row (reads past them are not stored)
        // all of the wave's rows at once where 8 such regions fit the ring, else one 16-row block after the other
        constexpr int SRB = C::kWaves * WR * PITCH <= C::SMEM ? RB : 1;      // row blocks per pass
        static_assert(C::kWaves * 16 * SRB * PITCH <= C::SMEM, "the staged output fits the ring");
        char* stage = smem + wave * (16 * SRB * PITCH);
        constexpr int RPP = 64 / C::CPR;                // rows per store instruction
        const int srow = lane / C::CPR, sch = lane % C::CPR;
        T* obase = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)head * p.o_head_stride + sch * 8;
#pragma unroll
        for (int pass = 0; pass < RB / SRB; pass++) {
#pragma unroll
            for (int sb = 0; sb < SRB; sb++) {
                const int rb = pass * SRB + sb;
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    const int d0 = db * 16 + 4 * g4;
                    const f32x4& o = o_acc[rb][db];
                    const u32x2 v = {pack2<T>(o[0] * inv[rb], o[1] * inv[rb]), pack2<T>(o[2] * inv[rb], o[3] * inv[rb])};
                    *reinterpret_cast<u32x2*>(stage + (16 * sb + m16) * PITCH + d0 * 2) = v;
                }
            }
#pragma unroll
            for (int j = 0; j < 16 * SRB / RPP; j++) {
                const int rr = j * RPP + srow, row = r0 + pass * 16 * SRB + rr;
                const u32x4 v = *reinterpret_cast<const u32x4*>(stage + rr * PITCH + sch * 16);
                if (row >= 0 && row < si.sq && sch * 8 < p.d) st_global16(obase + (int64_t)row * p.o_row_stride, v);
            }
        }
    }
}

template <typename T, int D, int BN, int DV = D, int RB = 2>
int launch_prefill_pp16_one(KParams kp, hipStream_t stream) {
    typedef PPCfg<T, D, BN> C;
    constexpr int BM = C::kWaves * 16 * RB;
    kp.num_m_blocks = (kp.p.seqlen_q + BM - 1) / BM;
    const int64_t total = (int64_t)kp.num_m_blocks * kp.p.h * kp.p.b;
    if (total <= 0) return 0;
    const int64_t nblocks = xcd_grid(kp.p, kp.num_m_blocks);
    if (nblocks == 0) return -2;
    dim3 grid((unsigned)nblocks), block(C::kThreads);
    if (int e = prepare_work_list(kp, BM, nblocks, stream)) return e;
    auto kern = prefill_pp16_kernel<T, D, BN, DV, RB>;
    hipError_t e = FA_ALLOW_DYNAMIC_LDS(kern, C::SMEM);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, grid, block, C::SMEM, stream, kp);
    return note_kernel((int)hipGetLastError(), D > 128 ? (RB == 2 ? FA_KERNEL_PINGPONG_WIDE32 : FA_KERNEL_PINGPONG_WIDE) : FA_KERNEL_PINGPONG, false, false, DV);
}

// Without dropout the 16x16x32 form; with dropout the 32x32x16 kernel of fa_prefill_pp.h, whose mask arithmetic
// is laid out for that instruction's one row per lane.
template <typename T, int D, int BN>
int launch_prefill_pp(const KParams& kp, hipStream_t stream) {
    if (kp.p.p_dropout > 0.f) return launch_prefill_pp_one<T, D, BN, true>(kp, stream);
    if constexpr (D == 128) {
        if (kp.p.d <= 96) return launch_prefill_pp16_one<T, D, BN, 96>(kp, stream);
    }
    return launch_prefill_pp16_one<T, D, BN>(kp, stream);
}

// Head dims 129..256 without dropout: 32-key tiles in the same four-slot rings, 16 query rows per wave (one row
// block: 64 accumulator registers of output and 32 of Q at head dim 256; 128 rows per workgroup) or 32 (up to head
// dim 192; 256 rows per workgroup); the reference's buckets 160, 192, 224, 256
// (csrc/flash_attn/src/flash_fwd_launch_template.h:236-336) leave out the k-steps and column blocks past the bucket.
template <typename T>
int launch_prefill_pp_wide(const KParams& kp, hipStream_t stream) {
    // Up to head dim 192 a wave's registers hold 32 query rows (two row blocks: 96 registers of output, 48 of Q), and
    // every K / V fragment read from LDS then feeds two matrix instructions: bf16 causal 8k at d 192 874 -> 1162
    // TFLOP/s, full 914 -> 1304, d 160 789 -> 1097, 64 packed sequences of 128-4096 tokens 3.32 -> 2.55 ms.  At 224
    // and 256 the same form spills 15 and 78 registers (+2 % and half the speed): those keep 16 rows per wave.
    // The 128-row blocks stay where 256-row blocks would leave CUs idle: sequences of up to 128 queries (-4 %
    // otherwise), launches of up to 128 blocks (64-128 blocks: 128-row blocks 27-38 % faster), and up to 256 under a
    // mask when a sequence has several blocks of unequal length (one heavy block per CU: 10-18 % faster; with one
    // block per sequence, 129-256 queries against 4096 keys, the 256-row form is 23-30 % ahead at 256 blocks).
    const bool masked = kp.has_right || kp.has_left;
    const int64_t wgs256 = (int64_t)((kp.p.seqlen_q + 255) / 256) * kp.p.h * kp.p.b;
    const bool rows32 = kp.p.d <= 192 && kp.p.seqlen_q > 128 && wgs256 > (masked && kp.p.seqlen_q > 256 ? 256 : 128);
    if (kp.p.d <= 160) return rows32 ? launch_prefill_pp16_one<T, 256, 32, 160, 2>(kp, stream) : launch_prefill_pp16_one<T, 256, 32, 160, 1>(kp, stream);
    if (kp.p.d <= 192) return rows32 ? launch_prefill_pp16_one<T, 256, 32, 192, 2>(kp, stream) : launch_prefill_pp16_one<T, 256, 32, 192, 1>(kp, stream);
    if (kp.p.d <= 224) return launch_prefill_pp16_one<T, 256, 32, 224, 1>(kp, stream);
    return launch_prefill_pp16_one<T, 256, 32, 256, 1>(kp, stream);
}

}  // namespace fa
