// Split-KV decode kernel for gfx950: few query rows against a long K/V stream (HBM-bound).
// Counterpart of the reference's compute_attn_1rowblock_splitkv used for seqlen_q == 1 after its
// "seqlen_q <-> ngroups" swap (csrc/flash_attn/flash_api.cpp:1096-1104,
// csrc/flash_attn/src/flash_fwd_kernel.h:584-1130), designed as a streaming kernel:
//
//  * One workgroup = one (batch, kv-head, key-chunk).  All query rows that share the kv head --
//    seqlen_q positions x (h / h_k) grouped heads, at most 16 -- are packed into the 16 columns of
//    v_mfma_f32_16x16x32, so every K/V byte is fetched once per group.
//  * The four waves of the workgroup stream disjoint quarters of the chunk on their own: 128-bit
//    row-contiguous global loads (a 16-lane group reads one whole K or V row), issued one 32-key
//    step ahead into registers, staged through a wave-private swizzled LDS tile to reach the MFMA
//    operand layouts (ds_read_b128 for K, transposing ds_read_b64_tr_b16 for V).  No workgroup
//    barrier in the loop.
//  * The four running (max, sum, O) states are merged through LDS at the end and written either as
//    the final output or as one fp32 partial + log-sum-exp per chunk for the combine kernel.
#include "fa_common.h"
#include "fa_launch.h"

namespace fa {

template <typename T, int D>
struct DecodeCfg {
    static constexpr int kThreads = 256, kWaves = 4;
    static constexpr int STEP = 32;                 // keys per wave step
    static constexpr int CPR = D / 8;
    static constexpr int ROWB = D * 2;
    static constexpr int TILE_BYTES = STEP * ROWB;  // one of K / V for one wave
    static constexpr int LD = STEP * CPR / 64;      // 16 B loads per lane per tensor per step
    static constexpr int KC = D / 32;               // k-steps of S^T
    static constexpr int DB = D / 16;               // 16-row blocks of O^T
    static constexpr int STAGE_BYTES = kWaves * 2 * TILE_BYTES;
    static constexpr int MERGE_BYTES = kWaves * 16 * (D + 2) * 4;
    static constexpr int SMEM = STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES;
};

// One (batch, kv head, key range) item: attention of the packed query rows over the range, written
// as the final output (SPLIT = false) or as partial `slot` (SPLIT = true).
// APPEND: rows [cache length, cache length + seqlen_knew) are not in the cache yet; the item whose key range
// holds them writes them first.  Every key belongs to exactly one item, so each row has one writer.
// STREAM: K and V rows are fetched with non-temporal loads.  Every row is read once, so nothing is gained by
// keeping it in the caches, and past the size the memory-side cache holds the hint is worth 8-11 % (4.5 GB of
// K/V: 0.747 -> 0.824 of 8 TB/s); caches of a few hundred MB that are read again step after step are up to 7 %
// faster without it.  (A template parameter and not a run-time branch: the compiler merges the loads of the
// two branches and drops the hint.)
template <typename T, int D, bool SPLIT, bool APPEND = false, bool STREAM = false>
FA_DEV void decode_item(const KParams& kp, char* smem, const int hk, const int b, const int slot,
                        const int mode, const int idx) {
    typedef DecodeCfg<T, D> C;
    typedef typename Elem<T>::v8 v8;
    const fa_fwd_params& p = kp.p;
    const int split = slot;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int m = lane & 15, g4 = lane >> 4;     // MFMA column (packed query row), lane group
    const int G = p.h / p.h_k;
    const int rows = p.seqlen_q * G;             // packed rows in use (<= 16)

    const SeqInfo si = seq_info(p, b);
    const int shift = si.sk - si.sq;
    const int wl = p.window_left, wr = p.window_right;
    const bool has_left = kp.has_left, has_right = kp.has_right;

    int hi = si.sk, lo = 0;
    if (has_right) hi = min(hi, si.sq + shift + wr);
    if (has_left) lo = max(0, shift - wl);
    if (SPLIT) {
        int c_lo, c_hi;
        item_key_range(kp, mode, idx, hi, c_lo, c_hi);
        lo = max(lo, c_lo);
        hi = min(hi, c_hi);
    }

    // packed row m -> query position and head
    const int qi = m / G, qg = m % G;
    const int head = hk * G + qg;
    const bool row_valid = m < rows;

    if (hi <= lo) {   // nothing visible in this chunk
        if (tid < rows) {
            const int i = tid / G, hd = hk * G + tid % G;
            if (SPLIT) {
                p.lse_accum[(((int64_t)split * p.b + b) * p.h + hd) * p.seqlen_q + i] = -INFINITY;
            } else {
                p.softmax_lse[((int64_t)b * p.h + hd) * p.seqlen_q + i] = INFINITY;
                T* orow = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)i * p.o_row_stride + (int64_t)hd * p.o_head_stride;
                for (int d0 = 0; d0 < p.d; d0 += 8) { u32x4 z = {0, 0, 0, 0}; st_global16(orow + d0, z); }
            }
        }
        return;
    }

    // ---- this wave's key range
    const int span = hi - lo;
    const int per_wave = ((span + C::kWaves - 1) / C::kWaves + C::STEP - 1) / C::STEP * C::STEP;
    const int w_lo = lo + wave * per_wave;
    const int w_hi = min(hi, w_lo + per_wave);

    const T* __restrict__ kg = reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)hk * p.k_head_stride;
    const T* __restrict__ vg = reinterpret_cast<const T*>(p.v) + si.v_off + (int64_t)hk * p.v_head_stride;
    char* kb = smem + wave * 2 * C::TILE_BYTES;
    char* vb = kb + C::TILE_BYTES;

    u32x4 kr[C::LD], vr[C::LD];
    // unconditional loads (clamped into range), zeroed on the way into LDS
    const int d_last_chunk = p.d / 8 - 1;
    auto load_step = [&](int n0) {
#pragma unroll
        for (int i = 0; i < C::LD; i++) {
            const int f = lane + i * 64;
            const int row = f / C::CPR, c = min(f % C::CPR, d_last_chunk);
            const int n = min(n0 + row, w_hi - 1);
            const T* kp_ = kg + (int64_t)n * p.k_row_stride + c * 8;
            const T* vp_ = vg + (int64_t)n * p.v_row_stride + c * 8;
            if constexpr (STREAM) {
                kr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp_));
                vr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vp_));
            } else {
                kr[i] = ld_global16(kp_);
                vr[i] = ld_global16(vp_);
            }
        }
    };
    auto store_step = [&](int n0) {
#pragma unroll
        for (int i = 0; i < C::LD; i++) {
            const int f = lane + i * 64;
            const int row = f / C::CPR, c = f % C::CPR;
            const bool ok = (n0 + row < w_hi) && (c <= d_last_chunk);
            const u32x4 z = {0, 0, 0, 0};
            *reinterpret_cast<u32x4*>(kb + row * C::ROWB + swz_k<D>(c, row) * 16) = ok ? kr[i] : z;
            *reinterpret_cast<u32x4*>(vb + row * C::ROWB + swz_vd<D>(c, row) * 16) = ok ? vr[i] : z;
        }
    };

    f32x4 o_acc[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++) o_acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;   // l_run: this lane's share of the row sum
    const float sl2 = kp.scale_log2;

    int lim_hi = si.sk - 1;
    if (has_right) lim_hi = min(lim_hi, qi + shift + wr);
    const int lim_lo = has_left ? qi + shift - wl : 0;
    const int tj = (lane & 15) >> 2, tq = lane & 3;

    if constexpr (APPEND) {
        // rows [cache length, cache length + seqlen_knew) that fall into this item's key range are not in the
        // cache yet: the workgroup writes them (new keys rotated, values copied, exactly as append_kv_kernel)
        // and waits until the stores have been performed before any wave loads its keys
        const int a_lo = max(lo, si.sk_cache);
        if (a_lo < hi) {
            const int cpr = p.d / 8;
            T* kdst = reinterpret_cast<T*>(const_cast<void*>(p.k)) + si.k_off + (int64_t)hk * p.k_head_stride;
            T* vdst = reinterpret_cast<T*>(const_cast<void*>(p.v)) + si.v_off + (int64_t)hk * p.v_head_stride;
            for (int e = tid; e < (hi - a_lo) * cpr; e += C::kThreads) {
                const int n = a_lo + e / cpr, d0 = (e % cpr) * 8, t = n - si.sk_cache;
                const T* vsrc = reinterpret_cast<const T*>(p.v_new) + (int64_t)b * p.vnew_batch_stride + (int64_t)t * p.vnew_row_stride + (int64_t)hk * p.vnew_head_stride;
                const T* ksrc = reinterpret_cast<const T*>(p.k_new) + (int64_t)b * p.knew_batch_stride + (int64_t)t * p.knew_row_stride + (int64_t)hk * p.knew_head_stride;
                st_global16(vdst + (int64_t)n * p.v_row_stride + d0, ld_global16(vsrc + d0));
                u32x4 raw = ld_global16(ksrc + d0);
                if (p.rotary_dim > 0 && d0 < p.rotary_dim) {
                    const T* cr = reinterpret_cast<const T*>(p.rotary_cos) + (int64_t)n * (p.rotary_dim / 2);
                    const T* sr = reinterpret_cast<const T*>(p.rotary_sin) + (int64_t)n * (p.rotary_dim / 2);
                    float x[8];
                    unpack8<T>(raw, x);
                    rotary8<T>(x, ksrc, cr, sr, d0, p.rotary_dim, p.is_rotary_interleaved != 0);
                    raw = pack8<T>(x);
                }
                st_global16(kdst + (int64_t)n * p.k_row_stride + d0, raw);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
        }
    }

    // the first K/V step is requested before anything else so that its latency overlaps the q
    // (and rotary table) fetches below
    if (w_lo < w_hi) load_step(w_lo);

    // ---- Q fragments (B operand): lane (m, g4) holds Q[row m][32c + 8*g4 .. +7]
    v8 qf[C::KC];
    {
        const T* qrow = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)qi * p.q_row_stride + (int64_t)head * p.q_head_stride;
#pragma unroll
        for (int c = 0; c < C::KC; c++) {
            const int d0 = c * 32 + 8 * g4;
            u32x4 raw = {0, 0, 0, 0};
            if (row_valid && d0 < p.d) {
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
            qf[c] = __builtin_bit_cast(v8, raw);
        }
    }

    for (int n0 = w_lo; n0 < w_hi; n0 += C::STEP) {
        // the previous step's LDS reads are complete (their results were consumed) before these
        // writes are issued; LDS operations of one wave execute in order.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        store_step(n0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (n0 + C::STEP < w_hi) load_step(n0 + C::STEP);

        // ---- S^T (2 blocks of 16 keys) = K Q^T
        f32x4 s_acc[2];
#pragma unroll
        for (int kbk = 0; kbk < 2; kbk++) {
            s_acc[kbk] = (f32x4){0.f, 0.f, 0.f, 0.f};
            const int krow = kbk * 16 + m;
#pragma unroll
            for (int c = 0; c < C::KC; c++) {
                const int ch = c * 4 + g4;
                const u32x4 raw = *reinterpret_cast<const u32x4*>(kb + krow * C::ROWB + swz_k<D>(ch, krow) * 16);
                s_acc[kbk] = Elem<T>::mfma16(__builtin_bit_cast(v8, raw), qf[c], s_acc[kbk]);
            }
        }
        // ---- mask + online softmax; lane (m, g4) holds keys n0 + 16*kbk + 4*g4 + r of row m
        float mx = -INFINITY;
#pragma unroll
        for (int kbk = 0; kbk < 2; kbk++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int n = n0 + kbk * 16 + 4 * g4 + r;
                if (n > lim_hi || n < lim_lo || n >= w_hi) s_acc[kbk][r] = -INFINITY;
                mx = fmaxf(mx, s_acc[kbk][r]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = fast_exp2((m_run - m_use) * sl2);
        const float msc = m_use * sl2;
        float sum = 0.f;
        float pv[8];
#pragma unroll
        for (int kbk = 0; kbk < 2; kbk++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float e = fast_exp2(s_acc[kbk][r] * sl2 - msc);
                pv[kbk * 4 + r] = e;
                sum += e;
            }
        l_run = l_run * corr + sum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < C::DB; db++) o_acc[db] *= corr;
        const v8 pf = __builtin_bit_cast(v8, pack8<T>(pv));

        // ---- O^T += V^T P^T ; A operand rows: keys {4*g4 + j, 16 + 4*g4 + j}
        const int vrow = 4 * g4 + tj;
#pragma unroll
        for (int db = 0; db < C::DB; db++) {
            const int ch = db * 2 + (tq >> 1);
            const int off = swz_vd<D>(ch, vrow) * 16 + (tq & 1) * 8;
            const u32x2 lo2 = lds_read_tr16(vb + vrow * C::ROWB + off);
            const u32x2 hi2 = lds_read_tr16(vb + (vrow + 16) * C::ROWB + off);
            u32x4 raw = {lo2[0], lo2[1], hi2[0], hi2[1]};
            o_acc[db] = Elem<T>::mfma16(__builtin_bit_cast(v8, raw), pf, o_acc[db]);
        }
    }

    // ---- merge the four waves through LDS.  Layout per wave: 16 rows x (D floats of O, m, l).
    l_run += __shfl_xor(l_run, 16);
    l_run += __shfl_xor(l_run, 32);
    __syncthreads();   // all waves are done with their staging tiles
    constexpr int RSTR = D + 2;
    float* msm = reinterpret_cast<float*>(smem);
    {
        float* mine = msm + (wave * 16 + m) * RSTR;
#pragma unroll
        for (int db = 0; db < C::DB; db++) {
            const int d0 = db * 16 + 4 * g4;
            mine[d0] = o_acc[db][0]; mine[d0 + 1] = o_acc[db][1];
            mine[d0 + 2] = o_acc[db][2]; mine[d0 + 3] = o_acc[db][3];
        }
        if (g4 == 0) { mine[D] = m_run; mine[D + 1] = l_run; }
    }
    __syncthreads();
    {
        constexpr int EPT = D / 16;              // elements per thread
        const int row = tid >> 4, dseg = (tid & 15) * EPT;
        float mw[4], lw[4], mfin = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            mw[w] = msm[(w * 16 + row) * RSTR + D];
            lw[w] = msm[(w * 16 + row) * RSTR + D + 1];
            mfin = fmaxf(mfin, mw[w]);
        }
        const float m_use = (mfin == -INFINITY) ? 0.f : mfin;
        float acc[EPT], ltot = 0.f;
#pragma unroll
        for (int e = 0; e < EPT; e++) acc[e] = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float sc = fast_exp2((mw[w] - m_use) * sl2);
            ltot += lw[w] * sc;
#pragma unroll
            for (int e = 0; e < EPT; e++) acc[e] += msm[(w * 16 + row) * RSTR + dseg + e] * sc;
        }
        const bool dead = (ltot == 0.f) || (ltot != ltot);
        const float inv = dead ? 1.f : 1.f / ltot;
        if (row < rows) {
            const int i = row / G, hd = hk * G + row % G;
            const float lse_fin = m_use * p.softmax_scale + __logf(ltot);
            if (SPLIT) {
                const int64_t ridx = (((int64_t)split * p.b + b) * p.h + hd) * p.seqlen_q + i;
                if ((tid & 15) == 0) p.lse_accum[ridx] = dead ? -INFINITY : lse_fin;
                float* orow = p.o_accum + ridx * kp.d_rounded;
#pragma unroll
                for (int e = 0; e < EPT; e += 4) {
                    if (dseg + e < kp.d_rounded) {
                        f32x4 v = {acc[e] * inv, acc[e + 1] * inv, acc[e + 2] * inv, acc[e + 3] * inv};
                        *reinterpret_cast<f32x4*>(orow + dseg + e) = v;
                    }
                }
            } else {
                if ((tid & 15) == 0) p.softmax_lse[((int64_t)b * p.h + hd) * p.seqlen_q + i] = dead ? INFINITY : lse_fin;
                T* orow = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)i * p.o_row_stride + (int64_t)hd * p.o_head_stride;
#pragma unroll
                for (int e = 0; e < EPT; e += 4) {
                    if (dseg + e < p.d) {
                        u32x2 v = {pack2<T>(acc[e] * inv, acc[e + 1] * inv), pack2<T>(acc[e + 2] * inv, acc[e + 3] * inv)};
                        st_global8(orow + dseg + e, v);
                    }
                }
            }
        }
    }
}

template <typename T, int D, bool SPLIT, bool STREAM>
__global__ void __launch_bounds__(256, (D > 128 ? 1 : 2)) decode_kernel(const KParams kp) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // kv heads vary fastest over the grid: the h_k workgroups that share the rows of one
    // (batch, chunk) of a (b, s, h_k, d) cache run together and consume whole cache rows.
    decode_item<T, D, SPLIT, false, STREAM>(kp, smem, blockIdx.x, blockIdx.z, blockIdx.y, kChunk, blockIdx.y);
}

// Persistent form: a fixed number of resident workgroups draw items from a ticket counter, in the
// same cache-row-friendly order (kv head fastest), first the kMacro pass then the kSub pass.
//  * The item whose key range reaches the new rows appends them (APPEND, see decode_item): no append launch.
//  * work_counter[0..1] is the ticket counter, work_counter[2..3] counts the workgroups that have left; the last
//    one puts both back to zero, and both are tagged with the call's epoch (epoch_counter_next, fa_common.h), so
//    no launch has to reset them, not even after a launch that never finished.
// Measured and not adopted: drawing the next ticket when an item's key loop ends, so that the counter's round
// trip runs under the merge and the output stores (+1 % on the step); drawing it early (before the item: the returning atomic sits in front
// of the item's first K/V loads in the wave's in-order memory queue, +7 % time; after the item's last load:
// no change, the second resident workgroup of the CU already covers the round trip), and merging a (batch,
// kv head)'s partials in the kernel by the last of its items to arrive (the partials must bypass the per-XCD
// L2, every stream completes in the remainder pass at the very end of the launch, and 512 latency-bound
// merges there cost 2-3 x the stand-alone merge kernel; cache write-back / invalidation fences at device scope
// around every item instead cost three times the whole kernel).
// (what for_each_ticket calls per ticket)
template <typename T, int D, bool APPEND, bool STREAM>
struct DecodeTicketItem {
    static FA_DEV void run(const KParams& kp, char* smem, int hk, int b, int slot, int mode, int idx) {
        decode_item<T, D, true, APPEND, STREAM>(kp, smem, hk, b, slot, mode, idx);
    }
};
template <typename T, int D, bool APPEND, bool STREAM>
__global__ void __launch_bounds__(256, (D > 128 ? 1 : 2)) decode_persistent_kernel(const KParams kp) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    for_each_ticket<DecodeTicketItem<T, D, APPEND, STREAM>>(kp, smem);
}

// (the kernel is a template argument, not a function argument: the once-per-device flag inside
// FA_ALLOW_DYNAMIC_LDS is then one per kernel)
template <auto KERN>
static int launch_decode_kernel(dim3 grid, int smem, const KParams& kp, hipStream_t stream) {
    const hipError_t e = FA_ALLOW_DYNAMIC_LDS(KERN, smem);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(KERN, grid, dim3(256), smem, stream, kp);
    return note_kernel((int)hipGetLastError(), kp.dec_persistent ? FA_KERNEL_DECODE_TICKETS : FA_KERNEL_DECODE, false, kp.num_splits > 1,
                       kp.p.d <= 64 ? 64 : kp.p.d <= 128 ? 128 : 256);
}

template <typename T, int D, bool STREAM>
static int launch_decode_ts(const KParams& kp, hipStream_t stream) {
    typedef DecodeCfg<T, D> C;
    static_assert(C::kThreads == 256, "launch_decode_kernel launches 256 lanes");
    if (kp.dec_persistent) {
        const int total = kp.p.b * (kp.dec_sa + kp.dec_sb) * kp.p.h_k;
        const int resident = 256 * (D > 128 ? 1 : 2);          // workgroups the 256 CUs hold at once
        const dim3 grid(total < resident ? total : resident);
        if (kp.dec_append) return launch_decode_kernel<decode_persistent_kernel<T, D, true, STREAM>>(grid, C::SMEM, kp, stream);
        return launch_decode_kernel<decode_persistent_kernel<T, D, false, STREAM>>(grid, C::SMEM, kp, stream);
    }
    const bool split = kp.num_splits > 1;
    const dim3 grid(kp.p.h_k, split ? kp.num_splits : 1, kp.p.b);
    if (split) return launch_decode_kernel<decode_kernel<T, D, true, STREAM>>(grid, C::SMEM, kp, stream);
    return launch_decode_kernel<decode_kernel<T, D, false, STREAM>>(grid, C::SMEM, kp, stream);
}

template <typename T, int D>
static int launch_decode_t(const KParams& kp, hipStream_t stream) {
    return kp.stream_kv ? launch_decode_ts<T, D, true>(kp, stream) : launch_decode_ts<T, D, false>(kp, stream);
}

int launch_decode(const KParams& kp, hipStream_t stream) {
    const int d = kp.p.d;
    const bool bf = kp.p.dtype == FA_DTYPE_BF16;
    if (d <= 64) return bf ? launch_decode_t<__bf16, 64>(kp, stream) : launch_decode_t<_Float16, 64>(kp, stream);
    if (d <= 128) return bf ? launch_decode_t<__bf16, 128>(kp, stream) : launch_decode_t<_Float16, 128>(kp, stream);
    return bf ? launch_decode_t<__bf16, 256>(kp, stream) : launch_decode_t<_Float16, 256>(kp, stream);
}

}  // namespace fa
