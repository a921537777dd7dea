// Shared device helpers for the gfx950 FlashAttention forward kernels.
//
// Everything here is written for CDNA4 wave64: MFMA 32x32x16 / 16x16x32 on 16-bit inputs,
// transposing LDS reads (ds_read_b64_tr_b16), and the cross-half lane swap (v_permlane32_swap).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include "fa_mi355x.h"

namespace fa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define FA_DEV __device__ __forceinline__

// Lets `kern` use `bytes` of dynamic LDS.  The limit is a property of the kernel on a device, so it is
// set on the first launch there and not again (each expansion of the macro has its own flags: one per
// kernel instantiation and call site).
#define FA_ALLOW_DYNAMIC_LDS(kern, bytes)                                                                  \
    ([&]() -> hipError_t {                                                                                 \
        static std::atomic<bool> done[64];                                                                 \
        int dev = 0;                                                                                       \
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)                                      \
            return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (bytes)); \
        if (done[dev].load(std::memory_order_acquire)) return hipSuccess;                                  \
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (bytes)); \
        if (e == hipSuccess) done[dev].store(true, std::memory_order_release);                             \
        return e;                                                                                          \
    }())
#define FA_LDS_PTR(T) __attribute__((address_space(3))) T*

// Kernel-side view of one problem: the caller's description plus values the host derives once.
struct KParams {
    fa_fwd_params p;
    float scale_log2;      // softmax_scale * log2(e)
    int32_t num_splits;    // resolved split count (>= 1)
    int32_t split_len;     // keys per split chunk (multiple of the key tile), when num_splits > 1
    int32_t d_rounded;     // d rounded up to 32: row pitch of o_accum
    int32_t num_m_blocks;  // query tiles per (batch, head)
    int32_t has_left, has_right;  // window bounds active (after causal normalisation)
    int32_t rotary_q;      // rotate q on load
    // persistent decode schedule (see fa_decode.hip): dec_sa slots of split_len keys, then dec_sb
    // slots of dec_sub keys for each sequence's ragged remainder; tickets from work_counter[0..1], workgroups
    // that have left counted in [2..3] (64-bit epoch counters, epoch_counter_next).
    // dec_append: the item that reaches rows [cache length, cache length + seqlen_knew) writes them
    // dec_compact: the tickets cover only the slots that hold keys (the kernel counts them per batch entry
    // from the lengths); the merge then derives which slots were written from the lengths as well
    int32_t dec_persistent, dec_sa, dec_sb, dec_sub, dec_append, dec_compact;
    // K and V together hold kStreamKvBytes or more (1.5 times what the 256 MB memory-side cache keeps): the decode
    // kernels, which read every row once, fetch them with non-temporal loads.  Measured, one query position, bf16
    // d 128, non-temporal against plain loads: 245 MB read per step -3..-6 %, 367-370 MB +10..+15 %, 414-491 MB
    // +2..+15 %, 983 MB +1 %.
    int32_t stream_kv;
    // Few query positions with grouped q heads (pack_g > 1): the rows of the tiled kernel's problem are the
    // (position, grouped head) pairs of one kv head, row = position * pack_g + head within the group; p.h is
    // then the number of kv heads, p.seqlen_q the number of such rows, p.q_head_stride / p.o_head_stride step
    // over a whole group and pack_q_hs / pack_o_hs over one q head.  Masks, rotary positions and softmax_lse
    // follow the position, row / pack_g.
    int32_t pack_g;
    int64_t pack_q_hs, pack_o_hs;
    int32_t* work_counter;
    uint32_t epoch;        // non-zero, drawn anew by the host for every call: tags the counters of this launch
    // Packed batches: work list built on the device from cu_seqlens_q just before the launch (work_list_kernel,
    // fa_aux.hip), or NULL.  8 item counts, then for XCD x a list of (gridDim.x / 8) slots of two words:
    // batch index, (q head << 16) | row block.
    const int32_t* work_items;
};
constexpr int64_t kStreamKvBytes = (int64_t)3 << 27;
constexpr int kDecCompactMaxBatch = 1024;    // batch entries whose slot counts the persistent decode kernel scans in LDS
constexpr int kWorkListHeaderWords = 8;
constexpr int kWorkListMaxBatch = 2048;      // sequences the list builder ranks (quadratic, in LDS)

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
    typedef bf16x8 v8; typedef bf16x4 v4; typedef bf16x2 v2;
    static FA_DEV f32x16 mfma32(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static FA_DEV f32x4 mfma16(v8 a, v8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Elem<_Float16> {
    typedef f16x8 v8; typedef f16x4 v4; typedef f16x2 v2;
    static FA_DEV f32x16 mfma32(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static FA_DEV f32x4 mfma16(v8 a, v8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

// round-to-nearest-even pack of two floats into one 32-bit register of T
template <typename T> FA_DEV uint32_t pack2(float a, float b) {
    typedef typename Elem<T>::v2 v2;
    f32x2 f = {a, b};
    v2 h = __builtin_convertvector(f, v2);
    return __builtin_bit_cast(uint32_t, h);
}
template <typename T> FA_DEV float to_float(T x) { return (float)x; }

template <typename T> FA_DEV void unpack8(const u32x4& raw, float* out) {
    typedef typename Elem<T>::v8 v8;
    v8 h = __builtin_bit_cast(v8, raw);
#pragma unroll
    for (int e = 0; e < 8; e++) out[e] = (float)h[e];
}
template <typename T> FA_DEV u32x4 pack8(const float* in) {
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = pack2<T>(in[2 * e], in[2 * e + 1]);
    return r;
}

FA_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max / sum over the two 32-lane halves of the wave (lane l <-> lane l^32)
FA_DEV float xhalf_max(float x) {
    uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
FA_DEV float xhalf_sum(float x) {
    uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

FA_DEV u32x4 ld_global16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
FA_DEV void st_global16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
FA_DEV void st_global8(void* p, u32x2 v) { *reinterpret_cast<u32x2*>(p) = v; }

// LDS transposing read: within each block of 16 lanes, lane 4*j+q supplies the address of four
// consecutive 16-bit elements (row j, columns 4q..4q+3 of a 4 x 16 tile); lane i of the block
// receives column i of rows 0..3.
FA_DEV u32x2 lds_read_tr16(const char* p) {
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FA_LDS_PTR(s16x4))(p));
    return __builtin_bit_cast(u32x2, v);
}

// 16-byte-chunk XOR swizzles of a row-major [rows][D] 16-bit tile in LDS.
// K tiles are read one 16 B chunk per lane by 16 consecutive rows at the same chunk index;
// V tiles are read by the transposing load as 4 consecutive rows x 4 consecutive chunks.
template <int D> FA_DEV int swz_k(int chunk, int row) {
    if constexpr (D >= 128) return chunk ^ (row & 15);
    else if constexpr (D == 64) return chunk ^ ((row >> 1) & 7);
    else return chunk ^ ((row >> 2) & 3);   // D == 32
}
template <int D> FA_DEV int swz_v(int chunk, int row) {
    if constexpr (D >= 128) return chunk ^ ((row & 3) << 2);
    else if constexpr (D == 64) return chunk ^ (((row >> 1) & 1) << 2);
    else return chunk;                       // D == 32: four rows fill the 256 B bank window
}

// V tiles read by the transposing load in the 16x16x32 geometry: a 16-lane block reads 4 consecutive rows x 2
// consecutive chunks, the wave 16 rows (8 per half-wave, which must fall into distinct 32-byte bank groups).
template <int D> FA_DEV int swz_vd(int chunk, int row) {
    if constexpr (D >= 128) return chunk ^ ((row & 7) << 1);
    else return chunk ^ (((row >> 1) & 3) << 1);   // D == 64
}

// One swizzle that serves BOTH read patterns on the same tile (the backward kernels read every
// streamed tile row-wise as one MFMA operand and transposed as another): a bijection of the rows that
// share a bank window for the row-wise read, whose upper bits separate the 4 consecutive rows of a
// transposing read.
template <int D> FA_DEV int swz_u(int chunk, int row) {
    if constexpr (D >= 128) return chunk ^ (((row & 3) << 2) | ((row >> 2) & 3));
    else if constexpr (D == 64) return chunk ^ ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
    else return chunk ^ ((row >> 2) & 3);   // D == 32
}

// ------------------------------------------------------------------------------------------------
// Dropout mask.  keep(b, h, i, j) is a pure function of (seed, offset, b, h, i, j): one 32-bit hash
// per 2 x 2 block of (row, key) supplies four random bytes, byte (i & 1) * 2 + (j & 1) belongs to
// element (i, j), and the element is kept iff its byte is below `thresh` (keep probability in 1/256
// steps, csrc/flash_attn/flash_api.cpp:104).  The 2 x 2 unit costs the same number of hashes in
// both register geometries: a lane that owns one row and 4 consecutive keys (forward, dQ kernel)
// and a lane that owns one key and 4 consecutive rows (dK / dV kernel).
// ------------------------------------------------------------------------------------------------
struct Drop {
    uint32_t k0, k1;     // per (batch, head) keys derived from seed and offset
    uint32_t thresh;     // 1..256
    float rp;            // 1 / (1 - p_dropout)
};
FA_DEV uint32_t fmix32(uint32_t h) {
    h ^= h >> 16; h *= 0x85ebca6bu; h ^= h >> 13; h *= 0xc2b2ae35u; h ^= h >> 16;
    return h;
}
FA_DEV Drop drop_init(const uint64_t* rng_state, float p_dropout, int b, int h, int nheads) {
    Drop d;
    const uint64_t seed = rng_state[0], off = rng_state[1];
    const uint32_t bh = (uint32_t)(b * nheads + h);
    d.k0 = fmix32((uint32_t)seed ^ fmix32((uint32_t)(seed >> 32) + bh * 0x9e3779b1u));
    d.k1 = fmix32(d.k0 + (uint32_t)off * 0x7f4a7c15u + fmix32((uint32_t)(off >> 32) ^ 0x2545f491u));
    const float keep = 1.f - p_dropout;
    d.thresh = (uint32_t)floorf(keep * 255.f) + 1u;
    d.rp = 1.f / keep;
    return d;
}
FA_DEV uint32_t drop_hash(const Drop& d, uint32_t i2, uint32_t j2) {
    return fmix32((i2 * 0x9e3779b1u + d.k0) ^ (j2 * 0x85ebca77u + d.k1));
}
FA_DEV bool drop_keep(const Drop& d, int i, int j) {          // one element (any kernel)
    const uint32_t w = drop_hash(d, (uint32_t)i >> 1, (uint32_t)j >> 1);
    return ((w >> (8 * ((i & 1) * 2 + (j & 1)))) & 0xffu) < d.thresh;
}
// Masks for the kernels, one 32-bit word per PAIR of accumulator registers (2 p, 2 p + 1) of a 32 x 32 block:
// 0xffff in the half of a kept element, 0 in the half of a dropped one -- the form that masks a packed 16-bit
// pair with one instruction.  Both register geometries give a lane one line of 2 x 2 blocks and its neighbour
// (lane ^ 1) the other line of the SAME blocks, so the pair shares the hashes: each lane makes four, both take
// the even lane's words for pairs 0..3 and the odd lane's for pairs 4..7 (DPP), pick their own two bytes of a
// word into the two halves (byte permute) and compare both at once: byte - thresh is negative exactly when
// the element is kept.  Must be called by all 64 lanes together; lanes l and l ^ 1 must own lines 2 m and
// 2 m + 1 (rows or keys follow the lane number from an even base) with the same block origin and hh.
typedef short s16x2 __attribute__((ext_vector_type(2)));
FA_DEV uint32_t drop_pair_mask(uint32_t w, uint32_t sel, uint32_t thresh2) {
    const uint32_t x = __builtin_amdgcn_perm(w, w, sel);
    const s16x2 t = __builtin_bit_cast(s16x2, x) - __builtin_bit_cast(s16x2, thresh2);
    return __builtin_bit_cast(uint32_t, t >> 15);
}
FA_DEV void drop_pair_masks(const uint32_t (&w)[4], uint32_t sel, uint32_t thresh2, uint32_t (&m)[8]) {
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t even = (uint32_t)__builtin_amdgcn_mov_dpp((int)w[k], 0xA0, 0xf, 0xf, true);   // quad_perm [0, 0, 2, 2]
        const uint32_t odd = (uint32_t)__builtin_amdgcn_mov_dpp((int)w[k], 0xF5, 0xf, 0xf, true);    // quad_perm [1, 1, 3, 3]
        m[k] = drop_pair_mask(even, sel, thresh2);
        m[4 + k] = drop_pair_mask(odd, sel, thresh2);
    }
}
// lane owns ROW `row`, registers walk keys kb0 + 8 (r >> 2) + 4 hh + (r & 3)   (kb0 a multiple of 32)
FA_DEV void drop_pairs_row(const Drop& d, int row, int kb0, int hh, uint32_t (&m)[8]) {
    const uint32_t odd = (uint32_t)row & 1u;
    const uint32_t j2 = (uint32_t)(kb0 + 16 * (int)odd + 4 * hh) >> 1;
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) w[k] = drop_hash(d, (uint32_t)row >> 1, j2 + 4 * (k >> 1) + (k & 1));
    // bytes 2 odd (even key) and 2 odd + 1 (odd key) of a word; selector byte 0x0c gives zero
    drop_pair_masks(w, 0x0c010c00u + odd * 0x00020002u, d.thresh * 0x00010001u, m);
}
// lane owns KEY `key`, registers walk rows rb0 + 8 (r >> 2) + 4 hh + (r & 3)   (rb0 a multiple of 32)
FA_DEV void drop_pairs_key(const Drop& d, int key, int rb0, int hh, uint32_t (&m)[8]) {
    const uint32_t odd = (uint32_t)key & 1u;
    const uint32_t i2 = (uint32_t)(rb0 + 16 * (int)odd + 4 * hh) >> 1;
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; k++) w[k] = drop_hash(d, i2 + 4 * (k >> 1) + (k & 1), (uint32_t)key >> 1);
    // bytes odd (even row) and 2 + odd (odd row) of a word
    drop_pair_masks(w, 0x0c020c00u + odd * 0x00010001u, d.thresh * 0x00010001u, m);
}

// x where half `hi` of a pair mask is set, +0 otherwise (for values that are not packed yet)
FA_DEV float drop_gate_half(float x, uint32_t pair, int hi) {
    const uint32_t w = hi ? (uint32_t)((int32_t)pair >> 16) : (uint32_t)((int32_t)(pair << 16) >> 16);
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x) & w);
}

// Rotary embedding of 8 consecutive elements [d0, d0+8) of one row, fp32 math.
// `x` are the row's own values, `row_ptr` points at the row start (to fetch the partner half for
// the non-interleaved form), cos/sin point at the table row for this token.
template <typename T>
FA_DEV void rotary8(float* x, const T* row_ptr, const T* cos_row, const T* sin_row, int d0,
                    int rotary_dim, bool interleaved) {
    if (d0 >= rotary_dim) return;
    if (interleaved) {
        float c[4], s[4];
#pragma unroll
        for (int e = 0; e < 4; e++) { c[e] = (float)cos_row[d0 / 2 + e]; s[e] = (float)sin_row[d0 / 2 + e]; }
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float x0 = x[2 * e], x1 = x[2 * e + 1];
            x[2 * e] = x0 * c[e] - x1 * s[e];
            x[2 * e + 1] = x0 * s[e] + x1 * c[e];
        }
    } else {
        const int half = rotary_dim / 2;
        const bool left = d0 < half;
        const int t0 = left ? d0 : d0 - half;           // table column
        const int partner = left ? d0 + half : d0 - half;
        u32x4 praw = ld_global16(row_ptr + partner);
        float y[8];
        unpack8<T>(praw, y);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float c = (float)cos_row[t0 + e], s = (float)sin_row[t0 + e];
            x[e] = left ? (x[e] * c - y[e] * s) : (x[e] * c + y[e] * s);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Tile products with the A operand in LDS (shared by the general forward kernel and the backward
// kernels)
// ------------------------------------------------------------------------------------------------
constexpr float kLog2e = 1.4426950408889634f;

// s_waitcnt vmcnt(0): placed after the resident operands are loaded, before the tile loop.  Without it
// the compiler cannot prove inside the loop that those loads have landed (a zero-trip path skips the
// first tile's wait) and guards the first product of every step with vmcnt(0), which also waits for
// the NEXT tile's prefetch, i.e. it serialises the prefetch with the products.
FA_DEV void wait_resident_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// accumulate step dk of a product; step 0 starts from an inline zero instead of a cleared accumulator
template <typename T> FA_DEV void mfma_step(f32x16& acc, typename Elem<T>::v8 a, typename Elem<T>::v8 b, int dk) {
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    acc = Elem<T>::mfma32(a, b, dk == 0 ? zero : acc);
}

// Mask of one 32-wide accumulator block: entry r of the lane stands at position
// pos0 + 8 * (r >> 2) + (r & 3) (pos0 includes the lane's 4 * hh) and is visible iff lo <= position <= hi.
// One add, one unsigned compare and one select per entry; hi < lo masks everything.
FA_DEV void mask_acc16(f32x16& s, int pos0, int lo, int hi) {
    const bool any = hi >= lo;
    const uint32_t span = any ? (uint32_t)(hi - lo) : 0u;
    const int z = any ? pos0 - lo : -64;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = (uint32_t)(z + (8 * (r >> 2) + (r & 3))) > span ? -INFINITY : s[r];
}

// accumulator registers [r8, r8+8) -> B operand of the next product
template <typename T> FA_DEV typename Elem<T>::v8 pack_acc8(const f32x16& a, int r8) {
    u32x4 pk;
#pragma unroll
    for (int e = 0; e < 4; e++) pk[e] = pack2<T>(a[r8 + 2 * e], a[r8 + 2 * e + 1]);
    return __builtin_bit_cast(typename Elem<T>::v8, pk);
}

// Per-lane LDS offsets of both read patterns, computed once: the swizzle only involves row & 15, so a
// block of 32 rows (row-wise) or 16 rows (transposed) further down is a compile-time byte offset; and it
// only changes the low four bits of the chunk index, so 16 chunks (8 k-steps, 4 column blocks: 256 bytes)
// further along a row is one too -- the tables hold the first 8 k-steps and 4 column blocks only.
constexpr int kOffsKS = 8, kOffsDB = 4, kOffsPeriodBytes = 256;
template <int D, int KS, int DB>
struct LdsOffs {
    int r[KS < kOffsKS ? KS : kOffsKS];       // row-wise: row l32, k-step dk
    int c[DB < kOffsDB ? DB : kOffsDB][2];    // transposed: column block db, rows 4hh + tj and 8 more
    FA_DEV void init(int lane, int db0 = 0) {      // db0: first 32-column block of the DB blocks this wave reads
        const int l32 = lane & 31, hh = lane >> 5;
#pragma unroll
        for (int dk = 0; dk < (KS < kOffsKS ? KS : kOffsKS); dk++) r[dk] = l32 * (D * 2) + swz_u<D>(dk * 2 + hh, l32) * 16;
        const int tj = (lane & 15) >> 2, tq = lane & 3, dhalf = (lane >> 4) & 1;
        const int row = 4 * hh + tj;
#pragma unroll
        for (int db = 0; db < (DB < kOffsDB ? DB : kOffsDB); db++) {
            const int cc = (db0 + db) * 4 + dhalf * 2 + (tq >> 1);
            c[db][0] = row * (D * 2) + swz_u<D>(cc, row) * 16 + (tq & 1) * 8;
            c[db][1] = (row + 8) * (D * 2) + swz_u<D>(cc, row + 8) * 16 + (tq & 1) * 8;
        }
    }
};
FA_DEV int offs_row(const int* offr, int dk) { return offr[dk % kOffsKS] + (dk / kOffsKS) * kOffsPeriodBytes; }
FA_DEV int offs_col(const int (*offc)[2], int db, int half) { return offc[db % kOffsDB][half] + (db / kOffsDB) * kOffsPeriodBytes; }
template <typename T, int D> FA_DEV typename Elem<T>::v8 lds_rows_at(const char* tile, int off, int blk32) {
    const u32x4 raw = *reinterpret_cast<const u32x4*>(tile + off + blk32 * 32 * (D * 2));
    return __builtin_bit_cast(typename Elem<T>::v8, raw);
}
template <typename T, int D> FA_DEV typename Elem<T>::v8 lds_cols_at(const char* tile, int off_lo, int off_hi, int t16) {
    const u32x2 lo = lds_read_tr16(tile + off_lo + t16 * 16 * (D * 2));
    const u32x2 hi = lds_read_tr16(tile + off_hi + t16 * 16 * (D * 2));
    const u32x4 raw = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(typename Elem<T>::v8, raw);
}

// Tile products whose A operands come from LDS, software-pipelined by hand: the operands of GRP MFMAs
// are read one group ahead into a second register set, and a scheduling fence keeps every group's
// reads in front of the previous group's MFMAs.  (Left to itself the compiler issues read, wait,
// MFMA, read, wait, MFMA ... with one operand register set, and every MFMA pays an LDS round trip.)
//
// acc[blk] (+)= rows [32 blk, 32 blk + 32) of `tile`  x  bfrag[dk]   for blk < NBLK, dk < KS
// (ZERO0 = false: the accumulators already hold the value the product is added to.)
// (GRP0 is the wanted group size; a product whose MFMA count it does not divide -- 6 k-steps of head dim 96 --
// runs in groups of 3 or 2.)
template <typename T, int D, int NBLK, int KS, int GRP0, bool ZERO0 = true>
FA_DEV void product_rows(f32x16* acc, const char* tile, const int* offr, const typename Elem<T>::v8* bfrag) {
    typedef typename Elem<T>::v8 v8;
    constexpr int TOTAL = NBLK * KS, GRP = TOTAL % GRP0 == 0 ? GRP0 : TOTAL % 3 == 0 ? 3 : 2, NG = TOTAL / GRP;
    static_assert(TOTAL % GRP == 0, "group shape");
    // step st -> (k-step st / NBLK, row block st % NBLK): consecutive MFMAs go to different accumulators
    v8 a[2][GRP];
#pragma unroll
    for (int j = 0; j < GRP; j++) a[0][j] = lds_rows_at<T, D>(tile, offs_row(offr, j / NBLK), j % NBLK);
#pragma unroll
    for (int g = 0; g < NG; g++) {
        if (g + 1 < NG) {
#pragma unroll
            for (int j = 0; j < GRP; j++) {
                const int st = (g + 1) * GRP + j;
                a[(g + 1) & 1][j] = lds_rows_at<T, D>(tile, offs_row(offr, st / NBLK), st % NBLK);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < GRP; j++) {
            const int st = g * GRP + j;
            mfma_step<T>(acc[st % NBLK], a[g & 1][j], bfrag[st / NBLK], ZERO0 ? st / NBLK : 1);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}
// acc[db] += columns [32 db, 32 db + 32) of tile rows [16 t16, 16 t16 + 16), transposed  x  bfrag[t16]
template <typename T, int D, int PT, int DB, int GRP0>
FA_DEV void product_cols(f32x16* acc, const char* tile, const int (*offc)[2], const typename Elem<T>::v8* bfrag) {
    typedef typename Elem<T>::v8 v8;
    constexpr int TOTAL = PT * DB, GRP = TOTAL % GRP0 == 0 ? GRP0 : TOTAL % 3 == 0 ? 3 : 2, NG = TOTAL / GRP;
    static_assert(TOTAL % GRP == 0, "group shape");
    v8 a[2][GRP];
#pragma unroll
    for (int j = 0; j < GRP; j++) a[0][j] = lds_cols_at<T, D>(tile, offs_col(offc, j % DB, 0), offs_col(offc, j % DB, 1), j / DB);
#pragma unroll
    for (int g = 0; g < NG; g++) {
        if (g + 1 < NG) {
#pragma unroll
            for (int j = 0; j < GRP; j++) {
                const int st = (g + 1) * GRP + j;
                a[(g + 1) & 1][j] = lds_cols_at<T, D>(tile, offs_col(offc, st % DB, 0), offs_col(offc, st % DB, 1), st / DB);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < GRP; j++) {
            const int st = g * GRP + j;
            acc[st % DB] = Elem<T>::mfma32(a[g & 1][j], bfrag[st / DB], acc[st % DB]);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}

// 16 B per lane from global memory (uniform base + per-lane byte offset) to LDS address
// m0_base + lane * 16, bypassing registers.  The base is uniform by construction; reading it through
// readfirstlane tells the compiler so (the instruction takes it in scalar registers).
FA_DEV void async_fill16(const void* base_uniform, uint32_t lane_offset, uint32_t lds_base_uniform) {
    const uint64_t a = (uint64_t)base_uniform;
    const uint64_t sbase = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a) |
                           ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)) << 32);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_base_uniform), "v"(lane_offset), "s"(sbase) : "memory", "m0");
}
// A pointer that is uniform over the wave by construction, read through readfirstlane so that the compiler keeps it --
// and whatever is stepped from it -- in scalar registers (it cannot always prove the uniformity of values derived
// from the work item, and then spends a 64-bit vector add and two readfirstlanes on every tile request).
template <typename P> FA_DEV const P* scalar_ptr(const P* ptr) {
    const uint64_t a = (uint64_t)ptr;
    return (const P*)((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a) |
                      ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)) << 32));
}
// wait until at most N of this wave's vector-memory operations are outstanding (N < 64: the counter's low four
// bits sit in bits 3:0 of the operand, its upper two in bits 15:14)
template <int N> FA_DEV void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// A wave's 32 resident rows (each lane keeps one row in registers as MFMA operand) fetched through a
// wave-private LDS region of 32 * D * 2 bytes instead of 16 B per lane from 32 different rows: the
// fills are whole 1 KB runs, so the memory system sees 64-byte requests instead of 32 row pieces per
// instruction.  `base` is uniform; row r of the wave is at element offset row_off(r) from it (the
// caller clamps rows past the sequence).  stage_rows_issue only requests; after the wave's vmcnt has
// drained, stage_rows_read hands every lane its row with columns >= d zeroed.
template <typename T, int D, typename RowOff>
FA_DEV void stage_rows_issue(const T* base, RowOff row_off, int d, uint32_t lds_region, int lane) {
    constexpr int ROWB = D * 2;
    const int d_last_chunk = d / 8 - 1;
#pragma unroll
    for (int j = 0; j < ROWB / 32; j++) {
        const int pos = j * 1024 + lane * 16;
        const int r = pos / ROWB;
        const int c = min(swz_u<D>((pos % ROWB) / 16, r), d_last_chunk);
        async_fill16(base, ((uint32_t)row_off(r) + (uint32_t)(c * 8)) * 2u, lds_region + j * 1024);
    }
}
template <typename T, int D, int KS = D / 16>
FA_DEV void stage_rows_read(typename Elem<T>::v8 (&rf)[KS], const char* region, int d, int lane) {
    typedef typename Elem<T>::v8 v8;
    const int l32 = lane & 31, hh = lane >> 5;
    asm volatile("" ::: "memory");     // the region was written by the fills, not by anything the compiler saw
#pragma unroll
    for (int dk = 0; dk < KS; dk++) {
        u32x4 a = *reinterpret_cast<const u32x4*>(region + l32 * (D * 2) + swz_u<D>(dk * 2 + hh, l32) * 16);
        if (dk * 16 + 8 * hh >= d) a = u32x4{0, 0, 0, 0};
        rf[dk] = __builtin_bit_cast(v8, a);
    }
}

// A wave's 32 x (32 DB) accumulator tile (lane l32 = row, registers = columns) to global memory
// through a wave-private LDS region of stage_tile_bytes<DB>() bytes, so that every store instruction
// writes whole rows, 16 B per lane, instead of 8-byte pieces of 32 rows.  `base` points at row 0,
// column 0 of the tile; rows >= rows_ok and columns >= cols_ok are not written.  A row takes a power
// of two of lanes (12 chunks of a 96-column tile: 16 lanes, 4 of them idle).
template <int DB> constexpr int stage_row_lanes() { return DB * 4 <= 4 ? 4 : DB * 4 <= 8 ? 8 : DB * 4 <= 16 ? 16 : 32; }
template <int DB> constexpr int stage_tile_bytes() { return 32 * (stage_row_lanes<DB>() * 16 + 16); }
template <typename T, int DB>
FA_DEV void store_tile_rows(const f32x16 (&acc)[DB], float sc, char* stage, int lane, T* base, int64_t row_stride,
                            int rows_ok, int cols_ok) {
    constexpr int CPR = DB * 4, CPP = stage_row_lanes<DB>(), PITCH = CPP * 16 + 16, RPP = 64 / CPP;
    static_assert(DB <= 8, "row lanes");
    const int l32 = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const int d0 = db * 32 + 8 * q4 + 4 * hh;
            const u32x2 v = {pack2<T>(acc[db][4 * q4] * sc, acc[db][4 * q4 + 1] * sc),
                             pack2<T>(acc[db][4 * q4 + 2] * sc, acc[db][4 * q4 + 3] * sc)};
            *reinterpret_cast<u32x2*>(stage + l32 * PITCH + d0 * 2) = v;
        }
    const int srow = lane / CPP, sch = lane % CPP;
#pragma unroll
    for (int j = 0; j < 32 / RPP; j++) {
        const int rr = j * RPP + srow;
        const u32x4 v = *reinterpret_cast<const u32x4*>(stage + rr * PITCH + sch * 16);
        if (rr < rows_ok && sch < CPR && sch * 8 < cols_ok) st_global16(base + (int64_t)rr * row_stride + sch * 8, v);
    }
}

// Log-sum-exp weighted merge of the split partials of one output row (b, h, i), by one wave: lanes first
// reduce the per-split log-sum-exp values, then stream the partial rows whose weight is non-zero.
// Reference: combine_attn_seqk_parallel, csrc/flash_attn/src/flash_fwd_kernel.h:1169-1327 (all splits
// empty: lse = +inf, out = 0, :1233-1241).
FA_DEV void dec_slot_counts(const KParams& kp, int b, int& n_macro, int& n_sub);
template <typename T>
FA_DEV void combine_row(const KParams& kp, const int64_t row, const int lane) {
    const fa_fwd_params& p = kp.p;
    const int64_t nrows = (int64_t)p.b * p.h * p.seqlen_q;
    const int S = kp.num_splits;

    // which partial slots hold a result: all of them, or (compact persistent decode schedule, whose kernel
    // visits and writes only the slots with keys) the leading complete chunks and the leading pieces of the
    // remainder, as dec_slot_counts gives them
    int n_a = S, n_b = 0, s_a = S;
    if (kp.dec_compact) {
        s_a = kp.dec_sa;
        dec_slot_counts(kp, (int)(row / ((int64_t)p.seqlen_q * p.h)), n_a, n_b);
    }
    auto written = [&](int s) { return s < S && (s < s_a ? s < n_a : s - s_a < n_b); };
    float l0 = written(lane) ? p.lse_accum[(int64_t)lane * nrows + row] : -INFINITY;
    float l1 = written(lane + 64) ? p.lse_accum[(int64_t)(lane + 64) * nrows + row] : -INFINITY;
    float mx = fmaxf(l0, l1);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    const float mref = (mx == -INFINITY) ? 0.f : mx;
    float sum = __expf(l0 - mref) + __expf(l1 - mref);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o);
    const bool dead = (sum == 0.f) || (sum != sum);
    const float lse = dead ? INFINITY : __logf(sum) + mref;
    const float w0 = dead ? 0.f : __expf(l0 - lse);
    const float w1 = dead ? 0.f : __expf(l1 - lse);

    const int i = (int)(row % p.seqlen_q);
    const int h = (int)((row / p.seqlen_q) % p.h);
    const int b = (int)(row / ((int64_t)p.seqlen_q * p.h));
    // rows that stand for (position, grouped head) pairs: see KParams::pack_g
    const int pg = kp.pack_g > 1 ? kp.pack_g : 1;
    const int qi = i / pg, gg = i - qi * pg;
    if (lane == 0) p.softmax_lse[(((int64_t)b * p.h + h) * pg + gg) * (p.seqlen_q / pg) + qi] = lse;

    // each lane owns 4 consecutive output dims (64 lanes x 4 = 256 dims max)
    const int d0 = lane * 4;
    // Only the splits of non-zero weight are fetched (a split of weight zero may never have been written: the
    // slots past a sequence's length), eight rows at a time before any of them is used (one memory round
    // trip per batch instead of one per split), and added in split order.  The set of splits is the same
    // for all lanes of the wave, so the walk over it is scalar.
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int BATCH = 8;
    uint64_t m0 = __builtin_amdgcn_ballot_w64(w0 != 0.f), m1 = __builtin_amdgcn_ballot_w64(w1 != 0.f);
    while ((m0 | m1) != 0) {
        f32x4 v[BATCH];
        float w[BATCH];
        int last = 0;
#pragma unroll
        for (int j = 0; j < BATCH; j++) {
            int sidx = -1;
            if (m0 != 0) { sidx = __builtin_ctzll(m0); m0 &= m0 - 1; }
            else if (m1 != 0) { sidx = 64 + __builtin_ctzll(m1); m1 &= m1 - 1; }
            w[j] = sidx >= 0 ? __shfl(sidx < 64 ? w0 : w1, sidx & 63) : 0.f;
            if (sidx >= 0) last = sidx;
            // (past the end of the set the last row is fetched again, with weight zero)
            const float* src = p.o_accum + ((int64_t)last * nrows + row) * kp.d_rounded + min(d0, kp.d_rounded - 4);
            v[j] = *reinterpret_cast<const f32x4*>(src);
        }
#pragma unroll
        for (int j = 0; j < BATCH; j++)
            if (w[j] != 0.f) acc += v[j] * w[j];
    }
    if (d0 < p.d) {
        int64_t off = (int64_t)qi * p.o_row_stride + (int64_t)h * p.o_head_stride + (int64_t)b * p.o_batch_stride;
        if (pg > 1) off += (int64_t)gg * kp.pack_o_hs;
        u32x2 v = {pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3])};
        st_global8(reinterpret_cast<T*>(p.o) + off + d0, v);
    }
}

// Resolved per-(batch) sequence bookkeeping.  Mirrors the reference's BlockInfo
// (csrc/flash_attn/src/block_info.h:11-42) with 64-bit offsets.
struct SeqInfo {
    int sq, sk, sk_cache;      // rows of q, visible keys, keys in the cache before the append
    int64_t q_off, k_off, v_off, o_off;   // element offsets of (row 0, head 0) of this batch entry
    int q_row0;                // first packed row (varlen) for lse indexing: unused for dense
};
FA_DEV SeqInfo seq_info(const fa_fwd_params& p, int b) {
    SeqInfo s;
    if (p.cu_seqlens_q) {
        int r0 = p.cu_seqlens_q[b];
        s.sq = p.cu_seqlens_q[b + 1] - r0;
        s.q_off = (int64_t)r0 * p.q_row_stride;
        s.o_off = (int64_t)r0 * p.o_row_stride;
    } else {
        s.sq = p.seqlen_q;
        s.q_off = (int64_t)b * p.q_batch_stride;
        s.o_off = (int64_t)b * p.o_batch_stride;
    }
    // the four strides are read as values before the branch: a choice between the ADDRESSES of two fields
    // makes the compiler keep a copy of them in per-lane scratch memory and index it
    const int64_t k_row = p.k_row_stride, v_row = p.v_row_stride, k_batch = p.k_batch_stride, v_batch = p.v_batch_stride;
    if (p.cu_seqlens_k && p.is_seqlens_k_cumulative) {
        int r0 = p.cu_seqlens_k[b];
        s.sk_cache = p.cu_seqlens_k[b + 1] - r0;
        s.sk = s.sk_cache;
        s.k_off = (int64_t)r0 * k_row;
        s.v_off = (int64_t)r0 * v_row;
    } else {
        const int bk = p.cache_batch_idx ? p.cache_batch_idx[b] : b;
        // a cache length outside [0, capacity] is a caller error; clamped so that no key, rotary
        // table row or appended row beyond the cache is ever touched
        s.sk_cache = p.cu_seqlens_k ? min(max(p.cu_seqlens_k[b], 0), p.seqlen_k) : p.seqlen_k;
        s.sk = min(s.sk_cache + p.seqlen_knew, p.seqlen_k);
        s.k_off = (int64_t)bk * k_batch;
        s.v_off = (int64_t)bk * v_batch;
    }
    s.q_row0 = 0;
    return s;
}

// Persistent decode schedule without a left window bound: the keys of batch entry b are [0, hi), hi = the
// sequence's length (a right bound of the mask never hides keys from the last query row).  Slots with keys:
// the first n_macro complete chunks of split_len keys, and the first n_sub pieces of dec_sub keys of the
// remainder (decode_item, kMacro / kSub).
FA_DEV void dec_slot_counts(const KParams& kp, int b, int& n_macro, int& n_sub) {
    const int hi = seq_info(kp.p, b).sk;
    const int whole = hi / kp.split_len;
    n_macro = min(kp.dec_sa, whole);
    n_sub = min(kp.dec_sb, (hi - whole * kp.split_len + kp.dec_sub - 1) / kp.dec_sub);
}

// Key range of one work item.  kChunk: chunk `idx` of kp.split_len keys.  kMacro / kSub are the two
// passes of the persistent schedule: first every COMPLETE chunk of kp.split_len keys, then the
// ragged remainder of each sequence in pieces of kp.dec_sub keys, so that the last items handed out
// are small and the workgroups finish together.
enum ItemMode { kChunk = 0, kMacro = 1, kSub = 2 };
// keys [c_lo, c_hi) of work item (mode, idx) of a sequence whose visible keys end at hi
FA_DEV void item_key_range(const KParams& kp, int mode, int idx, int hi, int& c_lo, int& c_hi) {
    if (mode == kSub) {
        const int base = hi / kp.split_len * kp.split_len;     // start of the incomplete chunk
        c_lo = base + idx * kp.dec_sub;
        c_hi = (base == hi) ? c_lo : c_lo + kp.dec_sub;
    } else {
        c_lo = idx * kp.split_len;
        c_hi = c_lo + kp.split_len;
        if (mode == kMacro && c_hi > hi) c_hi = c_lo;          // incomplete: left to the kSub pass
    }
}

// A counter that needs no set-up launch and survives a launch that never finished.  The 64-bit word (two of the
// caller's int32 words, 8-byte aligned) holds (epoch << 32) | count; `epoch` is a non-zero number the host draws
// anew, rising, for every call.  A word whose upper half is not this launch's epoch -- zero as every finished
// launch leaves it, or whatever a launch that was torn down mid-way, or a caller that did not clear the words, left
// behind -- counts as zero.  The usual draw is one atomic add.  A draw that finds a foreign upper half raises the
// word to (epoch, 0) with one atomic maximum (idempotent: whoever comes first installs, increments made on the old
// contents are dropped with them) and draws again; only contents ABOVE the epoch -- a word poisoned from outside,
// or the replay of an old graph after a younger call was torn down -- need the compare-and-swap loop, which ends
// after at most one failed attempt per other lane installing at that moment.  Nothing waits for another workgroup.
// Returns the value before the increment.
FA_DEV uint32_t epoch_counter_next(int32_t* words, uint32_t epoch) {
    uint64_t* w = reinterpret_cast<uint64_t*>(words);
    uint64_t old = __hip_atomic_fetch_add(w, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((uint32_t)(old >> 32) == epoch) return (uint32_t)old;
    __hip_atomic_fetch_max(w, (uint64_t)epoch << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    old = __hip_atomic_fetch_add(w, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((uint32_t)(old >> 32) == epoch) return (uint32_t)old;
    const uint64_t fresh = ((uint64_t)epoch << 32) | 1u;
    for (;;) {
        uint64_t cur = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((uint32_t)(cur >> 32) == epoch) {
            old = __hip_atomic_fetch_add(w, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return (uint32_t)old;
        }
        if (__hip_atomic_compare_exchange_strong(w, &cur, fresh, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            return 0u;
    }
}

// The persistent schedule itself, for a grid of resident workgroups: calls Item::run(kp, smem, kv head, batch
// entry, partial slot, mode, idx) for this workgroup's block id and then for every ticket it draws from
// the counter in kp.work_counter[0..1] until the items are used up; workgroups that have left are counted in
// kp.work_counter[2..3] and the last one puts all four words back to zero (epoch_counter_next).  All lanes of
// the workgroup must call it together and return from every item (it synchronises the workgroup between items,
// so an item may use all of the dynamic LDS, `smem`).
template <class Item>
FA_DEV void for_each_ticket(const KParams& kp, char* smem) {
    __shared__ int s_ticket;
    // compact schedule: s_pm[b] / s_ps[b] = slots with keys (complete chunks / remainder pieces) of the batch
    // entries before b; tickets then number only those slots, batch entry by batch entry, kv heads fastest
    __shared__ int s_pm[kDecCompactMaxBatch + 1], s_ps[kDecCompactMaxBatch + 1];
    const fa_fwd_params& p = kp.p;
    int n_macro = p.b * kp.dec_sa * p.h_k;
    int total = n_macro + p.b * kp.dec_sb * p.h_k;
    if (kp.dec_compact) {
        for (int bb = threadIdx.x; bb < p.b; bb += blockDim.x) {
            int nm, ns;
            dec_slot_counts(kp, bb, nm, ns);
            s_pm[bb + 1] = nm;
            s_ps[bb + 1] = ns;
        }
        __syncthreads();
        if (threadIdx.x < 64) {        // one wave turns the counts into running sums, 64 entries at a time
            const int lane = threadIdx.x;
            int carry_m = 0, carry_s = 0;
            for (int base = 0; base < p.b; base += 64) {
                const int i = base + lane;
                int vm = i < p.b ? s_pm[i + 1] : 0, vs = i < p.b ? s_ps[i + 1] : 0;
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) {
                    const int um = __shfl_up(vm, o), us = __shfl_up(vs, o);
                    if (lane >= o) { vm += um; vs += us; }
                }
                if (i < p.b) { s_pm[i + 1] = carry_m + vm; s_ps[i + 1] = carry_s + vs; }
                carry_m += __shfl(vm, 63);
                carry_s += __shfl(vs, 63);
            }
            if (lane == 0) { s_pm[0] = 0; s_ps[0] = 0; }
        }
        __syncthreads();
        n_macro = s_pm[p.b] * p.h_k;
        total = n_macro + s_ps[p.b] * p.h_k;
    }
    // the first item of a workgroup is the one its block id names (no round trip to the counter before any
    // work starts); the tickets drawn afterwards continue behind the grid
    for (bool first = true;; first = false) {
        int t = (int)blockIdx.x;
        if (!first) {
            __syncthreads();          // previous item is done with LDS and with s_ticket
            if (threadIdx.x == 0) s_ticket = (int)gridDim.x + (int)epoch_counter_next(kp.work_counter, kp.epoch);
            __syncthreads();
            t = s_ticket;
        }
        if (t >= total) break;
        const bool macro = t < n_macro;
        if (!macro) t -= n_macro;
        int hk, idx, b;
        if (kp.dec_compact) {
            const int* pre = macro ? s_pm : s_ps;
            hk = t % p.h_k;
            const int q = t / p.h_k;            // q-th slot with keys of its pass: the batch entry is the last b with pre[b] <= q
            int lo_b = 0, hi_b = p.b;           // invariant: pre[lo_b] <= q < pre[hi_b]
            while (hi_b - lo_b > 1) {
                const int mid = (lo_b + hi_b) >> 1;
                if (pre[mid] <= q) lo_b = mid; else hi_b = mid;
            }
            b = lo_b;
            idx = q - pre[b];
        } else {
            const int per_b = macro ? kp.dec_sa : kp.dec_sb;
            hk = t % p.h_k; idx = (t / p.h_k) % per_b; b = t / (p.h_k * per_b);
        }
        Item::run(kp, smem, hk, b, macro ? idx : kp.dec_sa + idx, macro ? kMacro : kSub, idx);
    }
    if (threadIdx.x == 0) {
        const uint32_t gone = epoch_counter_next(kp.work_counter + 2, kp.epoch);
        if (gone == gridDim.x - 1u) {     // every workgroup has drawn its last ticket: leave both counters fresh
            uint64_t* w = reinterpret_cast<uint64_t*>(kp.work_counter);
            __hip_atomic_store(w, (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(w + 1, (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Which work item a workgroup of the tiled forward and backward kernels takes.  Block ids are dealt round-robin
// over the 8 XCDs by hardware, each XCD has its own L2, and all row blocks of a (batch, kv head)
// stream should meet in one L2 (heavy blocks first; grouped q heads adjacent).
//  * Dense batches: every stream costs the same, so XCD x takes the x-th contiguous eighth of the
//    (batch, kv head, row block, group) order, which balances the XCDs to within one item.
//  * Packed variable-length batches: streams cost as their sequence length squared, and a contiguous
//    eighth is a handful of whole sequences (64 sequences x 16 heads: 8 sequences per XCD, whose
//    summed cost varies by tens of percent).  There XCD x takes every 8th stream of the order in which
//    kv heads vary fastest, so the heads of each sequence are spread over the XCDs.
__host__ __device__ inline bool xcd_strided(bool varlen, int64_t batch, int64_t h_k) { return varlen && batch * h_k >= 8; }
// Every (batch, kv head) stream has per_stream work units, heavy ones first; yields this workgroup's
// unit and stream.  `slots` is the number of workgroups an XCD holds at once (32 CUs x workgroups
// per CU).  A stream with fewer units than slots cannot keep an XCD busy by itself, and handing the
// streams out one after the other leaves the CUs that drew a stream's light units idle while its
// heavy ones finish (causal row blocks cost as their index; 16 blocks on 32 slots: 9 % lost, 8 on
// 64: 20-35 %).  So the streams of an XCD are taken k at a time, k * per_stream >= slots, and inside
// such a group the order is unit-major: the heaviest unit of each of the k streams, then the next.
// The k streams then share the L2 (k x K/V of a short sequence is no more than one long one).
// Callers pass slots = 0 (k = 1, one stream after the other) when no mask is active: all units of
// a stream then cost the same and sharing the L2 only costs (measured -1..2 %).
//
// The hardware hands the workgroups of a grid to the 4 shader engines of an XCD in strict rotation and in
// order: a workgroup waits for a free CU of its own engine, and every later workgroup waits behind it.
// Dealing one dense stream's units out in falling cost gives one engine the heaviest unit of every four and
// leaves the other three idle behind it (measured: 8 % of a causal 8k launch, 18 % at 4k).  `equal` is the
// number of consecutive units of a stream that cost the same (the grouped q heads of a row block); for
// dense batches k is rounded up so that k * equal is a multiple of 4: every four consecutive workgroups
// then cost the same and each engine works through streams of its own at the same pace.  Packed batches
// keep the smaller k: their streams differ in length, and giving an engine a stream of its own would
// unbalance the engines instead.
FA_DEV bool xcd_stream_unit(bool strided, uint32_t batch, uint32_t h_k, uint32_t per_stream, uint32_t slots, uint32_t equal,
                            uint32_t& unit, int& hk, int& b) {
    const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3, S = batch * h_k;
    uint32_t s;
    if (!strided && (S & 7u) != 0u) {
        // Dense batch whose streams do not divide over the XCDs: contiguous eighths of the unit
        // order.  With fewer than 8 streams (a single sequence on one to four kv heads, say) and a
        // mask, the units are ordered by falling cost and a contiguous eighth would hand XCD 0 the
        // heaviest row blocks of a stream (23 % of a causal stream's work instead of 12.5 %): there
        // the units are dealt to the XCDs one by one and a stream's K/V is read through every L2
        // (16k causal, 8 q heads on 1 kv head: 684 -> 1122 TFLOP/s).  From 8 streams on, an eighth
        // spans whole streams and dealing only costs L2 hits (36 streams, d 64: -28 %).
        const uint32_t w = (slots && S < 8u) ? j * 8u + x : x * (gridDim.x >> 3) + j;
        unit = w % per_stream;
        s = w / per_stream;
    } else {
        const uint32_t n_local = strided ? (S + 7u - x) >> 3 : S >> 3;       // streams of this XCD
        uint32_t k = (slots + per_stream - 1u) / per_stream;
        if (!strided && slots != 0u) {
            const uint32_t m = (equal & 3u) == 0u ? 1u : (equal & 1u) == 0u ? 2u : 4u;
            k = (k + m - 1u) / m * m;
        }
        k = max(1u, min(k, n_local));
        const uint32_t grp = j / (k * per_stream), first = grp * k;
        if (first >= n_local) return false;
        const uint32_t kk = min(k, n_local - first);                          // the last group may be short
        const uint32_t r = j - grp * k * per_stream;
        if (r >= kk * per_stream) return false;
        unit = r / kk;
        const uint32_t ls = first + r % kk;
        s = strided ? ls * 8u + x : x * n_local + ls;
    }
    if (s >= S) return false;
    hk = (int)(s % h_k);
    b = (int)(s / h_k);
    return true;
}
// grid size that goes with xcd_stream_unit (host side); 0 when it does not fit 31 bits
inline int64_t xcd_grid(bool strided, int64_t batch, int64_t h_k, int64_t per_stream) {
    const int64_t per_xcd = strided ? (batch * h_k + 7) / 8 * per_stream : (batch * h_k * per_stream + 7) / 8;
    return per_xcd * 8 > 0x7fffffffLL ? 0 : per_xcd * 8;
}
// Packed batches with one or two kv heads (MQA / GQA, or a tensor-parallel shard of them): whole
// (sequence, kv head) streams cannot give every XCD a piece of every sequence, so in the forward
// kernels the grouped q heads of a stream are cut into `parts` (h_k * parts = 8) and each part is
// handed out as a stream of its own: the XCDs get equal work whatever the sequence lengths are
// (64 sequences, 32 q heads on 1 kv head: 600-700 -> 940-960 TFLOP/s; 16 on 2: +17 %).  The parts
// of a stream read its K/V through different L2s; with 4 kv heads (2 parts) that costs more than
// the balance gains at head dim 64, and the dQ pass, which re-reads K and V per row block, loses
// with 2 kv heads too, so the backward kernels keep whole streams (split = false).
__host__ __device__ inline uint32_t xcd_parts(bool split, bool varlen, uint32_t h_k, uint32_t G) {
    if (!split || !varlen || h_k > 2u) return 1u;
    const uint32_t want = 8u / h_k;
    return G % want == 0u ? want : 1u;
}
// Forward kernels and the dQ pass: a stream's units are its row blocks (heavy, late ones first) x
// grouped q heads.
FA_DEV bool xcd_rows_item(bool split, bool varlen, uint32_t batch, uint32_t h_k, uint32_t G, uint32_t nmb, uint32_t slots,
                          int& g, int& mb, int& hk, int& b) {
    const uint32_t parts = xcd_parts(split, varlen, h_k, G), Gp = G / parts, hp = h_k * parts;
    uint32_t unit;
    int hkp;
    if (!xcd_stream_unit(xcd_strided(varlen, batch, hp), batch, hp, Gp * nmb, slots, Gp, unit, hkp, b)) return false;
    hk = (int)((uint32_t)hkp / parts);
    g = (int)(((uint32_t)hkp % parts) * Gp + unit % Gp);
    const uint32_t u = unit / Gp;
    mb = (int)(nmb - 1u - u);
    return true;
}
inline int64_t xcd_rows_grid(bool split, bool varlen, int64_t batch, int64_t h_k, int64_t G, int64_t nmb) {
    const int64_t parts = xcd_parts(split, varlen, (uint32_t)h_k, (uint32_t)G);
    return xcd_grid(xcd_strided(varlen, batch, h_k * parts), batch, h_k * parts, G / parts * nmb);
}
FA_DEV bool xcd_work_item(const KParams& kp, uint32_t nmb, uint32_t slots, int& g, int& mb, int& hk, int& b) {
    const fa_fwd_params& p = kp.p;
    const uint32_t G = (uint32_t)(p.h / p.h_k);
    if (kp.work_items) {
        const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3;
        if (j >= (uint32_t)kp.work_items[x]) return false;      // the slots past the list come last in the grid
        const int32_t* it = kp.work_items + kWorkListHeaderWords + ((size_t)x * (gridDim.x >> 3) + j) * 2;
        b = it[0];
        const uint32_t w = (uint32_t)it[1], head = w >> 16;
        mb = (int)(w & 0xffffu);
        hk = (int)(head / G);
        g = (int)(head % G);
        return true;
    }
    return xcd_rows_item(true, p.cu_seqlens_q != nullptr, (uint32_t)p.b, (uint32_t)p.h_k, G, nmb, slots, g, mb, hk, b);
}
inline int64_t xcd_grid(const fa_fwd_params& p, int64_t nmb) {
    return xcd_rows_grid(true, p.cu_seqlens_q != nullptr, p.b, p.h_k, p.h / p.h_k, nmb);
}

}  // namespace fa
