// Small memory-bound kernels around the attention kernels:
//  * combine: log-sum-exp weighted merge of split-KV partials
//    (reference: combine_attn_seqk_parallel, csrc/flash_attn/src/flash_fwd_kernel.h:1169-1327);
//  * append_kv: copy of k_new / v_new (new keys rotated) into the cache rows
//    [cache_seqlens[b], cache_seqlens[b] + seqlen_knew) of cache row cache_batch_idx[b]
//    (reference: the Append_KV prologue, flash_fwd_kernel.h:763-852, copy_w_min_idx /
//    copy_rotary_* in csrc/flash_attn/src/utils.h:358-517).
#include "fa_common.h"
#include "fa_launch.h"

namespace fa {

// One wave per output row (b, h, i): combine_row (fa_common.h).
template <typename T>
__global__ void __launch_bounds__(256) combine_kernel(const KParams kp) {
    const int64_t nrows = (int64_t)kp.p.b * kp.p.h * kp.p.seqlen_q;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= nrows) return;
    combine_row<T>(kp, row, threadIdx.x & 63);
}

int launch_combine(const KParams& kp, hipStream_t stream) {
    const int64_t nrows = (int64_t)kp.p.b * kp.p.h * kp.p.seqlen_q;
    if (nrows == 0) return 0;
    dim3 grid((unsigned)((nrows + 3) / 4)), block(256);
    if (kp.p.dtype == FA_DTYPE_BF16) hipLaunchKernelGGL(combine_kernel<__bf16>, grid, block, 0, stream, kp);
    else hipLaunchKernelGGL(combine_kernel<_Float16>, grid, block, 0, stream, kp);
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Work list of a packed (variable-length) forward launch.
//
// The hardware hands the workgroups that fall to an XCD to its 4 shader engines in strict rotation and in
// order (see xcd_stream_unit).  The arithmetic order of packed batches cannot follow that rule well: it
// does not know the lengths, so the row blocks a short sequence does not have are empty workgroups in the
// middle of the order, and streams of unequal length run side by side.  This kernel reads cu_seqlens_q on
// the device and writes, per XCD, the list the attention kernel then walks: sequences by falling length
// (so neighbouring streams cost about the same), four streams at a time, row block by row block from the
// last (heaviest under a causal mask) down, and nothing for row blocks that do not exist.  The slots of
// the grid past the end of a list exit at once, after all work has been handed out.
// XCD x owns q heads of kv-head parts x, x + 8, ... of every sequence (h_k * parts is a multiple of 8), as
// in the arithmetic order.  One workgroup per XCD.
// ------------------------------------------------------------------------------------------------
struct WorkListParams {
    const int32_t* cu_seqlens_q;
    int32_t b, h_k, G, parts, block_m, nmb, per_xcd;
    int32_t* out;            // kWorkListHeaderWords counts, then 8 lists of per_xcd two-word slots
};
__global__ void __launch_bounds__(1024) work_list_kernel(const WorkListParams w) {
    __shared__ int len_s[kWorkListMaxBatch];
    __shared__ int order_s[kWorkListMaxBatch];       // rank -> batch index
    __shared__ int scan_s[256];
    const int x = blockIdx.x, t = threadIdx.x, nb = w.b;
    for (int i = t; i < nb; i += 1024) len_s[i] = max(w.cu_seqlens_q[i + 1] - w.cu_seqlens_q[i], 0);
    __syncthreads();
    for (int i = t; i < nb; i += 1024) {
        const int li = len_s[i];
        int r = 0;
        for (int j = 0; j < nb; j++) r += (len_s[j] > li || (len_s[j] == li && j < i)) ? 1 : 0;
        order_s[r] = i;
    }
    __syncthreads();
    const int Gp = w.G / w.parts, E = (w.h_k * w.parts / 8) * Gp;     // streams per sequence on this XCD
    const int ns = nb * E, ng = (ns + 3) / 4;
    // (a length beyond the seqlen_q the grid was sized for is the caller's error; it must not overrun the list)
    auto units = [&](int s) { return s < ns ? min((len_s[order_s[s / E]] + w.block_m - 1) / w.block_m, w.nmb) : 0; };
    // Four threads per owner: owner o holds groups [o * gpt, (o + 1) * gpt), thread j of it writes stream j of
    // each.  Items before an owner's groups: inclusive scan over the owners' totals.
    const int o = t >> 2, jj = t & 3;
    const int gpt = (ng + 255) / 256;
    const int g_lo = min(o * gpt, ng), g_hi = min(g_lo + gpt, ng);
    int mine = 0;
    for (int g = g_lo; g < g_hi; g++) mine += units(4 * g) + units(4 * g + 1) + units(4 * g + 2) + units(4 * g + 3);
    if (jj == 0) scan_s[o] = mine;
    __syncthreads();
    const int owners = min(256, (ng + gpt - 1) / gpt);      // owners with work; the others hold zero
    for (int d = 1; d < owners; d <<= 1) {
        const int v = (jj == 0 && o >= d) ? scan_s[o - d] : 0;
        __syncthreads();
        if (jj == 0) scan_s[o] += v;
        __syncthreads();
    }
    int off = scan_s[o] - mine;
    if (t == 0) w.out[x] = owners > 0 ? scan_s[owners - 1] : 0;
    int32_t* list = w.out + kWorkListHeaderWords + (size_t)x * w.per_xcd * 2;
    for (int g = g_lo; g < g_hi; g++) {
        int u[4];
        for (int j = 0; j < 4; j++) u[j] = units(4 * g + j);
        const int s = 4 * g + jj;
        if (s < ns) {
            const int bb = order_s[s / E], e = s % E;
            const int hkp = x + 8 * (e / Gp);
            const int head = (hkp / w.parts) * w.G + (hkp % w.parts) * Gp + e % Gp;
            const int mine_u = u[jj];
            for (int un = 0; un < mine_u; un++) {
                // unit-major inside the group; lengths fall with the stream index, so the streams that still
                // have unit `un` are a prefix of the group
                const int pos = off + min(u[0], un) + min(u[1], un) + min(u[2], un) + min(u[3], un) + jj;
                list[2 * pos] = bb;
                list[2 * pos + 1] = (int32_t)(((uint32_t)head << 16) | (uint32_t)(mine_u - 1 - un));
            }
        }
        off += u[0] + u[1] + u[2] + u[3];
    }
}

static bool work_list_applies(const fa_fwd_params& p) {
    if (!p.cu_seqlens_q || p.b <= 0 || p.b > kWorkListMaxBatch || p.h >= 65536) return false;
    const uint32_t G = (uint32_t)(p.h / p.h_k), parts = xcd_parts(true, true, (uint32_t)p.h_k, G);
    return ((uint32_t)p.h_k * parts) % 8u == 0u;
}
int64_t work_list_words(const fa_fwd_params& p) {
    if (!work_list_applies(p)) return 0;
    // the smallest row block (128 rows) gives the longest lists
    const int64_t nmb = (p.seqlen_q + 127) / 128;
    return FA_WORK_COUNTER_WORDS + kWorkListHeaderWords + 2 * xcd_grid(p, nmb);
}
int prepare_work_list(KParams& kp, int block_m, int64_t nblocks, hipStream_t stream) {
    const fa_fwd_params& p = kp.p;
    kp.work_items = nullptr;
    if (!work_list_applies(p) || !kp.work_counter || nblocks <= 0 || (nblocks & 7) != 0) return 0;
    if ((p.seqlen_q + block_m - 1) / block_m >= 65536) return 0;
    if ((int64_t)p.work_counter_len < FA_WORK_COUNTER_WORDS + kWorkListHeaderWords + 2 * nblocks) return 0;
    WorkListParams w;
    w.cu_seqlens_q = p.cu_seqlens_q;
    w.b = p.b; w.h_k = p.h_k; w.G = p.h / p.h_k;
    w.parts = (int32_t)xcd_parts(true, true, (uint32_t)p.h_k, (uint32_t)w.G);
    w.block_m = block_m;
    w.nmb = (p.seqlen_q + block_m - 1) / block_m;
    w.per_xcd = (int32_t)(nblocks / 8);
    w.out = kp.work_counter + FA_WORK_COUNTER_WORDS;
    hipLaunchKernelGGL(work_list_kernel, dim3(8), dim3(1024), 0, stream, w);
    if (int e = (int)hipGetLastError()) return e;
    kp.work_items = w.out;
    return 0;
}

// One thread per 16-byte chunk of one new (token, kv-head) row.
template <typename T>
__global__ void __launch_bounds__(256) append_kv_kernel(const KParams kp) {
    const fa_fwd_params& p = kp.p;
    const int cpr = p.d / 8;
    const int64_t total = (int64_t)p.b * p.seqlen_knew * p.h_k * cpr;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int c = (int)(idx % cpr);
    const int hk = (int)((idx / cpr) % p.h_k);
    const int t = (int)((idx / ((int64_t)cpr * p.h_k)) % p.seqlen_knew);
    const int b = (int)(idx / ((int64_t)cpr * p.h_k * p.seqlen_knew));
    const int len = p.cu_seqlens_k ? min(max(p.cu_seqlens_k[b], 0), p.seqlen_k) : p.seqlen_k;
    const int pos = len + t;
    if (pos >= p.seqlen_k) return;     // never write past the cache capacity
    const int bk = p.cache_batch_idx ? p.cache_batch_idx[b] : b;
    const int d0 = c * 8;

    const T* vsrc = reinterpret_cast<const T*>(p.v_new) + (int64_t)b * p.vnew_batch_stride + (int64_t)t * p.vnew_row_stride + (int64_t)hk * p.vnew_head_stride;
    T* vdst = reinterpret_cast<T*>(const_cast<void*>(p.v)) + (int64_t)bk * p.v_batch_stride + (int64_t)pos * p.v_row_stride + (int64_t)hk * p.v_head_stride;
    st_global16(vdst + d0, ld_global16(vsrc + d0));

    const T* ksrc = reinterpret_cast<const T*>(p.k_new) + (int64_t)b * p.knew_batch_stride + (int64_t)t * p.knew_row_stride + (int64_t)hk * p.knew_head_stride;
    T* kdst = reinterpret_cast<T*>(const_cast<void*>(p.k)) + (int64_t)bk * p.k_batch_stride + (int64_t)pos * p.k_row_stride + (int64_t)hk * p.k_head_stride;
    u32x4 raw = ld_global16(ksrc + d0);
    if (p.rotary_dim > 0 && d0 < p.rotary_dim) {
        const T* cr = reinterpret_cast<const T*>(p.rotary_cos) + (int64_t)pos * (p.rotary_dim / 2);
        const T* sr = reinterpret_cast<const T*>(p.rotary_sin) + (int64_t)pos * (p.rotary_dim / 2);
        float x[8];
        unpack8<T>(raw, x);
        rotary8<T>(x, ksrc, cr, sr, d0, p.rotary_dim, p.is_rotary_interleaved != 0);
        raw = pack8<T>(x);
    }
    st_global16(kdst + d0, raw);
}

int launch_append_kv(const KParams& kp, hipStream_t stream) {
    const fa_fwd_params& p = kp.p;
    const int64_t total = (int64_t)p.b * p.seqlen_knew * p.h_k * (p.d / 8);
    if (total == 0) return 0;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (p.dtype == FA_DTYPE_BF16) hipLaunchKernelGGL(append_kv_kernel<__bf16>, grid, block, 0, stream, kp);
    else hipLaunchKernelGGL(append_kv_kernel<_Float16>, grid, block, 0, stream, kp);
    return (int)hipGetLastError();
}

// q rows of a kv-cache call rotated to their positions and written to the rows of the output tensor -- what the
// general tiled kernel does while it loads its Q fragments (prefill_item, fa_prefill.h; same arithmetic: fp32,
// rounded once; the position stops at the last row the table is known to cover), as a pass of its own for the
// launches that then take the pipelined / ping-pong kernels, which read Q without rotating it.  The attention
// kernel afterwards reads its Q rows from `o` and writes its results over them: a workgroup reads only the rows
// it writes, and all of them before it writes any.
template <typename T>
__global__ void __launch_bounds__(256) rotate_q_kernel(const KParams kp) {
    const fa_fwd_params& p = kp.p;
    const int cpr = p.d / 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.b * p.seqlen_q * p.h * cpr) return;
    const int c = (int)(idx % cpr);
    int64_t r = idx / cpr;
    const int head = (int)(r % p.h); r /= p.h;
    const int i = (int)(r % p.seqlen_q);
    const int b = (int)(r / p.seqlen_q);
    const SeqInfo si = seq_info(p, b);
    const T* qrow = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)i * p.q_row_stride + (int64_t)head * p.q_head_stride;
    T* orow = reinterpret_cast<T*>(p.o) + si.o_off + (int64_t)i * p.o_row_stride + (int64_t)head * p.o_head_stride;
    const int d0 = c * 8;
    u32x4 raw = ld_global16(qrow + d0);
    if (d0 < p.rotary_dim) {
        // (without a mask every row is rotated to the position of the first new token)
        const int pos = min(si.sk_cache + ((kp.has_left || kp.has_right) ? i : 0), p.seqlen_k - 1);
        const T* cr = reinterpret_cast<const T*>(p.rotary_cos) + (int64_t)pos * (p.rotary_dim / 2);
        const T* sr = reinterpret_cast<const T*>(p.rotary_sin) + (int64_t)pos * (p.rotary_dim / 2);
        float x[8];
        unpack8<T>(raw, x);
        rotary8<T>(x, qrow, cr, sr, d0, p.rotary_dim, p.is_rotary_interleaved != 0);
        raw = pack8<T>(x);
    }
    st_global16(orow + d0, raw);
}

int launch_rotate_q(const KParams& kp, hipStream_t stream) {
    const fa_fwd_params& p = kp.p;
    const int64_t total = (int64_t)p.b * p.seqlen_q * p.h * (p.d / 8);
    if (total == 0) return 0;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (p.dtype == FA_DTYPE_BF16) hipLaunchKernelGGL(rotate_q_kernel<__bf16>, grid, block, 0, stream, kp);
    else hipLaunchKernelGGL(rotate_q_kernel<_Float16>, grid, block, 0, stream, kp);
    return (int)hipGetLastError();
}

// Testing aid behind return_softmax (the reference's S_dmask, csrc/flash_attn/flash_api.cpp:351-357):
// s_dmask[b, h, i, j] = exp(scale q_i . k_j - lse_i), negated where dropout removed the entry, 0 where
// the mask hides it or outside (seqlen_q, seqlen_k).  Runs after the attention kernel, so lse is
// final and the value is the normalised probability.  One thread per entry, scalar dot product.
template <typename T>
__global__ void __launch_bounds__(256) attn_probs_kernel(const KParams kp) {
    const fa_fwd_params& p = kp.p;
    const int b = blockIdx.z / p.h, head = blockIdx.z % p.h;
    const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int j = blockIdx.x * 16 + (threadIdx.x & 15);
    if (i >= p.sdm_rows || j >= p.sdm_cols) return;
    const SeqInfo si = seq_info(p, b);
    const int hk = head / (p.h / p.h_k);
    const int shift = si.sk - si.sq;
    bool vis = i < si.sq && j < si.sk;
    if (kp.has_right) vis = vis && j <= i + shift + p.window_right;
    if (kp.has_left) vis = vis && j >= i + shift - p.window_left;
    float val = 0.f;
    if (vis) {
        const T* q = reinterpret_cast<const T*>(p.q) + si.q_off + (int64_t)i * p.q_row_stride + (int64_t)head * p.q_head_stride;
        const T* k = reinterpret_cast<const T*>(p.k) + si.k_off + (int64_t)j * p.k_row_stride + (int64_t)hk * p.k_head_stride;
        float dot = 0.f;
        for (int c = 0; c < p.d; c += 8) {
            float a[8], bb[8];
            unpack8<T>(ld_global16(q + c), a);
            unpack8<T>(ld_global16(k + c), bb);
#pragma unroll
            for (int e = 0; e < 8; e++) dot += a[e] * bb[e];
        }
        const float lse = p.softmax_lse[((int64_t)b * p.h + head) * p.seqlen_q + i];
        val = __expf(dot * p.softmax_scale - lse);
        if (p.p_dropout > 0.f) {
            const Drop drop = drop_init(p.rng_state, p.p_dropout, b, head, p.h);
            if (!drop_keep(drop, i, j)) val = -val;
        }
    }
    reinterpret_cast<T*>(p.s_dmask)[(((int64_t)b * p.h + head) * p.sdm_rows + i) * p.sdm_cols + j] = (T)val;
}

int launch_attn_probs(const KParams& kp, hipStream_t stream) {
    const fa_fwd_params& p = kp.p;
    if (p.sdm_rows <= 0 || p.sdm_cols <= 0) return 0;
    dim3 grid((unsigned)((p.sdm_cols + 15) / 16), (unsigned)((p.sdm_rows + 15) / 16), (unsigned)(p.b * p.h));
    if (p.dtype == FA_DTYPE_BF16) hipLaunchKernelGGL(attn_probs_kernel<__bf16>, grid, dim3(256), 0, stream, kp);
    else hipLaunchKernelGGL(attn_probs_kernel<_Float16>, grid, dim3(256), 0, stream, kp);
    return (int)hipGetLastError();
}


}  // namespace fa
