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
