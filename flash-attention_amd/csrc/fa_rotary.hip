// Standalone rotary embedding for gfx950: out[..., :rd] = x * cos + rotate_half(x) * sin on the first
// rotary_dim columns of every (token, head) row, the remaining columns copied through.  Replaces the
// reference's Triton kernel (flash_attn/ops/triton/rotary.py:15-240) behind apply_rotary_emb
// (flash_attn/layers/rotary.py:34-124).  HBM-bound: every element of x is read once and written
// once with 16-byte accesses; a work item owns both members of each rotated pair, so the operation
// is safe in place.  With `conjugate` the rotation is inverted (sin -> -sin): that is the backward
// of the operation.
#include "fa_common.h"
#include "fa_launch.h"

namespace fa {

// x and out of a problem that does not fit the 256 MB memory-side cache are moved with non-temporal accesses
// (+6-8 % on 0.5 GB in place: nothing is used twice, so nothing should displace what the other CUs wait for);
// smaller problems keep ordinary accesses, which are up to 1.5 x faster there.
template <bool STREAM> FA_DEV u32x4 ld_x16(const void* p) {
    if constexpr (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    else return ld_global16(p);
}
template <bool STREAM> FA_DEV void st_x16(void* p, u32x4 v) {
    if constexpr (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
    else st_global16(p, v);
}
constexpr int64_t kRotaryStreamBytes = (int64_t)384 << 20;

// N consecutive table values starting at element i (i a multiple of N, rows 16-byte aligned), as fp32
template <typename CS, int N> FA_DEV void cs_load(const void* base, int64_t i, bool valid, float fill, float* out) {
    if (!valid) {
#pragma unroll
        for (int e = 0; e < N; e++) out[e] = fill;
        return;
    }
    const CS* p = reinterpret_cast<const CS*>(base) + i;
    if constexpr (sizeof(CS) == 4) {
#pragma unroll
        for (int q = 0; q < N / 4; q++) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(p + 4 * q);
#pragma unroll
            for (int e = 0; e < 4; e++) out[4 * q + e] = v[e];
        }
    } else if constexpr (N == 8) {
        unpack8<CS>(ld_global16(p), out);
    } else {
        typedef typename Elem<CS>::v4 v4;
        const v4 v = *reinterpret_cast<const v4*>(p);
#pragma unroll
        for (int e = 0; e < 4; e++) out[e] = (float)v[e];
    }
}

// One work item = one 16-byte granule of a (token, head) row together with its rotation partner.
// I is the index type of the flattened (batch, token, head, granule) space: 32-bit when it fits.
template <typename T, typename CS, typename I, bool STREAM>
__global__ void __launch_bounds__(256) rotary_kernel(const fa_rotary_params p) {
    const int rd = p.rotary_dim;
    const bool inplace = p.out == p.x;
    const int rot_chunks = p.interleaved ? rd / 8 : rd / 16;        // work items that rotate
    const int pass_chunks = inplace ? 0 : (p.d - rd) / 8;           // work items that copy through
    const I ch = (I)(rot_chunks + pass_chunks);
    const I total = (I)p.b * (I)p.seqlen * (I)p.h * ch;
    const I stride = (I)gridDim.x * (I)blockDim.x;
    const float sign = p.conjugate ? -1.f : 1.f;
    for (I idx = (I)blockIdx.x * (I)blockDim.x + (I)threadIdx.x; idx < total; idx += stride) {
        const int c = (int)(idx % ch);
        I r = idx / ch;
        const int head = (int)(r % (I)p.h); r /= (I)p.h;
        const int t = (int)(r % (I)p.seqlen);
        const int b = (int)(r / (I)p.seqlen);
        int64_t xrow, orow;
        if (p.cu_seqlens) {
            const int s0 = p.cu_seqlens[b];
            if (t >= p.cu_seqlens[b + 1] - s0) continue;
            xrow = (int64_t)(s0 + t) * p.x_row_stride;
            orow = (int64_t)(s0 + t) * p.o_row_stride;
        } else {
            xrow = (int64_t)b * p.x_batch_stride + (int64_t)t * p.x_row_stride;
            orow = (int64_t)b * p.o_batch_stride + (int64_t)t * p.o_row_stride;
        }
        const T* x = reinterpret_cast<const T*>(p.x) + xrow + (int64_t)head * p.x_head_stride;
        T* o = reinterpret_cast<T*>(p.out) + orow + (int64_t)head * p.o_head_stride;
        if (c >= rot_chunks) {                                       // columns past rotary_dim
            const int d0 = rd + (c - rot_chunks) * 8;
            st_x16<STREAM>(o + d0, ld_x16<STREAM>(x + d0));
            continue;
        }
        const int pos = t + (p.seqlen_offsets ? p.seqlen_offsets[b] : p.seqlen_offset);
        const bool in_table = pos >= 0 && pos < p.seqlen_ro;        // past the table: identity
        const int64_t crow = (int64_t)pos * p.cs_row_stride;
        if (p.interleaved) {
            // pairs (2i, 2i+1): 8 consecutive columns = 4 pairs, table columns [4c, 4c+4)
            float v[8], cs[4], sn[4];
            unpack8<T>(ld_x16<STREAM>(x + c * 8), v);
            cs_load<CS, 4>(p.cos, crow + c * 4, in_table, 1.f, cs);
            cs_load<CS, 4>(p.sin, crow + c * 4, in_table, 0.f, sn);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float x0 = v[2 * e], x1 = v[2 * e + 1], s_ = sign * sn[e];
                v[2 * e] = x0 * cs[e] - x1 * s_;
                v[2 * e + 1] = x0 * s_ + x1 * cs[e];
            }
            st_x16<STREAM>(o + c * 8, pack8<T>(v));
        } else {
            // pairs (i, i + rd/2): columns [8c, 8c+8) with [rd/2 + 8c, +8), table columns [8c, 8c+8)
            float a[8], bb[8], cs[8], sn[8];
            unpack8<T>(ld_x16<STREAM>(x + c * 8), a);
            unpack8<T>(ld_x16<STREAM>(x + rd / 2 + c * 8), bb);
            cs_load<CS, 8>(p.cos, crow + c * 8, in_table, 1.f, cs);
            cs_load<CS, 8>(p.sin, crow + c * 8, in_table, 0.f, sn);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float x0 = a[e], x1 = bb[e], s_ = sign * sn[e];
                a[e] = x0 * cs[e] - x1 * s_;
                bb[e] = x0 * s_ + x1 * cs[e];
            }
            st_x16<STREAM>(o + c * 8, pack8<T>(a));
            st_x16<STREAM>(o + rd / 2 + c * 8, pack8<T>(bb));
        }
    }
}

// The general form, for what the granule form cannot address: any even rotary_dim, any head dim, any strides and
// alignment (the reference's kernel masks its loads instead, flash_attn/ops/triton/rotary.py:81-104).  One work
// item = one rotated pair, or one column past rotary_dim; 2-byte accesses, so far from the memory roofline, which
// is why the granule form takes everything it can.  A work item reads both members of its pair before it writes
// them: safe in place.
template <typename T, typename CS>
__global__ void __launch_bounds__(256) rotary_general_kernel(const fa_rotary_params p) {
    const int rd = p.rotary_dim, half = rd / 2;
    const bool inplace = p.out == p.x;
    const int64_t per_row = half + (inplace ? 0 : p.d - rd);
    const int64_t total = (int64_t)p.b * p.seqlen * p.h * per_row;
    const float sign = p.conjugate ? -1.f : 1.f;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(idx % per_row);
        int64_t r = idx / per_row;
        const int head = (int)(r % p.h); r /= p.h;
        const int t = (int)(r % p.seqlen);
        const int b = (int)(r / p.seqlen);
        int64_t xrow, orow;
        if (p.cu_seqlens) {
            const int s0 = p.cu_seqlens[b];
            if (t >= p.cu_seqlens[b + 1] - s0) continue;
            xrow = (int64_t)(s0 + t) * p.x_row_stride;
            orow = (int64_t)(s0 + t) * p.o_row_stride;
        } else {
            xrow = (int64_t)b * p.x_batch_stride + (int64_t)t * p.x_row_stride;
            orow = (int64_t)b * p.o_batch_stride + (int64_t)t * p.o_row_stride;
        }
        const T* x = reinterpret_cast<const T*>(p.x) + xrow + (int64_t)head * p.x_head_stride;
        T* o = reinterpret_cast<T*>(p.out) + orow + (int64_t)head * p.o_head_stride;
        if (c >= half) {                                             // columns past rotary_dim
            o[rd + (c - half)] = x[rd + (c - half)];
            continue;
        }
        const int i0 = p.interleaved ? 2 * c : c, i1 = p.interleaved ? 2 * c + 1 : c + half;
        const int pos = t + (p.seqlen_offsets ? p.seqlen_offsets[b] : p.seqlen_offset);
        float cs = 1.f, sn = 0.f;
        if (pos >= 0 && pos < p.seqlen_ro) {                         // past the table: identity
            cs = (float)reinterpret_cast<const CS*>(p.cos)[(int64_t)pos * p.cs_row_stride + c];
            sn = sign * (float)reinterpret_cast<const CS*>(p.sin)[(int64_t)pos * p.cs_row_stride + c];
        }
        const float x0 = (float)x[i0], x1 = (float)x[i1];
        o[i0] = (T)(x0 * cs - x1 * sn);
        o[i1] = (T)(x0 * sn + x1 * cs);
    }
}

template <typename T>
static int launch_rotary_general(const fa_rotary_params& p, hipStream_t stream) {
    const int64_t per_row = p.rotary_dim / 2 + (p.out == p.x ? 0 : p.d - p.rotary_dim);
    const int64_t total = (int64_t)p.b * p.seqlen * p.h * per_row;
    if (total <= 0) return 0;
    const dim3 grid((unsigned)std::min<int64_t>((total + 255) / 256, 256 * 32)), block(256);
    switch (p.cs_dtype) {
        case FA_DTYPE_FP16: hipLaunchKernelGGL((rotary_general_kernel<T, _Float16>), grid, block, 0, stream, p); break;
        case FA_DTYPE_BF16: hipLaunchKernelGGL((rotary_general_kernel<T, __bf16>), grid, block, 0, stream, p); break;
        default: hipLaunchKernelGGL((rotary_general_kernel<T, float>), grid, block, 0, stream, p); break;
    }
    return (int)hipGetLastError();
}

template <typename T, typename I, bool STREAM>
static void launch_rotary_is(const fa_rotary_params& p, dim3 grid, hipStream_t stream) {
    const dim3 block(256);
    switch (p.cs_dtype) {
        case FA_DTYPE_FP16: hipLaunchKernelGGL((rotary_kernel<T, _Float16, I, STREAM>), grid, block, 0, stream, p); break;
        case FA_DTYPE_BF16: hipLaunchKernelGGL((rotary_kernel<T, __bf16, I, STREAM>), grid, block, 0, stream, p); break;
        default: hipLaunchKernelGGL((rotary_kernel<T, float, I, STREAM>), grid, block, 0, stream, p); break;
    }
}
template <typename T, typename I>
static void launch_rotary_i(const fa_rotary_params& p, dim3 grid, hipStream_t stream) {
    // bytes of x (and of out, when it is another tensor) the launch walks; packed input: at most this
    const int64_t bytes = (int64_t)p.b * p.seqlen * p.h * p.d * (int64_t)sizeof(T) * (p.out == p.x ? 1 : 2);
    if (bytes >= kRotaryStreamBytes) launch_rotary_is<T, I, true>(p, grid, stream);
    else launch_rotary_is<T, I, false>(p, grid, stream);
}

template <typename T>
static int launch_rotary_t(const fa_rotary_params& p, hipStream_t stream) {
    const bool inplace = p.out == p.x;
    const int ch = (p.interleaved ? p.rotary_dim / 8 : p.rotary_dim / 16) + (inplace ? 0 : (p.d - p.rotary_dim) / 8);
    const int64_t total = (int64_t)p.b * p.seqlen * p.h * ch;
    if (total <= 0) return 0;
    // grid-stride: enough workgroups to keep every CU's wave slots full, each lane then walks the rest
    const int64_t blocks = std::min<int64_t>((total + 255) / 256, 256 * 32);
    const dim3 grid((unsigned)blocks);
    if (total + (int64_t)blocks * 256 < (int64_t)1 << 32) launch_rotary_i<T, uint32_t>(p, grid, stream);
    else launch_rotary_i<T, int64_t>(p, grid, stream);
    return (int)hipGetLastError();
}

// every access of the granule form is a 16-byte piece of a row (8 bytes for the tables of the interleaved form)
static bool rotary_granules_apply(const fa_rotary_params& p) {
    if (p.d % 8 != 0 || p.rotary_dim % 16 != 0) return false;
    const int64_t strides[] = {p.x_batch_stride, p.x_row_stride, p.x_head_stride, p.o_batch_stride,
                               p.o_row_stride, p.o_head_stride, p.cs_row_stride};
    for (int64_t s : strides) if (s % 8 != 0) return false;
    const void* ptrs[] = {p.x, p.out, p.cos, p.sin};
    for (const void* q : ptrs) if ((uintptr_t)q % 16 != 0) return false;
    return true;
}

int launch_rotary(const fa_rotary_params& p, hipStream_t stream) {
    if (!rotary_granules_apply(p))
        return p.dtype == FA_DTYPE_BF16 ? launch_rotary_general<__bf16>(p, stream) : launch_rotary_general<_Float16>(p, stream);
    return p.dtype == FA_DTYPE_BF16 ? launch_rotary_t<__bf16>(p, stream) : launch_rotary_t<_Float16>(p, stream);
}

}  // namespace fa
