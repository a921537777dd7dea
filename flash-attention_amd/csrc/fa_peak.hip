// Matrix-pipe microbenchmark: what one MI355X sustains on v_mfma_f32_32x32x16_bf16 (or 16x16x32) alone.
//
// The published dense bf16 peak (2.5 PFLOP/s) is 256 CUs x 4 SIMDs x one 32x32x16 MFMA per 32 cycles at
// 2.4 GHz.  With every CU busy the part does not hold 2.4 GHz: the clock follows the switching activity
// of the operands, so the sustained rate depends on the DATA.  This kernel runs nothing but independent
// MFMAs (four waves per SIMD, four or eight accumulators in rotation, operands resident in registers) on operands
// that are either random bf16 values (sign, three exponents around 1, random mantissa) or zeros, and the
// benchmark reports both next to the attention kernels' rates.  The two instruction shapes differ: 16x16x32
// moves 4 accumulator registers per 16K flops where 32x32x16 moves 16 per 32K, and on random operands the part
// holds a higher clock with the small shape (2.12 against 1.85 PFLOP/s).  Beside it: the same for HBM reads and for LDS reads.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "fa_mi355x.h"

namespace fa {

typedef __attribute__((ext_vector_type(8))) __bf16 peak_bf16x8;
typedef __attribute__((ext_vector_type(16))) float peak_f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t peak_u32x4;

typedef __attribute__((ext_vector_type(4))) float peak_f32x4;

template <int SHAPE>        // 0: 32x32x16, 1: 16x16x32 (twice as many instructions for the same flops)
__global__ void __launch_bounds__(256) mfma_peak_kernel(float* sink, int iters, int random_operands) {
    peak_u32x4 a[4], b[4];
    uint32_t st = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            uint32_t va = 0, vb = 0;
            if (random_operands) {
                for (int hlf = 0; hlf < 2; hlf++) {   // bf16: sign, exponent 125..127, 7 random mantissa bits
                    st = st * 1664525u + 1013904223u;
                    const uint32_t r = st >> 8;
                    va |= (((r & 1u) << 15) | ((125u + (r >> 1) % 3u) << 7) | ((r >> 4) & 0x7fu)) << (16 * hlf);
                    st = st * 1664525u + 1013904223u;
                    const uint32_t q = st >> 8;
                    vb |= (((q & 1u) << 15) | ((118u + (q >> 1) % 3u) << 7) | ((q >> 4) & 0x7fu)) << (16 * hlf);
                }
            }
            a[i][e] = va;
            b[i][e] = vb;
        }
    float res = 0.f;
    if constexpr (SHAPE == 0) {
        peak_f32x16 acc[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < 16; j++)
                acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(peak_bf16x8, a[j & 3]),
                                                                     __builtin_bit_cast(peak_bf16x8, b[(j >> 2) & 3]), acc[j & 3], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) res += acc[i][0] + acc[i][9];
    } else {
        peak_f32x4 acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = (peak_f32x4){0.f, 0.f, 0.f, 0.f};
        // Written as assembly with the accumulators as in/out operands: left to the register allocator, the
        // builtin form of this loop rotates the eight accumulators through copies on every iteration, which costs
        // a third of the issue slots.  Eight instructions lie between two uses of one accumulator.
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < 32; j++)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[j & 7]) : "v"(a[j & 3]), "v"(b[(j >> 3) & 3]));
        }
#pragma unroll
        for (int i = 0; i < 8; i++) res += acc[i][0] + acc[i][3];
    }
    if (res == 1.2345e-30f) *sink = res;        // keeps the accumulators alive; never true in practice
}

// Memory microbenchmark: what a kernel that only reads sustains from HBM.  Every workgroup walks a contiguous
// share of the buffer, 4 KB per step and kHbmPeakUnroll steps in flight per lane, with ordinary or non-temporal
// loads; nothing is written.
constexpr int kHbmPeakUnroll = 8;
#ifndef FA_HBM_PEAK_GRID
#define FA_HBM_PEAK_GRID 16384           // measured best of 1024 .. 16384 (7.13 TB/s non-temporal, 6.31 ordinary)
#endif
template <bool NT>
__global__ void __launch_bounds__(256) hbm_read_peak_kernel(const peak_u32x4* __restrict__ src, int64_t n16, uint32_t* sink) {
    const int64_t per_block = ((n16 + gridDim.x - 1) / gridDim.x + 255) / 256 * 256;
    const int64_t lo = (int64_t)blockIdx.x * per_block;
    const int64_t hi = lo + per_block < n16 ? lo + per_block : n16;
    peak_u32x4 acc = {0, 0, 0, 0};
    for (int64_t i = lo + threadIdx.x; i < hi; i += kHbmPeakUnroll * 256) {
        peak_u32x4 v[kHbmPeakUnroll];
#pragma unroll
        for (int u = 0; u < kHbmPeakUnroll; u++) {
            const int64_t j = i + u * 256;
            const peak_u32x4 z = {0, 0, 0, 0};
            if (j < hi) v[u] = NT ? __builtin_nontemporal_load(src + j) : src[j];
            else v[u] = z;
        }
#pragma unroll
        for (int u = 0; u < kHbmPeakUnroll; u++) acc ^= v[u];
    }
    const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (r == 0x9e3779b9u && n16 < 0) *sink = r;      // keeps the loads alive; never true
}

// LDS microbenchmark: what the LDS of a CU delivers to ds_read_b128 (one 1 KB operand fragment per wave
// instruction, the access the attention kernels feed their matrix instructions with).  One workgroup per CU,
// `waves` waves each reading its own conflict-free 16 KB window over and over; cycles[workgroup] receives the
// shader-clock cycles the workgroup's loop took.
__global__ void __launch_bounds__(1024) lds_read_peak_kernel(uint64_t* cycles, uint32_t* sink, int iters) {
    __shared__ __attribute__((aligned(16))) char window[65536];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < 65536 / 4; i += blockDim.x) reinterpret_cast<uint32_t*>(window)[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    const char* base = window + (wave & 3) * 16384 + lane * 16;
    peak_u32x4 acc = {0, 0, 0, 0};
    const uint64_t t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 16; u++) acc ^= *reinterpret_cast<const peak_u32x4*>(base + u * 1024);
        asm volatile("" : "+v"(acc));
    }
    const uint64_t t1 = __builtin_readcyclecounter();
    if (tid == 0) cycles[blockIdx.x] = t1 - t0;
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u && iters < 0) *sink = acc[0];     // never true
}

}  // namespace fa

extern "C" int fa_lds_read_peak(uint64_t* cycles, int32_t workgroups, int32_t waves, int32_t iters, int64_t* bytes_per_workgroup,
                                void* sink, void* hip_stream) {
    if (!cycles || !sink || !bytes_per_workgroup || workgroups <= 0 || waves <= 0 || waves > 16 || iters <= 0) return 1;
    hipLaunchKernelGGL(fa::lds_read_peak_kernel, dim3(workgroups), dim3(64 * waves), 0, (hipStream_t)hip_stream, cycles,
                       reinterpret_cast<uint32_t*>(sink), iters);
    *bytes_per_workgroup = (int64_t)waves * iters * 16 * 1024;
    return (int)hipGetLastError();
}

extern "C" int fa_hbm_read_peak(const void* src, int64_t bytes, int32_t nontemporal, void* sink, void* hip_stream) {
    if (!src || !sink || bytes < 16 || ((uintptr_t)src & 15) != 0) return 1;
    const int64_t n16 = bytes / 16;
    const dim3 grid(FA_HBM_PEAK_GRID), block(256);
    if (nontemporal)
        hipLaunchKernelGGL(fa::hbm_read_peak_kernel<true>, grid, block, 0, (hipStream_t)hip_stream,
                           reinterpret_cast<const fa::peak_u32x4*>(src), n16, reinterpret_cast<uint32_t*>(sink));
    else
        hipLaunchKernelGGL(fa::hbm_read_peak_kernel<false>, grid, block, 0, (hipStream_t)hip_stream,
                           reinterpret_cast<const fa::peak_u32x4*>(src), n16, reinterpret_cast<uint32_t*>(sink));
    return (int)hipGetLastError();
}

extern "C" int fa_mfma_peak_shape(float* sink, int32_t iters, int32_t random_operands, int32_t shape, int64_t* flops, void* hip_stream) {
    if (!sink || iters <= 0 || !flops || (shape != 0 && shape != 1)) return 1;
    const int grid = 1024;                      // four workgroups of 4 waves per CU: every SIMD holds 4 waves
    if (shape == 0) hipLaunchKernelGGL(fa::mfma_peak_kernel<0>, dim3(grid), dim3(256), 0, (hipStream_t)hip_stream, sink, iters, random_operands);
    else hipLaunchKernelGGL(fa::mfma_peak_kernel<1>, dim3(grid), dim3(256), 0, (hipStream_t)hip_stream, sink, iters, random_operands);
    *flops = (int64_t)grid * 4 * iters * 16 * 32768LL;      // 16 x 32x32x16 or 32 x 16x16x32 per iteration
    return (int)hipGetLastError();
}
extern "C" int fa_mfma_peak(float* sink, int32_t iters, int32_t random_operands, int64_t* flops, void* hip_stream) {
    return fa_mfma_peak_shape(sink, iters, random_operands, 0, flops, hip_stream);
}
