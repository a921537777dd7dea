// Backward kernels, one translation unit per (dtype, head-dim bucket): compiled with
// -DFA_T_BF16=0/1 -DFA_D=64/128/256.
#include "fa_bwd.h"
#include "fa_launch.h"

namespace fa {
#if FA_T_BF16
typedef __bf16 InstT;
#define FA_INST_NAME2(d) launch_bwd_bf16_##d
#else
typedef _Float16 InstT;
#define FA_INST_NAME2(d) launch_bwd_fp16_##d
#endif
#define FA_INST_NAME(d) FA_INST_NAME2(d)

// dQ pass then dK/dV pass on the same stream; both read softmax_d, which the caller's stream has
// already filled (launch_bwd_dot).
#ifndef FA_DQ_BN
#define FA_DQ_BN (FA_D > 64 ? 32 : 64)
#endif
// query rows per dK/dV step: with head dim 64 a 64-row step holds too few products to cover its fixed
// cost (tile requests, barrier), and the fp16 hand-over leaves room for 128 rows
#ifndef FA_BWD_BM
#define FA_BWD_BM (FA_D == 64 ? 128 : 64)
#endif
// DV: head dims the products run over (head dims up to 96 on the 128 bucket, up to 160 and up to 192 on the 256 bucket)
template <bool DROPOUT, int DV = FA_D>
static int run(const BwdKParams& kp, hipStream_t stream) {
#if FA_D <= 128
    // two workgroups (8 waves) per CU: the key tile is sized so that the kernel stays within 256 registers;
    // three at head dim 64 (168 registers), where the vector work per matrix instruction doubles -- without
    // dropout: the mask words do not fit in 168 registers (19 spilled, 7-15 % slower than two workgroups)
    if (int e = launch_bwd_dq<InstT, FA_D, FA_DQ_BN, (FA_D == 64 && !DROPOUT ? 3 : 2), DROPOUT, DV>(kp, stream)) return e;
    // Fewer key blocks than CUs (one long sequence on one or two kv heads, say): two workgroups per
    // key block, each accumulating half of the head dimension, fill the CUs at 3/4 of the work each.
    typedef BwdDkv3Cfg<InstT, FA_D, FA_BWD_BM, 1> C1;
    const int64_t key_blocks = (int64_t)((kp.p.seqlen_k + C1::BNW - 1) / C1::BNW) * kp.p.h_k * kp.p.b;
    if (key_blocks < 256 && kp.p.seqlen_q >= 1024) return launch_bwd_dkv3<InstT, FA_D, FA_BWD_BM, 2, DROPOUT>(kp, stream);
    return launch_bwd_dkv3<InstT, FA_D, FA_BWD_BM, 1, DROPOUT, DV>(kp, stream);
#else
    // Up to head dim 160 the dQ pass fits 256 registers with 32-key steps: two workgroups per CU, as at head dim 128
    // (d 160, bf16 causal 8k, 16 heads: backward 5.79 -> 5.07 ms against one workgroup with 64-key steps).  Beyond
    // that one workgroup (4 waves of 512 registers) per CU -- two spill 76 registers at 192 --; up to head dim 192
    // the registers also hold a 64-key step, which halves the barriers and tile requests per product (head dim 192,
    // causal 8k: dQ pass 7.28 -> 5.95 ms); at 256 a 64-key step spills and gains nothing.
    if constexpr (DV <= 160) {
        if (int e = launch_bwd_dq<InstT, FA_D, 32, 2, DROPOUT, DV>(kp, stream)) return e;
    } else {
        if (int e = launch_bwd_dq<InstT, FA_D, (DV <= 192 ? 64 : 32), 1, DROPOUT, DV>(kp, stream)) return e;
    }
    // Up to head dim 192 without dropout a wave holds its whole dK / dV accumulator (96 registers) next to its
    // resident key row; beyond that, or with the dropout mask words, two workgroups share a key block and each
    // accumulates half of the head dimension
    return launch_bwd_dkv3<InstT, FA_D, 32, (DV <= 192 && !DROPOUT ? 1 : 2), DROPOUT, DV>(kp, stream);
#endif
}

int FA_INST_NAME(FA_D)(const BwdKParams& kp, hipStream_t stream) {
    if (kp.p.p_dropout > 0.f) return run<true>(kp, stream);
#if FA_D == 128
    if (kp.p.d <= 96) return run<false, 96>(kp, stream);
#elif FA_D == 256
    if (kp.p.d <= 160) return run<false, 160>(kp, stream);
    if (kp.p.d <= 192) return run<false, 192>(kp, stream);
#endif
    return run<false>(kp, stream);
}

#if FA_D == 64
#if FA_T_BF16
int launch_bwd_dot_bf16(const BwdKParams& kp, hipStream_t stream) { return launch_bwd_dot<__bf16>(kp, stream); }
#else
int launch_bwd_dot_fp16(const BwdKParams& kp, hipStream_t stream) { return launch_bwd_dot<_Float16>(kp, stream); }
#endif
#endif
}  // namespace fa
