// One translation unit per (dtype, head-dim bucket): compiled with -DFA_T_BF16=0/1 -DFA_D=64/128/256.
#include "fa_prefill.h"
#include "fa_prefill_pp.h"
#include "fa_launch.h"

namespace fa {
#if FA_T_BF16
typedef __bf16 InstT;
#define FA_INST_NAME2(d) launch_prefill_bf16_##d
#else
typedef _Float16 InstT;
#define FA_INST_NAME2(d) launch_prefill_fp16_##d
#endif
#define FA_INST_NAME(d) FA_INST_NAME2(d)

int FA_INST_NAME(FA_D)(const KParams& kp, hipStream_t stream) {
    typedef PrefillTile<FA_D> Tile;
#if FA_D <= 128
#ifndef FA_PP_MIN_SQ
#define FA_PP_MIN_SQ (FA_D >= 128 ? 512 : 1024)     // measured cross-over against the 4-wave kernel
#endif
    // long query sequences: the 8-wave ping-pong kernel (256 rows per workgroup)
    if (kp.num_splits <= 1 && !kp.rotary_q && kp.p.seqlen_q >= FA_PP_MIN_SQ) {
        return launch_prefill_pp<InstT, FA_D, 64>(kp, stream);
    }
#endif
    return launch_prefill<InstT, FA_D, Tile::RB, Tile::BN, Tile::MINW>(kp, stream);
}
}  // namespace fa
