// One translation unit per (dtype, head-dim bucket): compiled with -DFA_T_BF16=0/1 -DFA_D=64/128/256.
#include "fa_prefill.h"
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
    return launch_prefill<InstT, FA_D, Tile::RB, Tile::BN, Tile::MINW>(kp, stream);
}
}  // namespace fa
