// One translation unit per (dtype, head-dim bucket): compiled with -DFA_T_BF16=0/1 -DFA_D=64/128/256.
#include "fa_prefill.h"
#include "fa_prefill_pp16.h"
#include "fa_prefill_il.h"
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
    // Long query sequences (measured cross-overs on MI355X):
    //  * head dim 128, from 2048 keys on (causal / windowed) or beyond 768 (full): the 8-wave ping-pong
    //    kernel, 256 rows per workgroup, each K/V tile fetched once per 256 rows;
    //  * otherwise (from prefill_long_rows query rows on): the software-pipelined kernel, two independent
    //    128-row workgroups per CU, whose start-up and output phases overlap.
    // Shorter sequences, split key ranges, q rotary and rows that stand for (position, grouped head) pairs take
    // the general 4-wave kernel.
    if (kp.num_splits <= 1 && !kp.rotary_q && kp.p.seqlen_q >= prefill_long_rows(FA_D) && kp.pack_g <= 1) {
        const bool masked = kp.has_right || kp.has_left;
        const bool long_keys = kp.p.seqlen_k >= (masked ? 2048 : 769);
        // When the 256-row blocks of the ping-pong kernel would occupy no more than half of the 256
        // CUs (a chunk of 1024 queries of one sequence with 32 heads: 128 blocks), the 128-row blocks
        // of the pipelined kernel fill them: measured +12..25 % at 128 blocks, -11 % at 192.  Under a mask up to
        // 256 blocks: one 256-row block per CU leaves every CU waiting for the one with the heaviest block
        // (causal 2k-8k at exactly 256 blocks: +4..12 %; 384 blocks: -2 %; without a mask the ping-pong kernel
        // stays 10-14 % ahead at 256).
        const int64_t pp_wgs = (int64_t)((kp.p.seqlen_q + 255) / 256) * kp.p.h * kp.p.b;
        // A window that spans few keys (left + right bound up to 768): a 256-row block visits the keys of its first
        // and of its last row, (256 + span) / 64 tiles for 256 rows against (128 + span) / 64 for 128; the 128-row
        // kernel then does less masked-out work (span 128: +16-35 %, 256: +13-18 %, 512: +3-10 %, 1024: -2 %).
        const bool narrow = kp.has_left && kp.has_right && (int64_t)kp.p.window_left + kp.p.window_right <= 768;
        if (FA_D >= 128 && long_keys && (narrow || pp_wgs <= (masked ? 256 : 128))) return launch_prefill_il<InstT, FA_D, 64>(kp, stream);
        if constexpr (FA_D >= 128) {
            if (long_keys) return launch_prefill_pp<InstT, FA_D, 64>(kp, stream);
        }
        return launch_prefill_il<InstT, FA_D, 64>(kp, stream);
    }
#else
    // head dim 129..256: the 8-wave ping-pong kernel with 16 query rows per wave (fa_prefill_pp16.h), or, with dropout,
    // pairs of waves that split the head dim (fa_prefill_il.h)
    if (kp.num_splits <= 1 && !kp.rotary_q && kp.p.seqlen_q >= prefill_long_rows(FA_D) && kp.pack_g <= 1) {
        if (kp.p.p_dropout > 0.f) return launch_prefill_il_256<InstT>(kp, stream);
        return launch_prefill_pp_wide<InstT>(kp, stream);
    }
#endif
    return launch_prefill<InstT, FA_D, Tile::RB, Tile::BN, Tile::MINW>(kp, stream);
}
}  // namespace fa
