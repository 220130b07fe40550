// Launch parameters shared by the attention kernels.
#pragma once
#include "common.h"

namespace flux {

struct AttnParams {
    const bf16_t* q; const bf16_t* k; const bf16_t* v; bf16_t* o; float* lse;
    int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl, o_sb, o_sh, o_sl;
    int H, L, n_qtiles, total_tiles;
    float scale_log2;  // sm_scale * log2(e)
    // 64-row-per-wave kernel only: query rows of a launch. (batch*head) pairs are taken two at a
    // time; the even one gets cnt_even tiles starting at row first_even, the odd one cnt_odd tiles
    // from first_odd.
    int cnt_even, cnt_odd, first_even, first_odd;
};

// Plain kernel for the head dims that the pipelined kernels do not cover (16, 32, 256).
void attn_launch_plain(const AttnParams& p, int64_t BH, int D, hipStream_t st);

}  // namespace flux
