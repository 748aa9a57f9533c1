// Shared between the attention translation units.
#pragma once
#include "common.h"

namespace ah {

struct FlashArgs {
  const void *q, *k, *v;
  void *o;
  float *lse;
  const void *d_o;
  void *dq, *dk, *dv;
  float *delta;            // [B, H, T] rowsum(dO * O)
  int B, H, T;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, o_st;
  float scale, cap;
};


// attention_bf16.hip
int32_t flash_fwd_bf16(const FlashArgs &a, int head_dim);
int32_t flash_bwd_bf16(FlashArgs &a, int head_dim);

}  // namespace ah
