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

// Which (batch x head, block along the sequence) this workgroup works on.  Workgroups are dealt to the 8 XCDs round-robin
// in launch order (x fastest), and each XCD has its own L2: with the natural mapping the 8 blocks of one head land on 8
// different XCDs and each of them fetches that head's K and V (or Q and dO) from HBM again.  Instead XCD x takes the heads
// congruent to x mod 8 and runs all blocks of a head back to back, so a head's operands are fetched once.
__device__ __forceinline__ void flash_block(int &bh, int &xblk) {
  const int nx = gridDim.x, lin = blockIdx.y * nx + blockIdx.x;
  if (lin < nx * (int)(gridDim.y & ~7u)) {                         // (heads past the last multiple of 8 keep the natural mapping)
    const int xcd = lin & 7, slot = lin >> 3;
    bh = (slot / nx) * 8 + xcd;
    xblk = slot % nx;
  } else {
    bh = blockIdx.y;
    xblk = blockIdx.x;
  }
}


// attention_bf16.hip
int32_t flash_fwd_bf16(const FlashArgs &a, int head_dim);
int32_t flash_bwd_bf16(FlashArgs &a, int head_dim);

}  // namespace ah
