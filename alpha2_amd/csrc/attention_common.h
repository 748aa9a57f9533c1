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
  int hd;                  // head size of the tensors; the kernels' D is the next of {32, 64, 128}, features hd .. D - 1 read as zero and are not stored
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, o_st;
  float scale, cap;
  int variant;             // AhFlash::bwd_variant
};

// Which (batch x head, block along the sequence) this workgroup works on.  Workgroups are dealt to the 8 XCDs round-robin
// in launch order (x fastest), and each XCD has its own L2: with the natural mapping the 8 blocks of one head land on 8
// different XCDs and each of them fetches that head's K and V (or Q and dO) from HBM again.  Instead XCD x takes the heads
// congruent to x mod 8, so a head's operands are fetched once.
// Causal blocks differ in length by a factor of the block count, and a CU takes the next workgroup in launch order as soon
// as one of its own ends.  Head by head (long block first within each head) the longest block of the LAST head starts
// when nearly everything else is done, and the launch ends with most CUs idle: 18 units of time for 13.5 units of work per
// slot at 24 heads x 8 blocks on an XCD's 64 slots.  So an XCD takes its heads a group at a time and, within such a
// group, all the longest blocks first, then all the second longest, ...: the launch ends on the shortest blocks (14 units
// in the same example).  A group is as many heads as have 6 MB of K and V between them (measured at head size 64: all 24
// heads of an XCD at T = 1024, 12 at T = 2048; a block reads only the keys up to its own position, so more than the 4 MB of
// an XCD's L2 is still served from it).
__device__ __forceinline__ int flash_head_group(int T, int head_dim, int esize) {
  const int64_t per_head = (int64_t)2 * T * head_dim * esize;
  const int64_t g = ((int64_t)6 << 20) / per_head;
  return g < 1 ? 1 : (g > 65535 ? 65535 : (int)g);
}
__device__ __forceinline__ void flash_block(int &bh, int &xblk, int group_heads) {
  const int nx = gridDim.x, lin = blockIdx.y * nx + blockIdx.x;
  const int per_xcd = gridDim.y >> 3;                              // heads each XCD takes
  if (lin < nx * per_xcd * 8) {                                    // (heads past the last multiple of 8 keep the natural mapping)
    const int xcd = lin & 7, slot = lin >> 3;
    const int group = slot / (nx * group_heads), first = group * group_heads;
    const int heads = min(group_heads, per_xcd - first), r = slot - first * nx;
    xblk = r / heads;
    bh = (first + r % heads) * 8 + xcd;
  } else {
    bh = blockIdx.y;
    xblk = blockIdx.x;
  }
}


// attention_bf16.hip
int32_t flash_fwd_bf16(const FlashArgs &a, int head_dim);
int32_t flash_bwd_bf16(FlashArgs &a, int head_dim);

}  // namespace ah
