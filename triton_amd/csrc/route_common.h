// Wave-level pieces of the top-k router shared by the routing kernels and the single-launch decode layer:
// the order-preserving float key, DPP reductions and the k-round selection of one row spread over a wave.
#pragma once
#include "common.h"

namespace tk {
namespace {

__device__ inline uint32_t ordered_key(float v) {
  const uint32_t u = f32_bits(v);
  return u ^ ((u & 0x80000000u) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ inline float key_to_float(uint32_t k) {
  return bits_f32(k ^ ((k & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu));
}

// Orders this wave's LDS accesses: lanes exchange data through LDS without a workgroup barrier.
// LDS instructions of one wave are executed in program order, so a lane's read that follows another lane's write in
// the instruction stream sees it without any wait; all that is needed is that the compiler keeps the order.  (A
// wavefront-scope fence does that too but also waits for the wave's outstanding GLOBAL stores, the results of the row
// it has just finished: a full memory latency per row for nothing.)
__device__ __forceinline__ void wave_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  asm volatile("" ::: "memory");
}

// Wave-wide reductions with DPP lane exchanges (no LDS round trips): xor-1 and xor-2 inside a quad, mirror inside 8
// and inside 16 lanes leave every lane with its row's result; the four rows are combined through scalar reads.
// The result is uniform.  All 64 lanes must be active.
#define TK_DPP_QUAD_XOR1 0xB1      /* quad_perm [1,0,3,2] */
#define TK_DPP_QUAD_XOR2 0x4E      /* quad_perm [2,3,0,1] */
#define TK_DPP_ROW_HALF_MIRROR 0x141
#define TK_DPP_ROW_MIRROR 0x140

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  int x = (int)v;
#define TK_STEP(ctrl)                                                                  \
  {                                                                                    \
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, x, ctrl, 0xF, 0xF, false); \
    x = (int)(o > (uint32_t)x ? o : (uint32_t)x);                                      \
  }
  TK_STEP(TK_DPP_QUAD_XOR1)
  TK_STEP(TK_DPP_QUAD_XOR2)
  TK_STEP(TK_DPP_ROW_HALF_MIRROR)
  TK_STEP(TK_DPP_ROW_MIRROR)
#undef TK_STEP
  const uint32_t a = (uint32_t)__builtin_amdgcn_readlane(x, 0), b = (uint32_t)__builtin_amdgcn_readlane(x, 16);
  const uint32_t c = (uint32_t)__builtin_amdgcn_readlane(x, 32), d = (uint32_t)__builtin_amdgcn_readlane(x, 48);
  const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}

__device__ __forceinline__ float wave_sum_f32(float v) {
  int x = __builtin_bit_cast(int, v);
#define TK_STEP(ctrl) x = __builtin_bit_cast(int, __builtin_bit_cast(float, x) + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, x, ctrl, 0xF, 0xF, false)));
  TK_STEP(TK_DPP_QUAD_XOR1)
  TK_STEP(TK_DPP_QUAD_XOR2)
  TK_STEP(TK_DPP_ROW_HALF_MIRROR)
  TK_STEP(TK_DPP_ROW_MIRROR)
#undef TK_STEP
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 0)), b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 32)), d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 48));
  return (a + b) + (c + d);
}

// Inclusive prefix sum over the 64 lanes with DPP lane exchanges (no LDS round trips): four shifts inside the rows of 16,
// then the row totals are broadcast on.  All 64 lanes must be active.
__device__ __forceinline__ int wave_scan_i32(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, true);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, true);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, true);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, true);  // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return x;
}
// reductions inside a DPP row of 16 lanes (every lane of the row ends up with the row's result)
#define TK_ROW16(OP)                                                                                   \
  OP(TK_DPP_QUAD_XOR1) OP(TK_DPP_QUAD_XOR2) OP(TK_DPP_ROW_HALF_MIRROR) OP(TK_DPP_ROW_MIRROR)
__device__ __forceinline__ uint32_t row16_max_u32(uint32_t v) {
  int x = (int)v;
#define TK_STEP(ctrl)                                                                                   \
  {                                                                                                     \
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, x, ctrl, 0xF, 0xF, false);             \
    x = (int)(o > (uint32_t)x ? o : (uint32_t)x);                                                       \
  }
  TK_ROW16(TK_STEP)
#undef TK_STEP
  return (uint32_t)x;
}
__device__ __forceinline__ int row16_min_i32(int x) {
#define TK_STEP(ctrl)                                                                                   \
  {                                                                                                     \
    const int o = __builtin_amdgcn_update_dpp(0, x, ctrl, 0xF, 0xF, false);                            \
    x = o < x ? o : x;                                                                                  \
  }
  TK_ROW16(TK_STEP)
#undef TK_STEP
  return x;
}
__device__ __forceinline__ float row16_sum_f32(float v) {
  int x = __builtin_bit_cast(int, v);
#define TK_STEP(ctrl) x = __builtin_bit_cast(int, __builtin_bit_cast(float, x) + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, x, ctrl, 0xF, 0xF, false)));
  TK_ROW16(TK_STEP)
#undef TK_STEP
  return __builtin_bit_cast(float, x);
}


// Top-k of FOUR rows at a time in one wave: the sixteen lanes of a DPP row own one row of logits, lane l of the row the
// VPL consecutive experts l * VPL .. l * VPL + VPL - 1 as order-preserving keys (`retired` bit i: key[i] is out of the
// running, columns past E from the start).  A round = the row's largest key still in the running (in-lane maximum,
// then four DPP steps inside the row) and the LOWEST expert index holding it (the same again with a minimum): ties go
// to the lower expert, as the reference's packed sort key does (topk_details/_topk_forward.py:27-35,61).  Round j's
// winner lands in lane j & 15 of the row, slot j >> 4 (k <= 32); key0 = the first round's key (the row maximum).  No
// lane leaves its row, so the four rows cost what one costs.
template <int VPL>
__device__ __forceinline__ void row16_topk(const uint32_t (&key)[VPL], uint32_t retired, int k, int l16, uint32_t (&sel_key)[2],
                                           int (&sel_idx)[2], uint32_t& key0) {
  uint32_t ret = retired;
  for (int j = 0; j < k; ++j) {
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < VPL; ++i) m = (!((ret >> i) & 1u) && key[i] > m) ? key[i] : m;
    m = row16_max_u32(m);
    int idx = 0x7FFFFFFF;
#pragma unroll
    for (int i = VPL - 1; i >= 0; --i) idx = (!((ret >> i) & 1u) && key[i] == m) ? l16 * VPL + i : idx;
    idx = row16_min_i32(idx);
    const int mine = idx - l16 * VPL;
    if (mine >= 0 && mine < VPL) ret |= 1u << mine;
    if (j == 0) key0 = m;
    if ((j & 15) == l16) {
      sel_key[j >> 4] = m;
      sel_idx[j >> 4] = idx;
    }
  }
}

// Top-k of one row spread over a wave: lane l holds the order-preserving keys of experts l, l + 64, ... in hi[]
// (0 for columns past E).  Round j picks the largest key, ties to the lowest expert index (the reference packs
// E_pad - idx under the key for the same effect, topk_details/_topk_forward.py:27-35,61), hands it to lane j and
// retires it.  Same selection as a stable descending sort.
template <int EPL>
__device__ __forceinline__ void wave_topk(uint32_t (&hi)[EPL], int k, int E, int lane, float& myval, int& myidx) {
  uint32_t retired = 0;  // bit i: hi[i] is out of the running (columns past E from the start)
#pragma unroll
  for (int i = 0; i < EPL; ++i) retired |= (lane + 64 * i >= E ? 1u : 0u) << i;
  for (int j = 0; j < k; ++j) {
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < EPL; ++i) m = (!((retired >> i) & 1u) && hi[i] > m) ? hi[i] : m;
    m = wave_max_u32(m);
    int sel = -1;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const unsigned long long mask = __ballot(!((retired >> i) & 1u) && hi[i] == m);
      if (sel < 0 && mask != 0ull) sel = 64 * i + (int)__builtin_ctzll(mask);
    }
    if (sel >= 0 && lane == (sel & 63)) retired |= 1u << (sel >> 6);
    if (lane == j) {
      myval = key_to_float(m);
      myidx = sel;
    }
  }
}

}  // namespace
}  // namespace tk
