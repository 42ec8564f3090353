// 64-lane wavefront primitives for gfx950, built on DPP lane moves (no LDS traffic).
//
// These replace the block-wide scan / reduce collectives the reference takes from CUB
// (BlockScan::ExclusiveScan with a reduce-by-key functor,
// cuda_template/reducer/merged_agent_spmv_template.cuh:33-54,272; BlockReduce::Sum,
// codegen/merged_gen_gpu.py:320-322).  A wavefront here is 64 lanes = 4 DPP rows of 16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace flex {

constexpr int WAVE = 64;

// DPP controls (GCN3/CDNA encoding).
constexpr int DPP_ROW_SHR1 = 0x111, DPP_ROW_SHR2 = 0x112, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHR8 = 0x118;
constexpr int DPP_WAVE_SHR1 = 0x138;
constexpr int DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;

// Move a 32-bit lane value through DPP; lanes without a source keep `old`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_i32(int old, int src) {
  return __builtin_amdgcn_update_dpp(old, src, CTRL, ROW_MASK, 0xf, false);
}

// Typed DPP move for 4- and 8-byte values (8-byte values move as two halves).
template <int CTRL, int ROW_MASK, typename T>
__device__ __forceinline__ T dpp_move(T old, T src) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "DPP moves 32-bit registers");
  if constexpr (sizeof(T) == 4) {
    int r = dpp_i32<CTRL, ROW_MASK>(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src));
    return __builtin_bit_cast(T, r);
  } else {
    uint64_t o = __builtin_bit_cast(uint64_t, old), s = __builtin_bit_cast(uint64_t, src);
    uint32_t lo = (uint32_t)dpp_i32<CTRL, ROW_MASK>((int)(uint32_t)o, (int)(uint32_t)s);
    uint32_t hi = (uint32_t)dpp_i32<CTRL, ROW_MASK>((int)(uint32_t)(o >> 32), (int)(uint32_t)(s >> 32));
    return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
  }
}

// One Hillis-Steele step of an inclusive segmented sum.  `key` is non-decreasing across lanes; a lane
// adds its source lane's running value only when both carry the same key.  Lanes with no source lane
// (or masked rows) receive key -2 from the move and therefore add nothing.
template <int CTRL, int ROW_MASK, typename V, int W>
__device__ __forceinline__ void seg_step(int key, V (&val)[W]) {
  const int src_key = dpp_i32<CTRL, ROW_MASK>(-2, key);
  const bool take = (src_key == key);
#pragma unroll
  for (int i = 0; i < W; ++i) {
    const V moved = dpp_move<CTRL, ROW_MASK>(V(0), val[i]);
    val[i] = take ? static_cast<V>(val[i] + moved) : val[i];
  }
}

// Inclusive segmented sum over the 64 lanes of a wavefront: afterwards val[] of lane l holds the sum
// over the maximal run of lanes <= l that share lane l's key.  Keys must be >= -1.
template <typename V, int W>
__device__ __forceinline__ void wave_segmented_inclusive_sum(int key, V (&val)[W]) {
  seg_step<DPP_ROW_SHR1, 0xf>(key, val);
  seg_step<DPP_ROW_SHR2, 0xf>(key, val);
  seg_step<DPP_ROW_SHR4, 0xf>(key, val);
  seg_step<DPP_ROW_SHR8, 0xf>(key, val);
  seg_step<DPP_ROW_BCAST15, 0xa>(key, val);  // lane 15 / 47 -> rows 1 / 3
  seg_step<DPP_ROW_BCAST31, 0xc>(key, val);  // lane 31 -> rows 2 and 3
}

// Shift a value one lane up the wavefront; lane 0 receives `fill`.
template <typename T>
__device__ __forceinline__ T wave_shift_up1(T v, T fill) {
  return dpp_move<DPP_WAVE_SHR1, 0xf>(fill, v);
}

// Sum over the 64 lanes; the total is valid in lane 63.
template <typename V, int W>
__device__ __forceinline__ void wave_sum_to_last_lane(V (&val)[W]) {
  wave_segmented_inclusive_sum<V, W>(0, val);
}

__device__ __forceinline__ int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

}  // namespace flex
