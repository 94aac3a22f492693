// MFMA fragments loaded straight from K-contiguous rows, for GEMM kernels whose operands are row-major (any K): lane l of
// a 16-row tile holds 16 bytes of row l % 16 at k-chunk l / 16. bf16 operands feed the 16x16x32 MFMA, fp32 operands four
// 16x16x4 MFMAs (products and sums in true 32-bit).
#pragma once
#include "common.h"

namespace dlia {

template <typename T>
__device__ __forceinline__ u32x4 load_frag(const T* __restrict__ row, int k, int K, bool valid, bool vec_ok) {
  constexpr int VEC = 16 / sizeof(T);
  u32x4 z = {0u, 0u, 0u, 0u};
  if (!valid || k >= K) return z;
  if (vec_ok) return ld16(row + k);
  T tmp[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) tmp[e] = (k + e < K) ? row[k + e] : (T)0.f;
  return *reinterpret_cast<u32x4*>(tmp);
}

__device__ __forceinline__ f32x4 mma_frag(bf16, u32x4 a, u32x4 b, f32x4 c) { return mfma16(a, b, c); }
__device__ __forceinline__ f32x4 mma_frag(float, u32x4 a, u32x4 b, f32x4 c) {
  const f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.x, bf.x, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.y, bf.y, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.z, bf.z, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.w, bf.w, c, 0, 0, 0);
  return c;
}

}  // namespace dlia
