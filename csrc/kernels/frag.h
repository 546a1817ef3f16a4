// MFMA operand fragments read straight from row-major global memory, for bf16 and for fp32 (true 32-bit products):
// shared by the general GEMM (gemm_rowmajor.hip) and the grouped expert GEMMs (moe.hip).  A lane (r = lane & 15,
// g = lane >> 4) holds PER consecutive k of row r; which k a (lane group, element) pair stands for only has to agree
// between the A and the B fragment, so both use k0 + PER g + j.
#pragma once
#include "common.h"

namespace dsse {
namespace {

template <typename T> struct Frag;
template <> struct Frag<bf16> {
  using V = bf16x8;
  static constexpr int PER = 8, KS = 32;
};
template <> struct Frag<float> {
  using V = f32x4;
  static constexpr int PER = 4, KS = 16;
};

template <typename T>
DEV typename Frag<T>::V load_frag(const T* row, int k, int K, bool valid, bool vec) {
  using F = Frag<T>;
  typename F::V v;
#pragma unroll
  for (int j = 0; j < F::PER; ++j) v[j] = (T)0.0f;
  if (!valid || k >= K) return v;
  if (vec && k + F::PER <= K) return ld_global<typename F::V>(row + k);
#pragma unroll
  for (int j = 0; j < F::PER; ++j)
    if (k + j < K) v[j] = row[k + j];
  return v;
}

DEV f32x4 mma(const bf16x8& a, const bf16x8& b, f32x4 c) { return mfma16x16x32(a, b, c); }
DEV f32x4 mma(const f32x4& a, const f32x4& b, f32x4 c) {
#pragma unroll
  for (int s = 0; s < 4; ++s) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], b[s], c, 0, 0, 0);
  return c;
}

DEV float gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

}  // namespace
}  // namespace dsse
