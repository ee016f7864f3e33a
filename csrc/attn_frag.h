// Fragment helpers shared by the attention kernels that read a paged K cache [blocks, G, BS, dim] and a
// key-contiguous V cache [blocks, G, vdim, BS] straight into MFMA operands (attn_sigmoid.hip,
// attn_sink.hip): element traits of the two activation types and the S^T += K . Q^T step.
#pragma once
#include "common.h"

namespace {

template <typename T>
struct El;
template <>
struct El<bf16_t> {
  static constexpr int V = 8;  // elements per 16-byte fragment
  static LK_DEVICE float ld(const bf16_t* p) { return bf2f(*p); }
  static LK_DEVICE void st(bf16_t* p, float v) { *p = f2bf(v); }
};
template <>
struct El<float> {
  static constexpr int V = 4;
  static LK_DEVICE float ld(const float* p) { return *p; }
  static LK_DEVICE void st(float* p, float v) { *p = v; }
};

LK_DEVICE uint4_t ld16(const void* p) { return *reinterpret_cast<const uint4_t*>(p); }

// S^T += A(16 keys x one 16-byte fragment of dims) . B(the columns' same dims)
template <typename T>
LK_DEVICE floatx4 mma_qk(uint4_t a, uint4_t b, floatx4 c) {
  if constexpr (sizeof(T) == 2) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(short8, a), __builtin_bit_cast(short8, b), c, 0, 0, 0);
  } else {
    const floatx4 fa = __builtin_bit_cast(floatx4, a), fb = __builtin_bit_cast(floatx4, b);
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[e], fb[e], c, 0, 0, 0);
    return c;
  }
}

}  // namespace
