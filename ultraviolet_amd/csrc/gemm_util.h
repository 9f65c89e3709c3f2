// Helpers shared by the GEMM kernels (gfx950): MFMA wrappers on 16-byte operand words and rounding / packing to the
// activation type.
#pragma once
#include "common.h"

namespace uvmi {

typedef _Float16 gh8 __attribute__((ext_vector_type(8)));
typedef __bf16 gb8 __attribute__((ext_vector_type(8)));
typedef float gf4 __attribute__((ext_vector_type(4)));
typedef unsigned int gu4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ gf4 gmfma(gu4 a, gu4 b, gf4 c) {
  if constexpr (DT == UVMI_F16) {
    gh8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, c, 0, 0, 0);
  } else {
    gb8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, c, 0, 0, 0);
  }
}

template <int DT> __device__ __forceinline__ float ground(float v) {
  if constexpr (DT == UVMI_F16) return (float)(half_t)v;
  else return bf16_to_float(float_to_bf16(v));
}
// silu(g) rounded to the activation type, for a g already on that type's grid.  bf16 divides through the hardware reciprocal
// (1 ulp in fp32, ahead of a rounding to 8 bits), as the standalone SwiGLU kernel does: a full IEEE division is ten
// instructions per element of the gate-up epilogue.
template <int DT> __device__ __forceinline__ float silu_round(float gv) {
  if constexpr (DT == UVMI_BF16) return ground<DT>(gv * __builtin_amdgcn_rcpf(1.0f + __expf(-gv)));
  else return ground<DT>(gv / (1.0f + __expf(-gv)));
}
template <int DT> __device__ __forceinline__ uint32_t gpack(float a, float b) {
  const uint32_t lo = DT == UVMI_BF16 ? float_to_bf16(a) : float_to_half_bits(a);
  const uint32_t hi = DT == UVMI_BF16 ? float_to_bf16(b) : float_to_half_bits(b);
  return lo | (hi << 16);
}

}  // namespace uvmi
