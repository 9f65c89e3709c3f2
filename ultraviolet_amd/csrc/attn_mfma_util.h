// Operand types and small helpers shared by the packed-attention MFMA kernels (forward and backward).
#pragma once
#include "common.h"

namespace uvmi {

typedef _Float16 ph8 __attribute__((ext_vector_type(8)));
typedef _Float16 ph2 __attribute__((ext_vector_type(2)));
typedef __bf16 pb8 __attribute__((ext_vector_type(8)));
typedef __bf16 pb2 __attribute__((ext_vector_type(2)));
typedef float pf4 __attribute__((ext_vector_type(4)));
typedef unsigned int pu4 __attribute__((ext_vector_type(4)));
typedef unsigned int pu2 __attribute__((ext_vector_type(2)));

template <int DT>
__device__ __forceinline__ pf4 mfma16(pu4 a, pu4 b, pf4 c) {
  if constexpr (DT == UVMI_F16) {
    ph8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, c, 0, 0, 0);
  } else {
    pb8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, c, 0, 0, 0);
  }
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {  // two fp32 -> one dword of 16-bit values, round to nearest even
  uint32_t r;
  if constexpr (DT == UVMI_F16) {
    const ph2 v = ph2{(_Float16)a, (_Float16)b};
    __builtin_memcpy(&r, &v, 4);
  } else {
    const pb2 v = pb2{(__bf16)a, (__bf16)b};
    __builtin_memcpy(&r, &v, 4);
  }
  return r;
}

__device__ __forceinline__ float pmax16(float v) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pmax32(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float psum16(float v) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float psum32(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// K / V (or Q / dO) tiles parked in LDS as 32 rows of 128 bytes: the 16-byte chunk c of row r sits at chunk c ^ ((r / 2) % 8),
// which keeps 16-byte stores (8 threads per row) and the operand reads below free of bank conflicts.
__device__ __forceinline__ uint32_t lds_chunk_off(int row, int chunk) { return (uint32_t)row * 128 + (uint32_t)((chunk ^ ((row >> 1) & 7)) << 4); }

// prefill_attn.hip: the segment table of a->cu_seqlens into seg_start (N ints; pidx: N ints of scratch) and the rows' softmax
// statistics - log2 of sum_j exp2(scale log2(e) q_i . k_j) - into lse (H, lse_stride) from a forward pass that stores no output.
int prefill_attn_stats(const uvmi_prefill_attn_args* a, int32_t* seg_start, int32_t* pidx, float* lse, int64_t lse_stride, void* stream);

}  // namespace uvmi
