// Shared helpers for the uvmi HIP kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/uvmi.h"

namespace uvmi {

void set_error(const char* fmt, ...);

#define UVMI_REQUIRE(cond, code, ...)       \
  do {                                      \
    if (!(cond)) {                          \
      ::uvmi::set_error(__VA_ARGS__);       \
      return (code);                        \
    }                                       \
  } while (0)

#define UVMI_CHECK_LAUNCH(what)                                                   \
  do {                                                                            \
    hipError_t e__ = hipGetLastError();                                           \
    if (e__ != hipSuccess) {                                                      \
      ::uvmi::set_error("%s: launch failed: %s", what, hipGetErrorString(e__));   \
      return UVMI_EHIP;                                                           \
    }                                                                             \
  } while (0)

typedef _Float16 half_t;
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_float(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
// round-to-nearest-even fp32 -> bf16: the hardware conversion of gfx950 (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t float_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  uint16_t r;
  __builtin_memcpy(&r, &b, 2);
  return r;
}
// two floats rounded to bf16 in one conversion (v_cvt_pk_bf16_f32): a in the low half of the word
__device__ __forceinline__ uint32_t float2_to_bf16x2(float a, float b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const bf16x2 r = __builtin_convertvector(f32x2{a, b}, bf16x2);
  uint32_t w;
  __builtin_memcpy(&w, &r, 4);
  return w;
}
__device__ __forceinline__ float half_bits_to_float(uint16_t b) {
  half_t h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}
__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
  half_t h = (half_t)f;  // v_cvt_f16_f32, round-to-nearest-even, fp16 subnormals kept
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

template <int DT> struct elem;  // load one element as float
template <> struct elem<UVMI_F16> {
  typedef uint16_t raw;
  static __device__ __forceinline__ float ld(const void* p, int64_t i) { return half_bits_to_float(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = float_to_half_bits(v); }
};
template <> struct elem<UVMI_BF16> {
  typedef uint16_t raw;
  static __device__ __forceinline__ float ld(const void* p, int64_t i) { return bf16_to_float(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = float_to_bf16(v); }
};
template <> struct elem<UVMI_F32> {
  typedef float raw;
  static __device__ __forceinline__ float ld(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
};

__device__ __forceinline__ int64_t load_index(const void* p, int is64, int64_t i) {
  return is64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}

inline bool is_float_dtype(int dt) { return dt == UVMI_F16 || dt == UVMI_BF16 || dt == UVMI_F32; }
inline int dtype_bytes(int dt) {
  switch (dt) {
    case UVMI_F16: case UVMI_BF16: return 2;
    case UVMI_F32: case UVMI_I32: return 4;
    case UVMI_I8: return 1;
    case UVMI_I64: return 8;
  }
  return 0;
}

// wave64 butterfly reductions (ds_bpermute based; used off the hot loops)
// a * b and a + b as operations of their own.  The compiler narrows float arithmetic on values that came from fp16 to
// native fp16 instructions and, with floating-point contraction on (the HIP default), would then fuse such a product and
// sum into one v_fma_f16 - one rounding where the reference's tensor expressions on 16-bit tensors round twice.  The
// pragma takes the contraction permission off these two operations wherever they are inlined.
__device__ __forceinline__ float mul_sep(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_sep(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}

// One element of the partial rotation: x cos - y sin for the first half of a pair, x cos + y sin for the second, with the
// roundings of the reference's expression x1 * cos - x2 * sin on tensors of the activation type (ultraviolet/model.py:219-226):
// each product is rounded to that type (rnd), then their sum.  Every kernel that rotates q or k goes through here, so
// they round alike.
template <class R>
__device__ __forceinline__ float rope_rot(float x, float y, float c, float s, bool first, R rnd) {
  const float a = rnd(mul_sep(x, c)), t = rnd(mul_sep(y, s));
  return rnd(add_sep(a, first ? -t : t));
}

// v + g * e with the roundings of the reference's v + g * ve on tensors of the activation type (ultraviolet/model.py:312-315)
template <class R>
__device__ __forceinline__ float ve_add(float v, float g, float e, R rnd) { return rnd(add_sep(v, rnd(mul_sep(g, e)))); }

// ---- cross-lane exchanges of a wave64 without the LDS crossbar where the hardware has another way: lanes l ^ 32 and l ^ 16 by
// the permlane swaps, l ^ 8 as a rotation inside a row of 16 (DPP), l ^ 4 by ds_swizzle, l ^ 2 and l ^ 1 as quad permutes (DPP)
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_mov_dpp((int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_xor1(float v) { return dpp_mov<0xb1>(v); }   // quad_perm [1, 0, 3, 2]
__device__ __forceinline__ float lane_xor2(float v) { return dpp_mov<0x4e>(v); }   // quad_perm [2, 3, 0, 1]
__device__ __forceinline__ float lane_xor4(float v) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_ds_swizzle((int)__float_as_uint(v), 0x101f));
}
__device__ __forceinline__ float lane_xor8(float v) { return dpp_mov<0x128>(v); }  // row_ror:8
__device__ __forceinline__ float lane_xor16(float v) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_ds_swizzle((int)__float_as_uint(v), 0x401f));
}
__device__ __forceinline__ float xmax16(float v) {  // max over lanes l, l ^ 16
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xmax32(float v) {  // max over lanes l, l ^ 32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// (the sums below add with contraction off: a reduction's first step must not fuse with the multiply that produced its
// argument - wave_sum(k * k) sums rounded squares wherever it is written)
__device__ __forceinline__ float xsum16(float v) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return add_sep(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xsum32(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return add_sep(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// Butterfly reductions over the 64 lanes, pairing lane ^ 32, 16, 8, 4, 2, 1 in that order: every kernel that sums or maximises
// over a wave goes through these, so that the same values round the same way wherever they are reduced.
__device__ __forceinline__ float wave_max(float v) {
  v = xmax32(v);
  v = xmax16(v);
  v = fmaxf(v, lane_xor8(v));
  v = fmaxf(v, lane_xor4(v));
  v = fmaxf(v, lane_xor2(v));
  v = fmaxf(v, lane_xor1(v));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = xsum32(v);
  v = xsum16(v);
  v = add_sep(v, lane_xor8(v));
  v = add_sep(v, lane_xor4(v));
  v = add_sep(v, lane_xor2(v));
  v = add_sep(v, lane_xor1(v));
  return v;
}

}  // namespace uvmi
