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
// One element of the partial rotation: x cos - y sin for the first half of a pair, x cos + y sin for the second, as one
// fma on the rounded product y sin.  Every kernel that rotates q or k goes through here, so they round alike.
__device__ __forceinline__ float rope_rot(float x, float y, float c, float s, bool first) {
  const float t = __fmul_rn(y, s);
  return __builtin_fmaf(x, c, first ? -t : t);
}

__device__ __forceinline__ float wave_max(float v) {
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

}  // namespace uvmi
