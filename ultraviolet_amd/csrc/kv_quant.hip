// int8 KV quantizer, flat-index cache write and the fused decode-time K+V append.
//
// Arithmetic contract (bit-exact with ultraviolet/kernels/kv_quant.py:12-19 of the reference):
//   s16 = fp16_rne(absmax(row) / 127)          IEEE fp32 division, round-to-nearest-even to fp16 (subnormals kept)
//   sf  = max(float(s16), 1e-30)
//   q   = int8(clamp(rint(x / sf), -127, 127))  IEEE fp32 division (no v_rcp shortcut), round-half-even
//
// Layout: a row of hd elements is owned by LPR = hd/4 adjacent lanes, 4 consecutive elements per lane, so a wave64
// quantizes 256/hd rows per pass with one 8-byte (bf16/fp16) load and one 4-byte packed int8 store per lane; the
// row absmax is a butterfly over the LPR lanes.  HBM-bound: 2*hd B read, hd+2 B written per row.
#include "common.h"

namespace uvmi {

template <int DT> struct vec4;
template <> struct vec4<UVMI_F16> {
  static __device__ __forceinline__ void ld(const void* p, int64_t off, float (&o)[4]) {
    const uint16_t* s = (const uint16_t*)p + off;
    uint2 w = *(const uint2*)s;
    o[0] = half_bits_to_float(w.x & 0xffff); o[1] = half_bits_to_float(w.x >> 16);
    o[2] = half_bits_to_float(w.y & 0xffff); o[3] = half_bits_to_float(w.y >> 16);
  }
};
template <> struct vec4<UVMI_BF16> {
  static __device__ __forceinline__ void ld(const void* p, int64_t off, float (&o)[4]) {
    const uint16_t* s = (const uint16_t*)p + off;
    uint2 w = *(const uint2*)s;
    o[0] = __uint_as_float(w.x << 16); o[1] = __uint_as_float(w.x & 0xffff0000u);
    o[2] = __uint_as_float(w.y << 16); o[3] = __uint_as_float(w.y & 0xffff0000u);
  }
};
template <> struct vec4<UVMI_F32> {
  static __device__ __forceinline__ void ld(const void* p, int64_t off, float (&o)[4]) {
    float4 w = *(const float4*)((const float*)p + off);
    o[0] = w.x; o[1] = w.y; o[2] = w.z; o[3] = w.w;
  }
};

// Quantize 4 values held by this lane given the row absmax; returns packed int8x4 and the fp16 scale bits.
__device__ __forceinline__ uint32_t quant4(const float (&x)[4], float amax, uint16_t& sbits) {
  float s = __fdiv_rn(amax, 127.0f);
  sbits = float_to_half_bits(s);
  float sf = fmaxf(half_bits_to_float(sbits), 1e-30f);
  uint32_t pk = 0;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float r = __builtin_rintf(__fdiv_rn(x[i], sf));
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    pk |= ((uint32_t)(int)r & 0xffu) << (8 * i);
  }
  return pk;
}

template <int LPR>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int o = LPR / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// mode 0: q/scale rows are contiguous (quantize_rows); mode 1: destination row = flat_idx[r] (kv_write)
template <int DT, int HD, int MODE>
__global__ __launch_bounds__(256) void quant_rows_kernel(const void* __restrict__ x, int64_t n_rows, int64_t xrs,
                                                         int8_t* __restrict__ q, uint16_t* __restrict__ sc,
                                                         const void* __restrict__ idx, int idx64, int64_t cache_rows) {
  constexpr int LPR = HD / 4;
  constexpr int RPB = 256 / LPR;  // rows per block pass
  const int lane_in_row = threadIdx.x % LPR;
  const int row_in_blk = threadIdx.x / LPR;
  for (int64_t r = (int64_t)blockIdx.x * RPB + row_in_blk; r < n_rows; r += (int64_t)gridDim.x * RPB) {
    float v[4];
    vec4<DT>::ld(x, r * xrs + lane_in_row * 4, v);
    float am = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    am = group_max<LPR>(am);
    uint16_t sb;
    uint32_t pk = quant4(v, am, sb);
    int64_t dst = r;
    if (MODE == 1) {
      dst = load_index(idx, idx64, r);
      if (dst < 0 || dst >= cache_rows) continue;
    }
    *(uint32_t*)(q + dst * HD + lane_in_row * 4) = pk;
    if (lane_in_row == 0) sc[dst] = sb;
  }
}

// Any hd (multiple of 1): one wave per row, strided lanes.  Slow path for shapes outside {16,32,64,128,256}.
template <int DT, int MODE>
__global__ __launch_bounds__(64) void quant_rows_generic(const void* __restrict__ x, int64_t n_rows, int hd, int64_t xrs,
                                                         int8_t* __restrict__ q, uint16_t* __restrict__ sc,
                                                         const void* __restrict__ idx, int idx64, int64_t cache_rows) {
  for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) {
    float am = 0.f;
    for (int d = threadIdx.x; d < hd; d += 64) am = fmaxf(am, fabsf(elem<DT>::ld(x, r * xrs + d)));
    am = wave_max(am);
    uint16_t sb = float_to_half_bits(__fdiv_rn(am, 127.0f));
    float sf = fmaxf(half_bits_to_float(sb), 1e-30f);
    int64_t dst = r;
    if (MODE == 1) {
      dst = load_index(idx, idx64, r);
      if (dst < 0 || dst >= cache_rows) continue;
    }
    for (int d = threadIdx.x; d < hd; d += 64) {
      float v = __builtin_rintf(__fdiv_rn(elem<DT>::ld(x, r * xrs + d), sf));
      q[dst * hd + d] = (int8_t)(int)fminf(fmaxf(v, -127.0f), 127.0f);
    }
    if (threadIdx.x == 0) sc[dst] = sb;
  }
}

// Un-quantized cache (fp16 / bf16): row copy with a cast.
template <int DT, int CDT>
__global__ __launch_bounds__(256) void copy_rows_kernel(const void* __restrict__ x, int64_t n_rows, int hd, int64_t xrs,
                                                        void* __restrict__ cache, const void* __restrict__ idx, int idx64,
                                                        int64_t cache_rows) {
  int64_t total = n_rows * hd;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t r = i / hd;
    int d = (int)(i % hd);
    int64_t dst = load_index(idx, idx64, r);
    if (dst < 0 || dst >= cache_rows) continue;
    elem<CDT>::st(cache, dst * hd + d, elem<DT>::ld(x, r * xrs + d));
  }
}

template <int DT, int HD>
__global__ __launch_bounds__(256) void dequant_rows_kernel(const int8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                           int64_t n_rows, void* __restrict__ out) {
  int64_t total = n_rows * HD;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t r = i / HD;
    elem<DT>::st(out, i, (float)q[i] * half_bits_to_float(sc[r]));
  }
}
__global__ __launch_bounds__(256) void dequant_rows_any(const int8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                        int64_t n_rows, int hd, void* __restrict__ out, int odt) {
  int64_t total = n_rows * hd;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    float v = (float)q[i] * half_bits_to_float(sc[i / hd]);
    if (odt == UVMI_F16) elem<UVMI_F16>::st(out, i, v);
    else if (odt == UVMI_BF16) elem<UVMI_BF16>::st(out, i, v);
    else elem<UVMI_F32>::st(out, i, v);
  }
}

// Fused K+V append: blockIdx.y selects K (0) or V (1); a group of HD/4 lanes owns one (row, kv head).
template <int DT, int HD>
__global__ __launch_bounds__(256) void kv_append_kernel(uvmi_kv_append_args a) {
  constexpr int LPR = HD / 4;
  constexpr int RPB = 256 / LPR;
  const int lane_in_row = threadIdx.x % LPR;
  const int64_t n = (int64_t)a.B * a.KH;
  const bool isv = blockIdx.y == 1;
  const void* x = isv ? a.v : a.k;
  int8_t* cache = isv ? a.v_cache : a.k_cache;
  uint16_t* sc = isv ? a.v_scale : a.k_scale;
  const int i64 = a.idx_dtype == UVMI_I64;
  for (int64_t r = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR; r < n; r += (int64_t)gridDim.x * RPB) {
    const int64_t b = r / a.KH, h = r % a.KH;
    float v[4];
    vec4<DT>::ld(x, b * a.sxb + h * a.sxh + lane_in_row * 4, v);
    float am = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    am = group_max<LPR>(am);
    uint16_t sb;
    uint32_t pk = quant4(v, am, sb);
    int64_t p = load_index(a.pos, i64, b);
    if (p < 0) continue;
    int64_t slot = a.ring ? p % a.S : p;
    if (slot >= a.S) continue;
    const int64_t cb = a.rows ? load_index(a.rows, i64, b) : b;
    if (cb < 0) continue;
    *(uint32_t*)(cache + cb * a.scb + h * a.sch + slot * a.scs + lane_in_row * 4) = pk;
    if (lane_in_row == 0) sc[cb * a.ssb + h * a.ssh + slot] = sb;
  }
}

static inline int grid_for(int64_t n_units, int per_block, int cap = 4096) {
  int64_t g = (n_units + per_block - 1) / per_block;
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return (int)g;
}

template <int DT, int MODE>
static int launch_quant(const void* x, int64_t n_rows, int hd, int64_t xrs, int8_t* q, uint16_t* sc, const void* idx,
                        int idx64, int64_t cache_rows, hipStream_t st) {
  const bool vec_ok = ((uintptr_t)x % (dtype_bytes(DT) * 4) == 0) && (xrs % 4 == 0) && ((uintptr_t)q % 4 == 0);
#define UVMI_Q(HDV)                                                                                              \
  case HDV:                                                                                                      \
    if (vec_ok) {                                                                                                \
      hipLaunchKernelGGL((quant_rows_kernel<DT, HDV, MODE>), dim3(grid_for(n_rows, 256 / (HDV / 4))), dim3(256), 0, st, \
                         x, n_rows, xrs, q, sc, idx, idx64, cache_rows);                                         \
      return 0;                                                                                                  \
    }                                                                                                            \
    break;
  switch (hd) {
    UVMI_Q(16) UVMI_Q(32) UVMI_Q(64) UVMI_Q(128) UVMI_Q(256)
    default: break;
  }
#undef UVMI_Q
  hipLaunchKernelGGL((quant_rows_generic<DT, MODE>), dim3(grid_for(n_rows, 1, 65535)), dim3(64), 0, st, x, n_rows, hd, xrs,
                     q, sc, idx, idx64, cache_rows);
  return 0;
}

template <int MODE>
static int dispatch_quant(int dt, const void* x, int64_t n_rows, int hd, int64_t xrs, int8_t* q, uint16_t* sc,
                          const void* idx, int idx64, int64_t cache_rows, hipStream_t st) {
  switch (dt) {
    case UVMI_F16: return launch_quant<UVMI_F16, MODE>(x, n_rows, hd, xrs, q, sc, idx, idx64, cache_rows, st);
    case UVMI_BF16: return launch_quant<UVMI_BF16, MODE>(x, n_rows, hd, xrs, q, sc, idx, idx64, cache_rows, st);
    case UVMI_F32: return launch_quant<UVMI_F32, MODE>(x, n_rows, hd, xrs, q, sc, idx, idx64, cache_rows, st);
  }
  return -1;
}

}  // namespace uvmi

using namespace uvmi;

extern "C" int uvmi_quantize_rows(const void* x, int x_dtype, int64_t n_rows, int hd, int64_t x_row_stride, int8_t* q,
                                  uint16_t* scale, void* stream) {
  UVMI_REQUIRE(x && q && scale, UVMI_EINVAL, "uvmi_quantize_rows: null pointer");
  UVMI_REQUIRE(is_float_dtype(x_dtype), UVMI_EINVAL, "uvmi_quantize_rows: x_dtype %d is not a float type", x_dtype);
  UVMI_REQUIRE(n_rows >= 0 && hd > 0 && hd <= 4096 && x_row_stride >= hd, UVMI_EINVAL,
               "uvmi_quantize_rows: bad sizes n_rows=%lld hd=%d stride=%lld", (long long)n_rows, hd, (long long)x_row_stride);
  if (n_rows == 0) return UVMI_OK;
  dispatch_quant<0>(x_dtype, x, n_rows, hd, x_row_stride, q, scale, nullptr, 0, 0, (hipStream_t)stream);
  UVMI_CHECK_LAUNCH("uvmi_quantize_rows");
  return UVMI_OK;
}

extern "C" int uvmi_dequantize_rows(const int8_t* q, const uint16_t* scale, int64_t n_rows, int hd, void* out, int out_dtype,
                                    void* stream) {
  UVMI_REQUIRE(q && scale && out, UVMI_EINVAL, "uvmi_dequantize_rows: null pointer");
  UVMI_REQUIRE(is_float_dtype(out_dtype), UVMI_EINVAL, "uvmi_dequantize_rows: bad out_dtype %d", out_dtype);
  UVMI_REQUIRE(n_rows >= 0 && hd > 0, UVMI_EINVAL, "uvmi_dequantize_rows: bad sizes");
  if (n_rows == 0) return UVMI_OK;
  hipLaunchKernelGGL(dequant_rows_any, dim3(grid_for(n_rows * hd, 256 * 8)), dim3(256), 0, (hipStream_t)stream, q, scale,
                     n_rows, hd, out, out_dtype);
  UVMI_CHECK_LAUNCH("uvmi_dequantize_rows");
  return UVMI_OK;
}

extern "C" int uvmi_kv_write(void* cache, int cache_dtype, uint16_t* scale, int64_t cache_rows, const void* flat_idx,
                             int idx_dtype, const void* x, int x_dtype, int64_t n_rows, int hd, int64_t x_row_stride,
                             void* stream) {
  UVMI_REQUIRE(cache && flat_idx && x, UVMI_EINVAL, "uvmi_kv_write: null pointer");
  UVMI_REQUIRE(idx_dtype == UVMI_I64 || idx_dtype == UVMI_I32, UVMI_EINVAL, "uvmi_kv_write: idx_dtype must be I32/I64");
  UVMI_REQUIRE(is_float_dtype(x_dtype), UVMI_EINVAL, "uvmi_kv_write: x_dtype %d is not a float type", x_dtype);
  UVMI_REQUIRE(n_rows >= 0 && hd > 0 && cache_rows >= 0 && x_row_stride >= hd, UVMI_EINVAL, "uvmi_kv_write: bad sizes");
  if (n_rows == 0) return UVMI_OK;
  hipStream_t st = (hipStream_t)stream;
  const int i64 = idx_dtype == UVMI_I64;
  if (scale) {
    UVMI_REQUIRE(cache_dtype == UVMI_I8, UVMI_EINVAL, "uvmi_kv_write: a scale tensor needs an int8 cache");
    dispatch_quant<1>(x_dtype, x, n_rows, hd, x_row_stride, (int8_t*)cache, scale, flat_idx, i64, cache_rows, st);
  } else {
    UVMI_REQUIRE(cache_dtype == UVMI_F16 || cache_dtype == UVMI_BF16, UVMI_EUNSUPPORTED,
                 "uvmi_kv_write: unquantized cache must be F16 or BF16");
    dim3 g(grid_for(n_rows * hd, 256 * 4)), blk(256);
#define UVMI_C(XD, CD) hipLaunchKernelGGL((copy_rows_kernel<XD, CD>), g, blk, 0, st, x, n_rows, hd, x_row_stride, cache, flat_idx, i64, cache_rows)
    if (cache_dtype == UVMI_F16) {
      if (x_dtype == UVMI_F16) UVMI_C(UVMI_F16, UVMI_F16); else if (x_dtype == UVMI_BF16) UVMI_C(UVMI_BF16, UVMI_F16); else UVMI_C(UVMI_F32, UVMI_F16);
    } else {
      if (x_dtype == UVMI_F16) UVMI_C(UVMI_F16, UVMI_BF16); else if (x_dtype == UVMI_BF16) UVMI_C(UVMI_BF16, UVMI_BF16); else UVMI_C(UVMI_F32, UVMI_BF16);
    }
#undef UVMI_C
  }
  UVMI_CHECK_LAUNCH("uvmi_kv_write");
  return UVMI_OK;
}

extern "C" int uvmi_kv_append(const uvmi_kv_append_args* a, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_kv_append: null args");
  UVMI_REQUIRE(a->k && a->v && a->k_cache && a->v_cache && a->k_scale && a->v_scale && a->pos, UVMI_EINVAL,
               "uvmi_kv_append: null pointer");
  UVMI_REQUIRE(a->idx_dtype == UVMI_I64 || a->idx_dtype == UVMI_I32, UVMI_EINVAL, "uvmi_kv_append: idx_dtype must be I32/I64");
  UVMI_REQUIRE(a->B >= 0 && a->KH > 0 && a->S > 0, UVMI_EINVAL, "uvmi_kv_append: bad sizes");
  UVMI_REQUIRE(a->hd == 64 || a->hd == 128 || a->hd == 32 || a->hd == 16, UVMI_EUNSUPPORTED,
               "uvmi_kv_append: head_dim %d not in {16,32,64,128}", a->hd);
  UVMI_REQUIRE(a->x_dtype == UVMI_F16 || a->x_dtype == UVMI_BF16 || a->x_dtype == UVMI_F32, UVMI_EINVAL,
               "uvmi_kv_append: x_dtype must be a float type");
  const int eb = dtype_bytes(a->x_dtype) * 4;
  UVMI_REQUIRE((uintptr_t)a->k % eb == 0 && (uintptr_t)a->v % eb == 0 && a->sxb % 4 == 0 && a->sxh % 4 == 0, UVMI_EUNSUPPORTED,
               "uvmi_kv_append: k/v rows must be aligned to 4 elements");
  UVMI_REQUIRE((uintptr_t)a->k_cache % 4 == 0 && (uintptr_t)a->v_cache % 4 == 0 && a->scb % 4 == 0 && a->sch % 4 == 0 &&
                   a->scs % 4 == 0, UVMI_EUNSUPPORTED, "uvmi_kv_append: cache rows must be 4-byte aligned");
  if (a->B == 0) return UVMI_OK;
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = (int64_t)a->B * a->KH;
#define UVMI_A(DT, HDV) hipLaunchKernelGGL((kv_append_kernel<DT, HDV>), dim3(grid_for(n, 256 / (HDV / 4)), 2), dim3(256), 0, st, *a)
#define UVMI_AH(DT)                                      \
  switch (a->hd) {                                       \
    case 16: UVMI_A(DT, 16); break;                      \
    case 32: UVMI_A(DT, 32); break;                      \
    case 64: UVMI_A(DT, 64); break;                      \
    default: UVMI_A(DT, 128); break;                     \
  }
  if (a->x_dtype == UVMI_F16) { UVMI_AH(UVMI_F16) } else if (a->x_dtype == UVMI_BF16) { UVMI_AH(UVMI_BF16) } else { UVMI_AH(UVMI_F32) }
#undef UVMI_AH
#undef UVMI_A
  UVMI_CHECK_LAUNCH("uvmi_kv_append");
  return UVMI_OK;
}
