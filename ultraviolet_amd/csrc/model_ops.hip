// Fused per-token kernels of the UV-50M decode / prefill step: everything between the GEMMs.
//
// One wave64 per token row.  All arithmetic is fp32; values are rounded to the activation type T (fp16 / bf16 / fp32)
// where the next GEMM reads them.  Weightless RMSNorm takes its eps from the caller: the reference calls
// torch.nn.functional.rms_norm(x, eps=None) (ultraviolet/model.py:190-191), whose default has been the machine epsilon
// of the input dtype in some torch releases and of fp32 in others, so the host passes what its torch does.
//
//   embed_norm   x = rmsnorm(E[tok]); n = rmsnorm(x)                                    (fast_decode.py:286, 305)
//   add_norm     h = a*x + b*y; n = rmsnorm(h)          residual lambdas + pre-norm     (model.py:567-571)
//   qkv_post     value-embedding gate, QK-norm, partial RoPE, q out, int8 K/V append    (model.py:302-319,
//                                                                                        fast_decode.py:291-294, 315-317)
//   attn_post    XSA projection removal + per-head sigmoid gate                         (model.py:321-333)
//   swiglu       silu(g) * u                                                            (model.py:388-391)
//
// All of them are HBM/launch-bound and tiny next to the GEMMs and attention; they exist to keep the step at a handful
// of launches per layer and to write K/V straight into the int8 cache without a round trip through HBM.
#include "common.h"

#include <type_traits>

namespace uvmi {

template <int DT> __device__ __forceinline__ float round_t(float v);
template <> __device__ __forceinline__ float round_t<UVMI_F32>(float v) { return v; }
template <> __device__ __forceinline__ float round_t<UVMI_F16>(float v) { return (float)(half_t)v; }
template <> __device__ __forceinline__ float round_t<UVMI_BF16>(float v) { return bf16_to_float(float_to_bf16(v)); }

// ------------------------------------------------------------------------------------------------ embed / residual
// MODE 0: src = E[tok[r]] ; x = rmsnorm(src)        MODE 1: x = a*xin + b*yin
// then n = rmsnorm(x) (of the rounded x).  d <= 64 * 2 * NP.
template <int DT, int MODE>
__global__ __launch_bounds__(256) void norm_kernel(const void* __restrict__ xin, const void* __restrict__ yin,
                                                   const int64_t* __restrict__ tok, int64_t vocab, float a, float b,
                                                   void* __restrict__ xout, void* __restrict__ nout, int64_t rows, int d, float eps) {
  constexpr int NP = 16;  // pairs per lane: d <= 2048
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int np = d / 2;
  float v0[NP], v1[NP];
  float ss = 0.f;
  int64_t src = r;
  if (MODE == 0) {
    src = tok[r];
    if (src < 0) src = 0;
    if (src >= vocab) src = vocab - 1;
  }
#pragma unroll
  for (int i = 0; i < NP; i++) {
    const int pidx = lane + 64 * i;
    v0[i] = v1[i] = 0.f;
    if (pidx < np) {
      float x0 = elem<DT>::ld(xin, src * d + 2 * pidx), x1 = elem<DT>::ld(xin, src * d + 2 * pidx + 1);
      if (MODE == 1) {
        x0 = round_t<DT>(a * x0 + b * elem<DT>::ld(yin, r * d + 2 * pidx));
        x1 = round_t<DT>(a * x1 + b * elem<DT>::ld(yin, r * d + 2 * pidx + 1));
      }
      v0[i] = x0; v1[i] = x1;
      ss += x0 * x0 + x1 * x1;
    }
  }
  if (MODE == 0) {
    const float rs = rsqrtf(wave_sum(ss) / (float)d + eps);
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < NP; i++) {
      v0[i] = round_t<DT>(v0[i] * rs); v1[i] = round_t<DT>(v1[i] * rs);
      ss += v0[i] * v0[i] + v1[i] * v1[i];
    }
  }
  const float rn = rsqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
  for (int i = 0; i < NP; i++) {
    const int pidx = lane + 64 * i;
    if (pidx < np) {
      if (xout) { elem<DT>::st(xout, r * d + 2 * pidx, v0[i]); elem<DT>::st(xout, r * d + 2 * pidx + 1, v1[i]); }
      elem<DT>::st(nout, r * d + 2 * pidx, v0[i] * rn);
      elem<DT>::st(nout, r * d + 2 * pidx + 1, v1[i] * rn);
    }
  }
}

// ------------------------------------------------------------------------------------------------ qkv_post (hd = 64)
struct QkvArgs {
  const void* qkv; const void* xn; const void* ve_table; const float* ve_gate; const int64_t* tok;
  const int64_t* pos; const int64_t* rows; const int64_t* last_pos; const float* inv_freq;
  void* q_out; void* k_out; void* v_out;
  int8_t* k_cache; int8_t* v_cache; uint16_t* k_scale; uint16_t* v_scale;
  int64_t scb, sch, scs, ssb, ssh;
  int64_t n, vocab;
  int H, KH, d, ve_ch, n_pairs, S, ring, has_ve, rope, q_dt;
  float eps;
};

__device__ __forceinline__ void store_q(void* p, int dt, int64_t i, float v) {
  if (dt == UVMI_BF16) elem<UVMI_BF16>::st(p, i, v); else elem<UVMI_F16>::st(p, i, v);
}

template <int DT>
__global__ __launch_bounds__(256) void qkv_post_kernel(QkvArgs A) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= A.n) return;
  const int W = (A.H + 2 * A.KH) * 64;
  const int64_t base = r * W;
  const int64_t p = A.pos[r];
  // RoPE angle of this lane's pair (lanes 0..n_pairs-1 and n_pairs..2n_pairs-1 share a frequency)
  float cs = 1.f, sn = 0.f;
  const bool rot = A.rope && lane < 2 * A.n_pairs;
  if (rot) {
    const float th = (float)p * A.inv_freq[lane % A.n_pairs];
    cs = round_t<DT>(cosf(th));
    sn = round_t<DT>(sinf(th));
  }
  auto norm_rope = [&](float x) -> float {  // QK-norm over the 64 lanes, then partial RoPE (half-split pairing)
    const float rs = rsqrtf(wave_sum(x * x) * (1.0f / 64.0f) + A.eps);
    const float xn = round_t<DT>(x * rs);
    if (!A.rope) return xn;
    const float other = __shfl_xor(xn, A.n_pairs, 64);  // lane d <-> d + n_pairs (n_pairs is a power of two)
    if (!rot) return xn;
    return lane < A.n_pairs ? round_t<DT>(xn * cs - other * sn) : round_t<DT>(other * sn + xn * cs);
  };
  // ---- queries
  for (int h = 0; h < A.H; h++) {
    const float q = norm_rope(elem<DT>::ld(A.qkv, base + h * 64 + lane));
    store_q(A.q_out, A.q_dt, (r * A.H + h) * 64 + lane, q);
  }
  // ---- keys / values per kv head
  const int64_t row = A.rows ? A.rows[r] : r;
  const int64_t slot = A.ring ? (p % A.S) : p;
  bool wr = A.k_cache && row >= 0 && p >= 0 && slot < A.S;
  if (wr && A.ring && A.last_pos) wr = p > A.last_pos[r] - A.S;  // only the last S positions of a prompt survive in a ring
  for (int kh = 0; kh < A.KH; kh++) {
    const float k = norm_rope(elem<DT>::ld(A.qkv, base + (A.H + kh) * 64 + lane));
    float v = elem<DT>::ld(A.qkv, base + (A.H + A.KH + kh) * 64 + lane);
    if (A.has_ve) {  // v += 2 sigmoid(W xn[:ve_ch]) * value_embed[tok]
      float dot = 0.f;
      if (lane < A.ve_ch) dot = elem<DT>::ld(A.xn, r * A.d + lane) * A.ve_gate[kh * A.ve_ch + lane];
      dot = round_t<DT>(wave_sum(dot));
      const float g = round_t<DT>(2.0f * round_t<DT>(1.0f / (1.0f + __expf(-dot))));
      int64_t t = A.tok[r];
      if (t < 0) t = 0;
      if (t >= A.vocab) t = A.vocab - 1;
      const float ve = elem<DT>::ld(A.ve_table, (t * A.KH + kh) * 64 + lane);
      v = round_t<DT>(v + round_t<DT>(g * ve));
    }
    if (A.k_out) elem<DT>::st(A.k_out, (r * A.KH + kh) * 64 + lane, k);
    if (A.v_out) elem<DT>::st(A.v_out, (r * A.KH + kh) * 64 + lane, v);
    if (wr) {  // int8 append, same arithmetic as the standalone quantizer
      const float vals[2] = {k, v};
      int8_t* caches[2] = {A.k_cache, A.v_cache};
      uint16_t* scales[2] = {A.k_scale, A.v_scale};
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const float am = wave_max(fabsf(vals[j]));
        const uint16_t sb = float_to_half_bits(__fdiv_rn(am, 127.0f));
        const float sf = fmaxf(half_bits_to_float(sb), 1e-30f);
        float qv = __builtin_rintf(__fdiv_rn(vals[j], sf));
        qv = fminf(fmaxf(qv, -127.0f), 127.0f);
        caches[j][row * A.scb + kh * A.sch + slot * A.scs + lane] = (int8_t)(int)qv;
        if (lane == 0) scales[j][row * A.ssb + kh * A.ssh + slot] = sb;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ attn_post (hd = 64)
struct PostArgs {
  const void* z; const void* v; const void* xn; const float* gate_w; const float* xsa;
  void* out; int64_t n; int H, KH, d, gate_ch, z_dt; float xsa_eps;
};

template <int DT>
__global__ __launch_bounds__(256) void attn_post_kernel(PostArgs A) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= A.n) return;
  const int G = A.H / A.KH;
  for (int h = 0; h < A.H; h++) {
    const int kh = h / G;
    float z = A.z_dt == UVMI_BF16 ? elem<UVMI_BF16>::ld(A.z, (r * A.H + h) * 64 + lane) : elem<UVMI_F16>::ld(A.z, (r * A.H + h) * 64 + lane);
    if (A.xsa) {  // z -= tanh(alpha_h) (z . v_hat) v_hat, v_hat = v / max(|v|, eps), in fp32
      const float v = elem<DT>::ld(A.v, (r * A.KH + kh) * 64 + lane);
      const float nv = sqrtf(wave_sum(v * v));
      const float vh = v / fmaxf(nv, A.xsa_eps);
      const float proj = wave_sum(z * vh);
      z = round_t<DT>(z - A.xsa[h] * proj * vh);
    }
    if (A.gate_w) {  // z *= 2 sigmoid(W_h . xn[:gate_ch])
      float dot = 0.f;
      for (int c = lane; c < A.gate_ch; c += 64) dot += elem<DT>::ld(A.xn, r * A.d + c) * A.gate_w[h * A.gate_ch + c];
      dot = round_t<DT>(wave_sum(dot));
      const float g = round_t<DT>(2.0f * round_t<DT>(1.0f / (1.0f + __expf(-dot))));
      z = z * g;
    }
    elem<DT>::st(A.out, (r * A.H + h) * 64 + lane, z);
  }
}

// ------------------------------------------------------------------------------------------------ swiglu
template <int DT>
__global__ __launch_bounds__(256) void swiglu_kernel(const void* __restrict__ gu, void* __restrict__ out, int64_t rows, int f) {
  const int64_t total = rows * f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / f;
    const int j = (int)(i % f);
    const float g = elem<DT>::ld(gu, r * 2 * f + j), u = elem<DT>::ld(gu, r * 2 * f + f + j);
    const float s = round_t<DT>(g / (1.0f + __expf(-g)));
    elem<DT>::st(out, i, s * u);
  }
}

}  // namespace uvmi

using namespace uvmi;

template <typename F>
static void dispatch_dt(int dt, F&& f) {
  if (dt == UVMI_F16) f(std::integral_constant<int, UVMI_F16>{});
  else if (dt == UVMI_BF16) f(std::integral_constant<int, UVMI_BF16>{});
  else f(std::integral_constant<int, UVMI_F32>{});
}

extern "C" int uvmi_embed_norm(const void* table, int dtype, int64_t vocab, const int64_t* tok, int64_t rows, int d, float eps,
                               void* x_out, void* n_out, void* stream) {
  UVMI_REQUIRE(table && tok && n_out, UVMI_EINVAL, "uvmi_embed_norm: null pointer");
  UVMI_REQUIRE(is_float_dtype(dtype) && rows >= 0 && d > 0 && d % 2 == 0 && d <= 2048 && vocab > 0, UVMI_EINVAL, "uvmi_embed_norm: bad arguments");
  if (rows == 0) return UVMI_OK;
  const dim3 grid((unsigned)((rows + 3) / 4)), blk(256);
  dispatch_dt(dtype, [&](auto DT) { hipLaunchKernelGGL((norm_kernel<decltype(DT)::value, 0>), grid, blk, 0, (hipStream_t)stream, table, nullptr, tok, vocab, 0.f, 0.f, x_out, n_out, rows, d, eps); });
  UVMI_CHECK_LAUNCH("uvmi_embed_norm");
  return UVMI_OK;
}

extern "C" int uvmi_add_norm(const void* x, const void* y, int dtype, float a, float b, int64_t rows, int d, float eps, void* h_out,
                             void* n_out, void* stream) {
  UVMI_REQUIRE(x && y && n_out, UVMI_EINVAL, "uvmi_add_norm: null pointer");
  UVMI_REQUIRE(is_float_dtype(dtype) && rows >= 0 && d > 0 && d % 2 == 0 && d <= 2048, UVMI_EINVAL, "uvmi_add_norm: bad arguments");
  if (rows == 0) return UVMI_OK;
  const dim3 grid((unsigned)((rows + 3) / 4)), blk(256);
  dispatch_dt(dtype, [&](auto DT) { hipLaunchKernelGGL((norm_kernel<decltype(DT)::value, 1>), grid, blk, 0, (hipStream_t)stream, x, y, nullptr, 0, a, b, h_out, n_out, rows, d, eps); });
  UVMI_CHECK_LAUNCH("uvmi_add_norm");
  return UVMI_OK;
}

extern "C" int uvmi_qkv_post(const uvmi_qkv_post_args* a, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_qkv_post: null args");
  UVMI_REQUIRE(a->qkv && a->pos && a->q_out, UVMI_EINVAL, "uvmi_qkv_post: null pointer");
  UVMI_REQUIRE(a->hd == 64, UVMI_EUNSUPPORTED, "uvmi_qkv_post: head_dim %d (only 64)", a->hd);
  UVMI_REQUIRE(is_float_dtype(a->dtype) && (a->q_dtype == UVMI_F16 || a->q_dtype == UVMI_BF16), UVMI_EINVAL, "uvmi_qkv_post: bad dtype");
  UVMI_REQUIRE(a->n >= 0 && a->H > 0 && a->KH > 0 && a->H % a->KH == 0, UVMI_EINVAL, "uvmi_qkv_post: bad sizes");
  UVMI_REQUIRE(!a->rope || (a->inv_freq && a->n_pairs > 0 && a->n_pairs <= 32 && (a->n_pairs & (a->n_pairs - 1)) == 0), UVMI_EUNSUPPORTED,
               "uvmi_qkv_post: rope needs inv_freq and a power-of-two pair count <= 32");
  UVMI_REQUIRE(!a->has_ve || (a->xn && a->ve_table && a->ve_gate && a->tok && a->ve_ch > 0 && a->ve_ch <= 64 && a->vocab > 0), UVMI_EINVAL,
               "uvmi_qkv_post: value-embedding inputs missing");
  UVMI_REQUIRE(!a->k_cache || (a->v_cache && a->k_scale && a->v_scale && a->S > 0), UVMI_EINVAL, "uvmi_qkv_post: incomplete cache arguments");
  if (a->n == 0) return UVMI_OK;
  QkvArgs A;
  A.qkv = a->qkv; A.xn = a->xn; A.ve_table = a->ve_table; A.ve_gate = a->ve_gate; A.tok = a->tok; A.pos = a->pos; A.rows = a->rows;
  A.last_pos = a->last_pos; A.inv_freq = a->inv_freq; A.q_out = a->q_out; A.k_out = a->k_out; A.v_out = a->v_out;
  A.k_cache = a->k_cache; A.v_cache = a->v_cache; A.k_scale = a->k_scale; A.v_scale = a->v_scale;
  A.scb = a->scb; A.sch = a->sch; A.scs = a->scs; A.ssb = a->ssb; A.ssh = a->ssh; A.n = a->n; A.vocab = a->vocab;
  A.H = a->H; A.KH = a->KH; A.d = a->d; A.ve_ch = a->ve_ch; A.n_pairs = a->n_pairs; A.S = a->S; A.ring = a->ring; A.has_ve = a->has_ve;
  A.rope = a->rope; A.q_dt = a->q_dtype; A.eps = a->eps;
  const dim3 grid((unsigned)((a->n + 3) / 4)), blk(256);
  dispatch_dt(a->dtype, [&](auto DT) { hipLaunchKernelGGL((qkv_post_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, A); });
  UVMI_CHECK_LAUNCH("uvmi_qkv_post");
  return UVMI_OK;
}

extern "C" int uvmi_attn_post(const void* z, int z_dtype, const void* v, const void* xn, int dtype, const float* gate_w, const float* xsa,
                              float xsa_eps, int64_t n, int H, int KH, int hd, int d, int gate_ch, void* out, void* stream) {
  UVMI_REQUIRE(z && out, UVMI_EINVAL, "uvmi_attn_post: null pointer");
  UVMI_REQUIRE(hd == 64, UVMI_EUNSUPPORTED, "uvmi_attn_post: head_dim %d (only 64)", hd);
  UVMI_REQUIRE(is_float_dtype(dtype) && (z_dtype == UVMI_F16 || z_dtype == UVMI_BF16), UVMI_EINVAL, "uvmi_attn_post: bad dtype");
  UVMI_REQUIRE(!xsa || v, UVMI_EINVAL, "uvmi_attn_post: XSA needs v");
  UVMI_REQUIRE(!gate_w || (xn && gate_ch > 0 && gate_ch <= d), UVMI_EINVAL, "uvmi_attn_post: gate needs xn and gate_ch");
  UVMI_REQUIRE(n >= 0 && H > 0 && KH > 0 && H % KH == 0, UVMI_EINVAL, "uvmi_attn_post: bad sizes");
  if (n == 0) return UVMI_OK;
  PostArgs A{z, v, xn, gate_w, xsa, out, n, H, KH, d, gate_ch, z_dtype, xsa_eps};
  const dim3 grid((unsigned)((n + 3) / 4)), blk(256);
  dispatch_dt(dtype, [&](auto DT) { hipLaunchKernelGGL((attn_post_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, A); });
  UVMI_CHECK_LAUNCH("uvmi_attn_post");
  return UVMI_OK;
}

extern "C" int uvmi_swiglu(const void* gu, int dtype, int64_t rows, int f, void* out, void* stream) {
  UVMI_REQUIRE(gu && out, UVMI_EINVAL, "uvmi_swiglu: null pointer");
  UVMI_REQUIRE(is_float_dtype(dtype) && rows >= 0 && f > 0, UVMI_EINVAL, "uvmi_swiglu: bad arguments");
  if (rows == 0) return UVMI_OK;
  int64_t blocks = (rows * f + 256 * 4 - 1) / (256 * 4);
  if (blocks > 8192) blocks = 8192;
  const dim3 grid((unsigned)blocks), blk(256);
  dispatch_dt(dtype, [&](auto DT) { hipLaunchKernelGGL((swiglu_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, gu, out, rows, f); });
  UVMI_CHECK_LAUNCH("uvmi_swiglu");
  return UVMI_OK;
}
