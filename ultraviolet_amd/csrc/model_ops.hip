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

template <int DT>
__device__ __forceinline__ void ld2(const void* p, int64_t i, float& a, float& b) {  // elements i, i+1 (i even)
  if (DT == UVMI_F32) { const float2 v = *(const float2*)((const float*)p + i); a = v.x; b = v.y; }
  else {
    const uint32_t w = *(const uint32_t*)((const uint16_t*)p + i);
    if (DT == UVMI_BF16) { a = __uint_as_float(w << 16); b = __uint_as_float(w & 0xffff0000u); }
    else { a = half_bits_to_float(w & 0xffff); b = half_bits_to_float(w >> 16); }
  }
}
template <int DT>
__device__ __forceinline__ void st2(void* p, int64_t i, float a, float b) {
  if (DT == UVMI_F32) *(float2*)((float*)p + i) = float2{a, b};
  else {
    const uint32_t lo = DT == UVMI_BF16 ? float_to_bf16(a) : float_to_half_bits(a);
    const uint32_t hi = DT == UVMI_BF16 ? float_to_bf16(b) : float_to_half_bits(b);
    *(uint32_t*)((uint16_t*)p + i) = lo | (hi << 16);
  }
}

template <int DT>
__device__ __forceinline__ void ld8(const void* p, int64_t i, float (&o)[8]) {  // 8 consecutive elements starting at i
  if (DT == UVMI_F32) {
    const float4 a = *(const float4*)((const float*)p + i), b = *(const float4*)((const float*)p + i + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
    const uint4 w = *(const uint4*)((const uint16_t*)p + i);
    const uint32_t r[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (DT == UVMI_BF16) { o[2 * j] = __uint_as_float(r[j] << 16); o[2 * j + 1] = __uint_as_float(r[j] & 0xffff0000u); }
      else { o[2 * j] = half_bits_to_float(r[j] & 0xffff); o[2 * j + 1] = half_bits_to_float(r[j] >> 16); }
    }
  }
}
template <int DT>
__device__ __forceinline__ void st8(void* p, int64_t i, const float (&v)[8]) {
  if (DT == UVMI_F32) {
    *(float4*)((float*)p + i) = float4{v[0], v[1], v[2], v[3]};
    *(float4*)((float*)p + i + 4) = float4{v[4], v[5], v[6], v[7]};
  } else {
    uint32_t r[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (DT == UVMI_BF16) r[j] = float2_to_bf16x2(v[2 * j], v[2 * j + 1]);
      else r[j] = (uint32_t)float_to_half_bits(v[2 * j]) | ((uint32_t)float_to_half_bits(v[2 * j + 1]) << 16);
    }
    *(uint4*)((uint16_t*)p + i) = uint4{r[0], r[1], r[2], r[3]};
  }
}

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
      float x0, x1;
      ld2<DT>(xin, src * d + 2 * pidx, x0, x1);
      if (MODE == 1) {
        float y0, y1;
        ld2<DT>(yin, r * d + 2 * pidx, y0, y1);
        x0 = round_t<DT>(a * x0 + b * y0);
        x1 = round_t<DT>(a * x1 + b * y1);
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
      if (xout) st2<DT>(xout, r * d + 2 * pidx, v0[i], v1[i]);
      st2<DT>(nout, r * d + 2 * pidx, v0[i] * rn, v1[i] * rn);
    }
  }
}

// ------------------------------------------------------------------------------------------------ qkv_post (hd = 64)
struct QkvArgs {
  const void* qkv; const void* xn; const void* ve_table; const float* ve_gate; const int64_t* tok;
  const int64_t* pos; const int64_t* rows; const int64_t* last_pos; const float* inv_freq;
  void* q_out; void* k_out; void* v_out;
  int8_t* k_cache; int8_t* v_cache; uint16_t* k_scale; uint16_t* v_scale;
  const float* gate_w; float* gate_out; float* vhat_out;
  int64_t scb, sch, scs, ssb, ssh;
  int64_t n, vocab;
  int H, KH, d, ve_ch, n_pairs, S, ring, has_ve, rope, q_dt, gate_ch;
  float eps, xsa_eps;
  const float* rope_tab; int rope_n;   // optional table of the rounded cos / sin per position (row: cos[n_pairs], sin[n_pairs])
  int64_t ld; int ext;                 // row pitch of qkv; gate logits read from columns W .. of the row instead of formed from xn
};

template <int DT>
__global__ __launch_bounds__(256) void qkv_post_kernel(QkvArgs A) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= A.n) return;
  const int W = (A.H + 2 * A.KH) * 64;
  const int64_t base = r * A.ld;
  const int64_t p = A.pos[r];
  const int np_ = A.n_pairs;
  const float* tab = A.rope_tab && p >= 0 && p < A.rope_n ? A.rope_tab + p * 2 * np_ : nullptr;   // (wave-uniform)
  // ---- queries: lane (hh = lane / 8, c = lane % 8) owns dims 8c..8c+7 of head 8*pass + hh
  {
    const int hh = lane >> 3, c = lane & 7;
    // RoPE angles of this lane's 8 dims (dims < 2 n_pairs rotate; dim j pairs with j +- n_pairs): one cos / sin per
    // frequency is computed by lanes 0..n_pairs-1 and fetched by shuffle
    float cs[8], sn[8];
    {
      float cl = 1.f, sl = 0.f;
      if (A.rope && lane < np_) {
        if (tab) {
          cl = tab[lane];
          sl = tab[np_ + lane];
        } else {
          const float th = (float)p * A.inv_freq[lane];
          cl = round_t<DT>(cosf(th));
          sl = round_t<DT>(sinf(th));
        }
      }
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int dim = 8 * c + j;
        const int src = A.rope ? dim % np_ : 0;
        const float cj = __shfl(cl, src, 64), sj = __shfl(sl, src, 64);
        const bool rot = A.rope && dim < 2 * np_;
        cs[j] = rot ? cj : 1.f;
        sn[j] = rot ? sj : 0.f;
      }
    }
    const int pl = np_ / 8;  // lane distance of the RoPE partner chunk (n_pairs is a multiple of 8, host-checked)
    for (int h0 = 0; h0 < A.H; h0 += 8) {
      const int h = h0 + hh;
      float x[8];
      if (h < A.H) ld8<DT>(A.qkv, base + h * 64 + 8 * c, x);
      else {
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = 0.f;
      }
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; j++) ss += x[j] * x[j];
      ss += lane_xor1(ss); ss += lane_xor2(ss); ss += lane_xor4(ss);
      const float rs = rsqrtf(ss * (1.0f / 64.0f) + A.eps);
#pragma unroll
      for (int j = 0; j < 8; j++) x[j] = round_t<DT>(x[j] * rs);
      if (A.rope) {
        const bool first = 8 * c < np_, rot = 8 * c < 2 * np_;
        float y[8];
#pragma unroll
        for (int j = 0; j < 8; j++) y[j] = pl == 2 ? lane_xor2(x[j]) : __shfl_xor(x[j], pl, 64);  // partner chunk: c <-> c ^ pl inside the head
        if (rot) {
#pragma unroll
          for (int j = 0; j < 8; j++) x[j] = rope_rot(x[j], y[j], cs[j], sn[j], first, [](float f) { return round_t<DT>(f); });
        }
      }
      if (h < A.H) {
        const int64_t o = (r * A.H + h) * 64 + 8 * c;
        if (A.q_dt == UVMI_BF16) st8<UVMI_BF16>(A.q_out, o, x); else if (A.q_dt == UVMI_F32) st8<UVMI_F32>(A.q_out, o, x); else st8<UVMI_F16>(A.q_out, o, x);
      }
    }
    // ---- per-head output gate 2 sigmoid(W_h . xn[:gate_ch]) for the attention epilogue (model.py:330-333)
    if (A.gate_out) {
      const int cpl = A.gate_ch / 8;  // channels per lane (a multiple of 8 when gate_ch % 64 == 0, else the scalar loop)
      for (int h0 = 0; h0 < A.H; h0 += 8) {
        const int h = h0 + hh;
        float dot = 0.f;
        if (A.ext) {   // the projection formed the logit (already rounded to the activation type)
          if (h < A.H && c == 0) dot = elem<DT>::ld(A.qkv, base + W + h);
        } else if (h < A.H) {
          if (cpl % 8 == 0 && (A.d % 8) == 0) {
            for (int j = 0; j < cpl; j += 8) {
              float xv[8];
              ld8<DT>(A.xn, r * A.d + c * cpl + j, xv);
              const float4 w0 = *(const float4*)(A.gate_w + h * A.gate_ch + c * cpl + j), w1 = *(const float4*)(A.gate_w + h * A.gate_ch + c * cpl + j + 4);
              dot += xv[0] * w0.x + xv[1] * w0.y + xv[2] * w0.z + xv[3] * w0.w + xv[4] * w1.x + xv[5] * w1.y + xv[6] * w1.z + xv[7] * w1.w;
            }
          } else {
            for (int j = 0; j < cpl; j++) dot += elem<DT>::ld(A.xn, r * A.d + c * cpl + j) * A.gate_w[h * A.gate_ch + c * cpl + j];
          }
        }
        dot += lane_xor1(dot); dot += lane_xor2(dot); dot += lane_xor4(dot);
        dot = round_t<DT>(dot);
        if (h < A.H && c == 0) A.gate_out[r * A.H + h] = round_t<DT>(2.0f * round_t<DT>(1.0f / (1.0f + __expf(-dot))));
      }
    }
  }
  // ---- keys / values per kv head: lane = dim
  float cs1 = 1.f, sn1 = 0.f;
  const bool rot1 = A.rope && lane < 2 * np_;
  if (rot1) {
    if (tab) {
      cs1 = tab[lane % np_];
      sn1 = tab[np_ + lane % np_];
    } else {
      const float th = (float)p * A.inv_freq[lane % np_];
      cs1 = round_t<DT>(cosf(th));
      sn1 = round_t<DT>(sinf(th));
    }
  }
  const int64_t row = A.rows ? A.rows[r] : r;
  const int64_t slot = A.ring ? (p % A.S) : p;
  bool wr = A.k_cache && row >= 0 && p >= 0 && slot < A.S;
  if (wr && A.ring && A.last_pos) wr = p > A.last_pos[r] - A.S;  // only the last S positions of a prompt survive in a ring
  for (int kh = 0; kh < A.KH; kh++) {
    float k = elem<DT>::ld(A.qkv, base + (A.H + kh) * 64 + lane);
    {
      const float rs = rsqrtf(wave_sum(k * k) * (1.0f / 64.0f) + A.eps);
      k = round_t<DT>(k * rs);
      if (A.rope) {
        const float other = np_ == 16 ? lane_xor16(k) : __shfl_xor(k, np_, 64);
        if (rot1) k = rope_rot(k, other, cs1, sn1, lane < np_, [](float f) { return round_t<DT>(f); });
      }
    }
    float v = elem<DT>::ld(A.qkv, base + (A.H + A.KH + kh) * 64 + lane);
    if (A.has_ve) {  // v += 2 sigmoid(W xn[:ve_ch]) * value_embed[tok]
      float dot = 0.f;
      if (A.ext) dot = elem<DT>::ld(A.qkv, base + W + A.H + kh);
      else {
        if (lane < A.ve_ch) dot = elem<DT>::ld(A.xn, r * A.d + lane) * A.ve_gate[kh * A.ve_ch + lane];
        dot = round_t<DT>(wave_sum(dot));
      }
      const float g = round_t<DT>(2.0f * round_t<DT>(1.0f / (1.0f + __expf(-dot))));
      int64_t t = A.tok[r];
      if (t < 0) t = 0;
      if (t >= A.vocab) t = A.vocab - 1;
      const float ve = elem<DT>::ld(A.ve_table, (t * A.KH + kh) * 64 + lane);
      v = ve_add(v, g, ve, [](float f) { return round_t<DT>(f); });
    }
    if (A.k_out) elem<DT>::st(A.k_out, (r * A.KH + kh) * 64 + lane, k);
    if (A.v_out) elem<DT>::st(A.v_out, (r * A.KH + kh) * 64 + lane, v);
    if (A.vhat_out) {  // v / max(|v|, eps) in fp32 for the XSA epilogue (model.py:327)
      const float nv = sqrtf(wave_sum(v * v));
      A.vhat_out[(r * A.KH + kh) * 64 + lane] = v / fmaxf(nv, A.xsa_eps);
    }
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

// The same post-processing for the engine's shape - 8 query heads on one kv head, 16 rotated pairs with the rotation
// table, gate logits formed by the projection (ext), q written in the activation type - with everything a row needs
// requested in two batches: first what depends on the row index alone (position, cache row, token, the row's q / k / v and
// logits), then what depends on those (the rotation table's row, the value embedding).  The general kernel above meets
// these loads one after the other between branches and loops, a chain of six memory latencies per row; the arithmetic,
// its order and its roundings are the same, so the two kernels agree bit for bit.
template <int DT>
__global__ __launch_bounds__(256) void qkv_post_fast_kernel(QkvArgs A) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= A.n) return;
  constexpr int W = 10 * 64;
  auto rnd = [](float f) { return round_t<DT>(f); };
  const int64_t base = r * A.ld;
  const int hh = lane >> 3, c = lane & 7;
  // ---- requests that depend on the row index alone
  const int64_t p = A.pos[r];
  const int64_t row = A.rows ? A.rows[r] : r;
  const int64_t lastp = A.last_pos ? A.last_pos[r] : 0;
  int64_t t = A.has_ve ? A.tok[r] : 0;
  float x[8];
  ld8<DT>(A.qkv, base + hh * 64 + 8 * c, x);
  float k = elem<DT>::ld(A.qkv, base + 8 * 64 + lane);
  float v = elem<DT>::ld(A.qkv, base + 9 * 64 + lane);
  const float glog = A.gate_out ? elem<DT>::ld(A.qkv, base + W + hh) : 0.f;
  const float vlog = A.has_ve ? elem<DT>::ld(A.qkv, base + W + 8) : 0.f;
  // ---- requests that depend on the position and the token
  const bool in_tab = p >= 0 && p < A.rope_n;   // (wave-uniform)
  const float* tab = A.rope_tab + (in_tab ? p : 0) * 32;
  float cs[8], sn[8], cs1 = 1.f, sn1 = 0.f;
  if (A.rope) {
    const float* tq = tab + 8 * (c & 1);   // dim 8 c + j turns by frequency (8 c + j) % 16
    const float4 c0 = *(const float4*)tq, c1 = *(const float4*)(tq + 4), s0 = *(const float4*)(tq + 16), s1 = *(const float4*)(tq + 20);
    cs[0] = c0.x; cs[1] = c0.y; cs[2] = c0.z; cs[3] = c0.w; cs[4] = c1.x; cs[5] = c1.y; cs[6] = c1.z; cs[7] = c1.w;
    sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
    cs1 = tab[lane & 15];
    sn1 = tab[16 + (lane & 15)];
  }
  if (t < 0) t = 0;
  if (t >= A.vocab) t = A.vocab - 1;
  const float ve = A.has_ve ? elem<DT>::ld(A.ve_table, t * 64 + lane) : 0.f;
  if (A.rope && !in_tab) {   // a position outside the table: the angles are formed here, as the general kernel does
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float th = (float)p * A.inv_freq[8 * (c & 1) + j];
      cs[j] = rnd(cosf(th));
      sn[j] = rnd(sinf(th));
    }
    const float th = (float)p * A.inv_freq[lane & 15];
    cs1 = rnd(cosf(th));
    sn1 = rnd(sinf(th));
  }
  // ---- queries: lane (hh, c) owns dims 8c..8c+7 of head hh
  {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) ss += x[j] * x[j];
    ss += lane_xor1(ss); ss += lane_xor2(ss); ss += lane_xor4(ss);
    const float rs = rsqrtf(ss * (1.0f / 64.0f) + A.eps);
#pragma unroll
    for (int j = 0; j < 8; j++) x[j] = rnd(x[j] * rs);
    if (A.rope) {
      float y[8];
#pragma unroll
      for (int j = 0; j < 8; j++) y[j] = lane_xor2(x[j]);   // partner chunk: c <-> c ^ 2 inside the head
      if (c < 4) {
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = rope_rot(x[j], y[j], cs[j], sn[j], c < 2, rnd);
      }
    }
    st8<DT>(A.q_out, (r * 8 + hh) * 64 + 8 * c, x);
    if (A.gate_out && c == 0) A.gate_out[r * 8 + hh] = rnd(2.0f * rnd(1.0f / (1.0f + __expf(-glog))));
  }
  // ---- key and value: lane = dim
  {
    const float rs = rsqrtf(wave_sum(k * k) * (1.0f / 64.0f) + A.eps);
    k = rnd(k * rs);
    if (A.rope) {
      const float other = lane_xor16(k);
      if (lane < 32) k = rope_rot(k, other, cs1, sn1, lane < 16, rnd);
    }
  }
  if (A.has_ve) {
    const float g = rnd(2.0f * rnd(1.0f / (1.0f + __expf(-vlog))));
    v = ve_add(v, g, ve, rnd);
  }
  if (A.k_out) elem<DT>::st(A.k_out, r * 64 + lane, k);
  if (A.v_out) elem<DT>::st(A.v_out, r * 64 + lane, v);
  if (A.vhat_out) {
    const float nv = sqrtf(wave_sum(v * v));
    A.vhat_out[r * 64 + lane] = v / fmaxf(nv, A.xsa_eps);
  }
  const int64_t slot = A.ring ? (p % A.S) : p;
  bool wr = A.k_cache && row >= 0 && p >= 0 && slot < A.S;
  if (wr && A.ring && A.last_pos) wr = p > lastp - A.S;
  if (wr) {
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
      caches[j][row * A.scb + slot * A.scs + lane] = (int8_t)(int)qv;
      if (lane == 0) scales[j][row * A.ssb + slot] = sb;
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
    const int64_t zi = (r * A.H + h) * 64 + lane;
    float z = A.z_dt == UVMI_BF16 ? elem<UVMI_BF16>::ld(A.z, zi) : (A.z_dt == UVMI_F32 ? elem<UVMI_F32>::ld(A.z, zi) : elem<UVMI_F16>::ld(A.z, zi));
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
// f % 8 == 0 (host-checked): thread t handles 8 consecutive columns of one row
template <int DT>
__global__ __launch_bounds__(256) void swiglu_kernel(const void* __restrict__ gu, void* __restrict__ out, int64_t rows, int f) {
  const int f8 = f / 8;
  const int64_t total = rows * f8;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / f8;
    const int j = (int)(i % f8) * 8;
    float g[8], u[8], o[8];
    ld8<DT>(gu, r * 2 * f + j, g);
    ld8<DT>(gu, r * 2 * f + f + j, u);
#pragma unroll
    for (int k = 0; k < 8; k++) o[k] = round_t<DT>(g[k] / (1.0f + __expf(-g[k]))) * u[k];
    st8<DT>(out, r * (int64_t)f + j, o);
  }
}

// SwiGLU on the gate/up product of the UN-normalised hidden h: the block's pre-norm is the row scale rn = rsqrt(mean(h^2) + eps)
// of that product, so the norm never needs a launch (or a buffer) of its own.  One workgroup per row; every wave sums
// the row's squares itself (d / 64 elements per lane), which needs no LDS and no barrier.  f % 8 == 0, d % 2 == 0.
template <int DT>
__global__ __launch_bounds__(256) void swiglu_norm_kernel(const void* __restrict__ gu, const void* __restrict__ h, void* __restrict__ out, int f,
                                                          int d, float eps) {
  const int64_t r = blockIdx.x;
  const int lane = threadIdx.x & 63;
  // the thread's first 8 gate / up columns are requested before the row's squares, so that both round trips to memory
  // overlap (f <= 2048: the only ones)
  int j = threadIdx.x * 8;
  float g[8], u[8], o[8];
  if (j < f) {
    ld8<DT>(gu, r * 2 * f + j, g);
    ld8<DT>(gu, r * 2 * f + f + j, u);
  }
  float ss = 0.f;
  for (int i = 2 * lane; i < d; i += 128) {
    float a, b;
    ld2<DT>(h, r * d + i, a, b);
    ss = fmaf(a, a, ss);
    ss = fmaf(b, b, ss);
  }
  const float rn = rsqrtf(wave_sum(ss) / (float)d + eps);
  while (j < f) {
    if (DT == UVMI_BF16) {
      // pairs share a conversion, and silu divides through the hardware reciprocal (1 ulp in fp32, before the rounding
      // to bf16): a third fewer instructions in a launch that is bound by them
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        const uint32_t gw = float2_to_bf16x2(g[k] * rn, g[k + 1] * rn), uw = float2_to_bf16x2(u[k] * rn, u[k + 1] * rn);
        const float g0 = __uint_as_float(gw << 16), g1 = __uint_as_float(gw & 0xffff0000u);
        const float s0 = g0 * __builtin_amdgcn_rcpf(1.0f + __expf(-g0)), s1 = g1 * __builtin_amdgcn_rcpf(1.0f + __expf(-g1));
        const uint32_t sw = float2_to_bf16x2(s0, s1);
        o[k] = __uint_as_float(sw << 16) * __uint_as_float(uw << 16);
        o[k + 1] = __uint_as_float(sw & 0xffff0000u) * __uint_as_float(uw & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; k++) {
        const float gv = round_t<DT>(g[k] * rn), uv = round_t<DT>(u[k] * rn);
        o[k] = round_t<DT>(gv / (1.0f + __expf(-gv))) * uv;
      }
    }
    st8<DT>(out, r * (int64_t)f + j, o);
    j += 256 * 8;
    if (j < f) {
      ld8<DT>(gu, r * 2 * f + j, g);
      ld8<DT>(gu, r * 2 * f + f + j, u);
    }
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
  UVMI_REQUIRE(is_float_dtype(a->dtype) && is_float_dtype(a->q_dtype), UVMI_EINVAL, "uvmi_qkv_post: bad dtype");
  UVMI_REQUIRE(a->n >= 0 && a->H > 0 && a->KH > 0 && a->H % a->KH == 0, UVMI_EINVAL, "uvmi_qkv_post: bad sizes");
  UVMI_REQUIRE(!a->rope || (a->inv_freq && a->n_pairs >= 8 && a->n_pairs <= 32 && (a->n_pairs & (a->n_pairs - 1)) == 0), UVMI_EUNSUPPORTED,
               "uvmi_qkv_post: rope needs inv_freq and 8, 16 or 32 rotated pairs");
  UVMI_REQUIRE(!a->gate_out || a->ext_logits || (a->gate_w && a->xn && a->gate_ch > 0 && a->gate_ch % 8 == 0 && a->gate_ch <= a->d), UVMI_EINVAL,
               "uvmi_qkv_post: gate_out needs gate_w, xn and a gate_ch that is a multiple of 8 (or ext_logits)");
  const int64_t qkv_w = (int64_t)(a->H + 2 * a->KH) * a->hd;
  UVMI_REQUIRE(a->qkv_ld == 0 || a->qkv_ld >= qkv_w, UVMI_EINVAL, "uvmi_qkv_post: qkv_ld below the row width");
  UVMI_REQUIRE(a->qkv_ld % 8 == 0, UVMI_EUNSUPPORTED, "uvmi_qkv_post: qkv_ld must be a multiple of 8 (16-byte rows)");
  UVMI_REQUIRE(!a->ext_logits || a->qkv_ld >= qkv_w + a->H + a->KH, UVMI_EINVAL,
               "uvmi_qkv_post: ext_logits needs a row pitch that holds the H + KH logits behind q, k, v");
  UVMI_REQUIRE(((uintptr_t)a->qkv % 16) == 0 && ((uintptr_t)a->q_out % 16) == 0, UVMI_EUNSUPPORTED, "uvmi_qkv_post: qkv and q_out must be 16-byte aligned");
  UVMI_REQUIRE(!a->has_ve || (a->ve_table && a->tok && a->vocab > 0 && (a->ext_logits || (a->xn && a->ve_gate && a->ve_ch > 0 && a->ve_ch <= 64))), UVMI_EINVAL,
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
  A.gate_w = a->gate_w; A.gate_out = a->gate_out; A.vhat_out = a->vhat_out; A.gate_ch = a->gate_ch; A.xsa_eps = a->xsa_eps;
  A.rope_tab = a->rope && a->rope_positions > 0 ? a->rope_table : nullptr;
  A.rope_n = a->rope_positions;
  A.ld = a->qkv_ld ? a->qkv_ld : qkv_w;
  A.ext = a->ext_logits != 0;
  const dim3 grid((unsigned)((a->n + 3) / 4)), blk(256);
  const bool fast = (a->dtype == UVMI_F16 || a->dtype == UVMI_BF16) && a->q_dtype == a->dtype && a->H == 8 && a->KH == 1 && A.ext &&
                    (!a->rope || (a->n_pairs == 16 && A.rope_tab && ((uintptr_t)A.rope_tab % 16) == 0));
  if (fast) {
    if (a->dtype == UVMI_F16) hipLaunchKernelGGL((qkv_post_fast_kernel<UVMI_F16>), grid, blk, 0, (hipStream_t)stream, A);
    else hipLaunchKernelGGL((qkv_post_fast_kernel<UVMI_BF16>), grid, blk, 0, (hipStream_t)stream, A);
  } else {
    dispatch_dt(a->dtype, [&](auto DT) { hipLaunchKernelGGL((qkv_post_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, A); });
  }
  UVMI_CHECK_LAUNCH("uvmi_qkv_post");
  return UVMI_OK;
}

// cos / sin of position * inv_freq per frequency, rounded to the activation type as the rotation applies them
// (round_t(cosf(th)) above), as an fp32 table: row p holds cos[0..n_pairs) then sin[0..n_pairs)
template <int DT>
__global__ __launch_bounds__(256) void rope_table_kernel(const float* __restrict__ inv_freq, int n_pairs, int64_t n_pos, float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_pos * n_pairs) return;
  const int64_t p = i / n_pairs;
  const int j = (int)(i % n_pairs);
  const float th = (float)p * inv_freq[j];
  out[p * 2 * n_pairs + j] = round_t<DT>(cosf(th));
  out[p * 2 * n_pairs + n_pairs + j] = round_t<DT>(sinf(th));
}

extern "C" int uvmi_rope_table(const float* inv_freq, int n_pairs, int64_t n_positions, int round_dtype, float* out, void* stream) {
  UVMI_REQUIRE(inv_freq && out, UVMI_EINVAL, "uvmi_rope_table: null pointer");
  UVMI_REQUIRE(n_pairs > 0 && n_positions >= 0 && is_float_dtype(round_dtype), UVMI_EINVAL, "uvmi_rope_table: bad arguments");
  if (n_positions == 0) return UVMI_OK;
  const dim3 grid((unsigned)((n_positions * n_pairs + 255) / 256)), blk(256);
  dispatch_dt(round_dtype, [&](auto DT) {
    hipLaunchKernelGGL((rope_table_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, inv_freq, n_pairs, n_positions, out);
  });
  UVMI_CHECK_LAUNCH("uvmi_rope_table");
  return UVMI_OK;
}

extern "C" int uvmi_attn_post(const void* z, int z_dtype, const void* v, const void* xn, int dtype, const float* gate_w, const float* xsa,
                              float xsa_eps, int64_t n, int H, int KH, int hd, int d, int gate_ch, void* out, void* stream) {
  UVMI_REQUIRE(z && out, UVMI_EINVAL, "uvmi_attn_post: null pointer");
  UVMI_REQUIRE(hd == 64, UVMI_EUNSUPPORTED, "uvmi_attn_post: head_dim %d (only 64)", hd);
  UVMI_REQUIRE(is_float_dtype(dtype) && is_float_dtype(z_dtype), UVMI_EINVAL, "uvmi_attn_post: bad dtype");
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
  UVMI_REQUIRE(f % 8 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0, UVMI_EUNSUPPORTED, "uvmi_swiglu: f %% 8 and 16-byte alignment needed");
  if (rows == 0) return UVMI_OK;
  int64_t blocks = (rows * (f / 8) + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  const dim3 grid((unsigned)blocks), blk(256);
  dispatch_dt(dtype, [&](auto DT) { hipLaunchKernelGGL((swiglu_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, gu, out, rows, f); });
  UVMI_CHECK_LAUNCH("uvmi_swiglu");
  return UVMI_OK;
}

extern "C" int uvmi_swiglu_norm(const void* gu, const void* h, int dtype, int64_t rows, int f, int d, float eps, void* out, void* stream) {
  UVMI_REQUIRE(gu && h && out, UVMI_EINVAL, "uvmi_swiglu_norm: null pointer");
  UVMI_REQUIRE(is_float_dtype(dtype) && rows >= 0 && rows <= 0x7fffffff && f > 0 && d > 0 && eps >= 0.f, UVMI_EINVAL, "uvmi_swiglu_norm: bad arguments");
  UVMI_REQUIRE(f % 8 == 0 && d % 2 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)h % 8) == 0, UVMI_EUNSUPPORTED,
               "uvmi_swiglu_norm: f %% 8, d %% 2 and 16-byte alignment needed");
  if (rows == 0) return UVMI_OK;
  const dim3 grid((unsigned)rows), blk(256);
  dispatch_dt(dtype, [&](auto DT) { hipLaunchKernelGGL((swiglu_norm_kernel<decltype(DT)::value>), grid, blk, 0, (hipStream_t)stream, gu, h, out, f, d, eps); });
  UVMI_CHECK_LAUNCH("uvmi_swiglu_norm");
  return UVMI_OK;
}
