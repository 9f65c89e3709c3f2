// Ragged single-query (decode) attention over a slot-indexed KV cache, split-K with an fp32 combine.
//
// Contract (ultraviolet/kernels/decode_attn.py:193-230 of the reference): row b attends the absolute positions
// lo_b..pos_b, lo_b = max(starts_b, pos_b - window + 1, 0); position t lives in slot t (linear) or t % S (ring);
// int8 caches carry one fp16 scale per (row, kv head, slot): the K scale multiplies the score column, the V scale
// multiplies the probability before P.V, and the softmax denominator is summed before that scaling.
//
// Two kernels:
//   * attn_mfma_i8_hd64: head_dim 64, int8 cache, up to 8 query heads per kv head (UV-50M: G = 8, KH = 1).  One
//     wave64 per (row, kv head, split).  HBM-bound (132 B per key), but at 2048 FLOP per key it only stays
//     HBM-bound if the contraction runs on MFMA and the int8 -> fp16 conversion is a handful of VALU ops per dword:
//       - a super-tile is 32 keys: two 16-key streams A and B.  S^T = [K_A | K_B] . blockdiag(Q^T, Q^T) is four
//         v_mfma_f32_16x16x32_f16; accumulator column n < 8 is (stream A, head n), n >= 8 is (stream B, head n-8),
//         so all 64 lanes of the 16x16 tile do useful softmax work although only 8 heads exist;
//       - a lane of the accumulator layout holds 4 consecutive keys of one (stream, head) column, which is exactly
//         the B-operand layout of the P.V MFMA (O^T = V^T . P^T) when contraction slot 8g+j is key 4g+j of stream
//         A and 8g+4+j is key 4g+j of stream B: probabilities never move between lanes;
//       - K rows are read as one 16-byte load per lane (lane = key m, bytes 16g..16g+15), V as dwords
//         (lane = bytes 4m..4m+3 of 8 keys), both fully coalesced over 64-byte rows; int8 is turned into fp16 with
//         v_perm_b32 against 0x64 bytes (fp16 0x64uu = 1024 + u, u = x ^ 0x80 = x + 128): K keeps the +1152 bias,
//         which is cancelled by the accumulator's initial value -1152 * sum(q), V removes it with a packed add;
//       - online softmax per (stream, head) column; the two streams are merged once at the end.
//   * attn_generic: any head_dim <= 256, G <= 16, int8 / fp16 / bf16 caches, arbitrary alignment: plain fp32 VALU.
//
// Split partials (acc, m, l) go to a caller-provided workspace; attn_combine merges them.
#include "common.h"

namespace uvmi {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr float LOG2E = 1.4426950408889634f;

struct AttnParams {
  const void* q; const void* kc; const void* vc; const void* ks; const void* vs;
  const void* pos; const void* starts;
  void* out; float* ws_o; float* ws_m; float* ws_l;
  int64_t sqb, sqh, skb, skh, sks, svb, svh, svs, ssb, ssh, stb, sth, sob, soh;
  int B, H, KH, G, S, hd, window, ring, splits, idx64;
  int64_t n_items;
  float scale_log2;
};

// Row range and this split's chunk.  Chunks are multiples of 32 keys starting at lo rounded down to 32, so a
// 16-key tile never straddles two splits and tiles stay aligned to the slot grid.
struct Chunk { int lo, p, s0, s1; };
__device__ __forceinline__ Chunk split_range(const AttnParams& P, int b, int sid) {
  int p = (int)load_index(P.pos, P.idx64, b);
  int st = (int)load_index(P.starts, P.idx64, b);
  int lo = st > 0 ? st : 0;
  if (P.window > 0 && p - P.window + 1 > lo) lo = p - P.window + 1;
  Chunk c;
  c.lo = lo;
  c.p = p;
  int a0 = lo & ~31;
  int span = p + 1 - a0;
  if (span < 0) span = 0;
  int chunk = (((span + P.splits - 1) / P.splits) + 31) & ~31;
  c.s0 = a0 + sid * chunk;
  c.s1 = min(c.s0 + chunk, p + 1);
  return c;
}

// ---------------------------------------------------------------------------------------------------- MFMA kernel
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

template <typename T>
__device__ __forceinline__ T bitcast_h8(const uint32_t (&r)[4]) {
  T v;
  __builtin_memcpy(&v, r, 16);
  return v;
}

__device__ __forceinline__ float xmax16(float v) {  // max over lanes l, l^16 (rows of 16 lanes pairwise)
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xmax32(float v) {  // max over lanes l, l^32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xsum16(float v) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xsum32(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

struct Tile {         // one 32-key super-tile as loaded from HBM
  uint4 kA, kB;       // key m of stream A / B, bytes 16g..16g+15
  uint32_t vA[4], vB[4];  // keys 4g+j of stream A / B, bytes 4m..4m+3
  uint2 ksc, vsc;     // 4 fp16 scales of keys 4g..4g+3 of this lane's stream
};

template <int QDT, int ODT>
__global__ __launch_bounds__(256) void attn_mfma_i8_hd64(AttnParams P) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= P.n_items) return;
  const int sid = (int)(item % P.splits);
  const int64_t bk = item / P.splits;
  const int b = (int)(bk / P.KH), h = (int)(bk % P.KH);
  const int m = lane & 15, g = lane >> 4;  // also (n, g) of the accumulator layout
  const int strm = m >> 3, head = m & 7;
  const Chunk c = split_range(P, b, sid);
  const int G = P.G;

  // ---- Q^T operands: lane (n, g) holds q[head][16g + 8s + j]; fp16 (bf16 inputs are converted, exact for
  // 2^-14 <= |q| <= 65504)
  uint32_t qr[8];
  float qsum = 0.f;
  {
    const uint16_t* qp = (const uint16_t*)P.q + (int64_t)b * P.sqb + (int64_t)(h * G + head) * P.sqh + 16 * g;
    float qf[16];
    if (head < G) {
      uint4 w0 = *(const uint4*)qp, w1 = *(const uint4*)(qp + 8);
      const uint32_t w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
      for (int i = 0; i < 8; i++) {
        if (QDT == UVMI_BF16) {
          qf[2 * i] = __uint_as_float(w[i] << 16);
          qf[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        } else {
          qf[2 * i] = half_bits_to_float(w[i] & 0xffff);
          qf[2 * i + 1] = half_bits_to_float(w[i] >> 16);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; i++) qf[i] = 0.f;
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      uint16_t lo16 = float_to_half_bits(qf[2 * i]), hi16 = float_to_half_bits(qf[2 * i + 1]);
      qr[i] = (uint32_t)lo16 | ((uint32_t)hi16 << 16);
      qsum += half_bits_to_float(lo16) + half_bits_to_float(hi16);
    }
    // sum over the 4 lane groups -> sum over all 64 dims of this head
    qsum = xsum16(qsum);
    qsum = xsum32(qsum);
  }
  const uint32_t mA = strm == 0 ? 0xffffffffu : 0u, mB = ~mA;
  uint32_t qa0[4], qa1[4], qb0[4], qb1[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    qa0[i] = qr[i] & mA; qa1[i] = qr[4 + i] & mA;
    qb0[i] = qr[i] & mB; qb1[i] = qr[4 + i] & mB;
  }
  const h8 QA0 = bitcast_h8<h8>(qa0), QA1 = bitcast_h8<h8>(qa1), QB0 = bitcast_h8<h8>(qb0), QB1 = bitcast_h8<h8>(qb1);
  const float cinit = -1152.0f * qsum;

  // ---- state
  f4 O[4];
#pragma unroll
  for (int t = 0; t < 4; t++) O[t] = f4{0.f, 0.f, 0.f, 0.f};
  float mrun = -INFINITY, lrun = 0.f;

  const int lo_eff = max(c.lo, c.s0);
  const int8_t* kbase = (const int8_t*)P.kc + (int64_t)b * P.skb + (int64_t)h * P.skh;
  const int8_t* vbase = (const int8_t*)P.vc + (int64_t)b * P.svb + (int64_t)h * P.svh;
  const uint16_t* ksb = (const uint16_t*)P.ks + (int64_t)b * P.ssb + (int64_t)h * P.ssh;
  const uint16_t* vsb = (const uint16_t*)P.vs + (int64_t)b * P.stb + (int64_t)h * P.sth;
  const int S = P.S;
  const int smax = S - 1;

  auto slot_of = [&](int t) -> int {  // t is a multiple of 16 here; ring needs S % 16 == 0 (host-checked)
    if (P.ring) return t % S;
    return t;
  };
  auto load_tile = [&](int tb, Tile& T) {
    const int sa = slot_of(tb), sb2 = slot_of(tb + 16);
    // K: key m of each stream
    int ka = min(sa + m, smax), kb = min(sb2 + m, smax);
    T.kA = *(const uint4*)(kbase + (int64_t)ka * P.sks + 16 * g);
    T.kB = *(const uint4*)(kbase + (int64_t)kb * P.sks + 16 * g);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int va = min(sa + 4 * g + j, smax), vb = min(sb2 + 4 * g + j, smax);
      T.vA[j] = *(const uint32_t*)(vbase + (int64_t)va * P.svs + 4 * m);
      T.vB[j] = *(const uint32_t*)(vbase + (int64_t)vb * P.svs + 4 * m);
    }
    int ss = min((strm ? sb2 : sa) + 4 * g, S - 4);
    T.ksc = *(const uint2*)(ksb + ss);
    T.vsc = *(const uint2*)(vsb + ss);
  };

  if (c.s0 < c.s1) {
    Tile cur, nxt;
    load_tile(c.s0, cur);
    for (int tb = c.s0; tb < c.s1; tb += 32) {
      const bool more = tb + 32 < c.s1;
      if (more) load_tile(tb + 32, nxt);

      // ---- K -> fp16 (1024 + u), S^T = K . Q^T - 1152 sum(q)
      f4 acc = f4{cinit, cinit, cinit, cinit};
      {
        const uint32_t wa[4] = {cur.kA.x ^ 0x80808080u, cur.kA.y ^ 0x80808080u, cur.kA.z ^ 0x80808080u, cur.kA.w ^ 0x80808080u};
        const uint32_t wb[4] = {cur.kB.x ^ 0x80808080u, cur.kB.y ^ 0x80808080u, cur.kB.z ^ 0x80808080u, cur.kB.w ^ 0x80808080u};
        uint32_t a0[4], a1[4], b0[4], b1[4];
#pragma unroll
        for (int i = 0; i < 2; i++) {
          a0[2 * i] = perm(0x64646464u, wa[i], 0x04010400u);     a0[2 * i + 1] = perm(0x64646464u, wa[i], 0x04030402u);
          a1[2 * i] = perm(0x64646464u, wa[2 + i], 0x04010400u); a1[2 * i + 1] = perm(0x64646464u, wa[2 + i], 0x04030402u);
          b0[2 * i] = perm(0x64646464u, wb[i], 0x04010400u);     b0[2 * i + 1] = perm(0x64646464u, wb[i], 0x04030402u);
          b1[2 * i] = perm(0x64646464u, wb[2 + i], 0x04010400u); b1[2 * i + 1] = perm(0x64646464u, wb[2 + i], 0x04030402u);
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast_h8<h8>(a0), QA0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast_h8<h8>(a1), QA1, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast_h8<h8>(b0), QB0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast_h8<h8>(b1), QB1, acc, 0, 0, 0);
      }
      // ---- scores in the exp2 domain: s_i = acc_i * kscale_i * scale * log2(e); lane (n, g) key = base + 4g + i
      float s[4];
      {
        const float k0 = half_bits_to_float(cur.ksc.x & 0xffff), k1 = half_bits_to_float(cur.ksc.x >> 16);
        const float k2 = half_bits_to_float(cur.ksc.y & 0xffff), k3 = half_bits_to_float(cur.ksc.y >> 16);
        s[0] = acc[0] * (k0 * P.scale_log2); s[1] = acc[1] * (k1 * P.scale_log2);
        s[2] = acc[2] * (k2 * P.scale_log2); s[3] = acc[3] * (k3 * P.scale_log2);
      }
      float vsf[4] = {half_bits_to_float(cur.vsc.x & 0xffff), half_bits_to_float(cur.vsc.x >> 16),
                      half_bits_to_float(cur.vsc.y & 0xffff), half_bits_to_float(cur.vsc.y >> 16)};
      if (tb < lo_eff || tb + 32 > c.s1) {  // edge tiles: mask keys outside [lo_eff, s1); their (possibly stale,
        const int t0 = tb + 16 * strm + 4 * g;  // non-finite) V scale must not meet p = 0
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (t0 + i < lo_eff || t0 + i >= c.s1) { s[i] = -INFINITY; vsf[i] = 0.f; }
      }
      float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
      mx = xmax16(mx);
      mx = xmax32(mx);
      const float mnew = fmaxf(mrun, mx);
      const float msafe = mnew == -INFINITY ? 0.f : mnew;
      const float alpha = __builtin_amdgcn_exp2f(mrun - msafe);
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; i++) p[i] = __builtin_amdgcn_exp2f(s[i] - msafe);
      lrun = lrun * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
      mrun = mnew;
      // ---- P' = p * vscale -> fp16 pairs in this stream's half of the contraction slots
      h8 PB;
      {
        h2 p01 = h2{(_Float16)(p[0] * vsf[0]), (_Float16)(p[1] * vsf[1])};
        h2 p23 = h2{(_Float16)(p[2] * vsf[2]), (_Float16)(p[3] * vsf[3])};
        uint32_t u01, u23;
        __builtin_memcpy(&u01, &p01, 4);
        __builtin_memcpy(&u23, &p23, 4);
        const uint32_t r[4] = {u01 & mA, u23 & mA, u01 & mB, u23 & mB};
        PB = bitcast_h8<h8>(r);
      }
      // ---- O^T = alpha * O^T + V^T . P'^T ; tile t, row m of the A operand is head dim 4m + t
#pragma unroll
      for (int t = 0; t < 4; t++) {
        O[t] *= alpha;
      }
      {
        uint32_t xa[4], xb[4];
#pragma unroll
        for (int j = 0; j < 4; j++) { xa[j] = cur.vA[j] ^ 0x80808080u; xb[j] = cur.vB[j] ^ 0x80808080u; }
#pragma unroll
        for (int t = 0; t < 4; t++) {
          const uint32_t sel = 0x0c000c00u | ((4u + t) << 16) | (uint32_t)t;  // [0, S0.byte t, 0, S1.byte t]
          uint32_t r[4];
          r[0] = perm(xa[1], xa[0], sel) | 0x64006400u;
          r[1] = perm(xa[3], xa[2], sel) | 0x64006400u;
          r[2] = perm(xb[1], xb[0], sel) | 0x64006400u;
          r[3] = perm(xb[3], xb[2], sel) | 0x64006400u;
          h8 va = bitcast_h8<h8>(r);
          va = va - (h8)((_Float16)1152.0f);
          O[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, PB, O[t], 0, 0, 0);
        }
      }
      if (more) cur = nxt;
    }
  }

  // ---- reduce l over the 4 lane groups, merge stream B into stream A (lanes n and n+8 of each 16-lane row)
  lrun = xsum16(lrun);
  lrun = xsum32(lrun);
  const float m_o = __shfl_xor(mrun, 8, 64), l_o = __shfl_xor(lrun, 8, 64);
  const float mm = fmaxf(mrun, m_o);
  const float ms = mm == -INFINITY ? 0.f : mm;
  const float w_s = __builtin_amdgcn_exp2f(mrun - ms), w_o = __builtin_amdgcn_exp2f(m_o - ms);
  const float lm = lrun * w_s + l_o * w_o;
  float o[16];  // head dims 16g .. 16g+15: O[t][i] is dim 16g + 4i + t
#pragma unroll
  for (int t = 0; t < 4; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float mine = O[t][i];
      const float oth = __shfl_xor(mine, 8, 64);
      o[4 * i + t] = mine * w_s + oth * w_o;
    }
  if (strm == 0 && head < G) {
    if (P.splits == 1) {
      const float inv = lm > 0.f ? 1.0f / lm : 0.f;
      const int64_t off = (int64_t)b * P.sob + (int64_t)(h * G + head) * P.soh + 16 * g;
      if (ODT == UVMI_F32) {
        float* op = (float*)P.out + off;
#pragma unroll
        for (int i = 0; i < 4; i++) *(float4*)(op + 4 * i) = float4{o[4 * i] * inv, o[4 * i + 1] * inv, o[4 * i + 2] * inv, o[4 * i + 3] * inv};
      } else {
        uint32_t w[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const float x0 = o[2 * i] * inv, x1 = o[2 * i + 1] * inv;
          const uint32_t l16 = ODT == UVMI_BF16 ? float_to_bf16(x0) : float_to_half_bits(x0);
          const uint32_t h16 = ODT == UVMI_BF16 ? float_to_bf16(x1) : float_to_half_bits(x1);
          w[i] = l16 | (h16 << 16);
        }
        uint16_t* op = (uint16_t*)P.out + off;
        *(uint4*)op = uint4{w[0], w[1], w[2], w[3]};
        *(uint4*)(op + 8) = uint4{w[4], w[5], w[6], w[7]};
      }
    } else {
      const int64_t r = item * G + head;
      float* op = P.ws_o + r * 64 + 16 * g;
#pragma unroll
      for (int i = 0; i < 4; i++) *(float4*)(op + 4 * i) = float4{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
      if (g == 0) {
        P.ws_m[r] = mm;
        P.ws_l[r] = lm;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------- generic kernel
// One wave per (row, kv head, split).  Lanes own keys for Q.K (64 keys per tile), then own head dims for P.V.
template <int KVDT>
__device__ __forceinline__ float kv_ld(const void* p, int64_t i) {
  if (KVDT == UVMI_I8) return (float)((const int8_t*)p)[i];
  if (KVDT == UVMI_F16) return half_bits_to_float(((const uint16_t*)p)[i]);
  return bf16_to_float(((const uint16_t*)p)[i]);
}

template <int QDT, int KVDT, int ODT>
__global__ __launch_bounds__(64) void attn_generic(AttnParams P) {
  extern __shared__ float smem[];  // q[G][hd] then pbuf[G][64]
  const int lane = threadIdx.x;
  const int64_t item = blockIdx.x;
  const int sid = (int)(item % P.splits);
  const int64_t bk = item / P.splits;
  const int b = (int)(bk / P.KH), h = (int)(bk % P.KH);
  const int G = P.G, hd = P.hd;
  float* qs = smem;
  float* pb = smem + G * hd;
  for (int i = lane; i < G * hd; i += 64) {
    int gi = i / hd, d = i % hd;
    qs[i] = elem<QDT>::ld(P.q, (int64_t)b * P.sqb + (int64_t)(h * G + gi) * P.sqh + d);
  }
  __syncthreads();
  const Chunk c = split_range(P, b, sid);
  const int lo_eff = max(c.lo, c.s0);
  constexpr int MAXG = 16, MAXD = 4;  // hd <= 256
  float mrun[MAXG], lrun[MAXG], acc[MAXG][MAXD];
#pragma unroll
  for (int gi = 0; gi < MAXG; gi++) {
    mrun[gi] = -INFINITY;
    lrun[gi] = 0.f;
#pragma unroll
    for (int j = 0; j < MAXD; j++) acc[gi][j] = 0.f;
  }
  const int64_t kb0 = (int64_t)b * P.skb + (int64_t)h * P.skh, vb0 = (int64_t)b * P.svb + (int64_t)h * P.svh;
  const int64_t ks0 = (int64_t)b * P.ssb + (int64_t)h * P.ssh, vs0 = (int64_t)b * P.stb + (int64_t)h * P.sth;
  for (int tb = lo_eff; tb < c.s1; tb += 64) {
    const int t = tb + lane;
    const bool valid = t < c.s1;
    const int slot = valid ? (P.ring ? t % P.S : min(t, P.S - 1)) : 0;
    float sc[MAXG];
#pragma unroll
    for (int gi = 0; gi < MAXG; gi++) sc[gi] = 0.f;
    if (valid) {
      for (int d = 0; d < hd; d++) {
        const float kv = kv_ld<KVDT>(P.kc, kb0 + (int64_t)slot * P.sks + d);
#pragma unroll
        for (int gi = 0; gi < MAXG; gi++)
          if (gi < G) sc[gi] += qs[gi * hd + d] * kv;
      }
    }
    float kscale = 1.f, vscale = 1.f;
    if (KVDT == UVMI_I8 && valid) {
      kscale = half_bits_to_float(((const uint16_t*)P.ks)[ks0 + slot]);
      vscale = half_bits_to_float(((const uint16_t*)P.vs)[vs0 + slot]);
    }
    __syncthreads();  // previous tile's pb fully consumed
#pragma unroll
    for (int gi = 0; gi < MAXG; gi++) {
      if (gi < G) {
        const float s = valid ? sc[gi] * kscale * P.scale_log2 : -INFINITY;
        const float mx = wave_max(s);
        const float mnew = fmaxf(mrun[gi], mx);
        const float ms = mnew == -INFINITY ? 0.f : mnew;
        const float alpha = exp2f(mrun[gi] - ms);
        const float p = exp2f(s - ms);
        lrun[gi] = lrun[gi] * alpha + wave_sum(p);
        mrun[gi] = mnew;
#pragma unroll
        for (int j = 0; j < MAXD; j++) acc[gi][j] *= alpha;
        pb[gi * 64 + lane] = p * vscale;
      }
    }
    __syncthreads();
    const int nk = min(64, c.s1 - tb);
    for (int j = 0; j < nk; j++) {
      const int tj = tb + j;
      const int sj = P.ring ? tj % P.S : min(tj, P.S - 1);
#pragma unroll
      for (int dj = 0; dj < MAXD; dj++) {
        const int d = lane + 64 * dj;
        if (d < hd) {
          const float vv = kv_ld<KVDT>(P.vc, vb0 + (int64_t)sj * P.svs + d);
#pragma unroll
          for (int gi = 0; gi < MAXG; gi++)
            if (gi < G) acc[gi][dj] += pb[gi * 64 + j] * vv;
        }
      }
    }
  }
#pragma unroll
  for (int gi = 0; gi < MAXG; gi++) {
    if (gi < G) {
#pragma unroll
      for (int dj = 0; dj < MAXD; dj++) {
        const int d = lane + 64 * dj;
        if (d < hd) {
          if (P.splits == 1) {
            const float v = lrun[gi] > 0.f ? acc[gi][dj] / lrun[gi] : 0.f;
            elem<ODT>::st(P.out, (int64_t)b * P.sob + (int64_t)(h * G + gi) * P.soh + d, v);
          } else {
            P.ws_o[(item * G + gi) * hd + d] = acc[gi][dj];
          }
        }
      }
      if (P.splits > 1 && lane == 0) {
        P.ws_m[item * G + gi] = mrun[gi];
        P.ws_l[item * G + gi] = lrun[gi];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------- combine
// One wave per (row, kv head, query head): out = sum_s w_s o_s / sum_s w_s l_s, w_s = 2^(m_s - max m); empty splits
// (m = -inf) get weight 0 (decode_attn.py:96-115 of the reference).
template <int ODT>
__global__ __launch_bounds__(256) void attn_combine(AttnParams P) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (bk * G + gi)
  if (r >= (int64_t)P.B * P.KH * P.G) return;
  const int64_t bk = r / P.G;
  const int gi = (int)(r % P.G);
  const int b = (int)(bk / P.KH), h = (int)(bk % P.KH);
  float mx = -INFINITY;
  for (int s = 0; s < P.splits; s++) mx = fmaxf(mx, P.ws_m[(bk * P.splits + s) * P.G + gi]);
  const float ms = mx == -INFINITY ? 0.f : mx;
  float den = 0.f;
  float num[4] = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < P.splits; s++) {
    const int64_t pr = (bk * P.splits + s) * P.G + gi;
    const float m = P.ws_m[pr];
    if (m == -INFINITY) continue;
    const float w = exp2f(m - ms);
    den += w * P.ws_l[pr];
#pragma unroll
    for (int dj = 0; dj < 4; dj++) {
      const int d = lane + 64 * dj;
      if (d < P.hd) num[dj] += w * P.ws_o[pr * P.hd + d];
    }
  }
  const float inv = den > 0.f ? 1.0f / den : 0.f;
#pragma unroll
  for (int dj = 0; dj < 4; dj++) {
    const int d = lane + 64 * dj;
    if (d < P.hd) elem<ODT>::st(P.out, (int64_t)b * P.sob + (int64_t)(h * P.G + gi) * P.soh + d, num[dj] * inv);
  }
}

// ---------------------------------------------------------------------------------------------------- host side
static int check_common(const uvmi_attn_args* a) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_decode_attn: null args");
  UVMI_REQUIRE(a->q && a->k_cache && a->v_cache && a->pos && a->starts && a->out, UVMI_EINVAL, "uvmi_decode_attn: null pointer");
  UVMI_REQUIRE(a->B >= 0 && a->H > 0 && a->KH > 0 && a->S > 0 && a->hd > 0, UVMI_EINVAL, "uvmi_decode_attn: bad sizes");
  UVMI_REQUIRE(a->H % a->KH == 0, UVMI_EINVAL, "uvmi_decode_attn: H=%d is not a multiple of KH=%d", a->H, a->KH);
  UVMI_REQUIRE(a->q_dtype == UVMI_F16 || a->q_dtype == UVMI_BF16, UVMI_EUNSUPPORTED, "uvmi_decode_attn: q must be F16 or BF16");
  UVMI_REQUIRE(a->out_dtype == UVMI_F16 || a->out_dtype == UVMI_BF16 || a->out_dtype == UVMI_F32, UVMI_EUNSUPPORTED,
               "uvmi_decode_attn: out must be F16, BF16 or F32");
  UVMI_REQUIRE(a->kv_dtype == UVMI_I8 || a->kv_dtype == UVMI_F16 || a->kv_dtype == UVMI_BF16, UVMI_EUNSUPPORTED,
               "uvmi_decode_attn: cache must be I8, F16 or BF16");
  UVMI_REQUIRE(a->kv_dtype != UVMI_I8 || (a->k_scale && a->v_scale), UVMI_EINVAL, "uvmi_decode_attn: int8 cache needs k_scale and v_scale");
  UVMI_REQUIRE(a->idx_dtype == UVMI_I64 || a->idx_dtype == UVMI_I32, UVMI_EINVAL, "uvmi_decode_attn: pos/starts must be I32 or I64");
  UVMI_REQUIRE(a->num_splits >= 1 && a->num_splits <= 1024, UVMI_EINVAL, "uvmi_decode_attn: num_splits=%d out of range", a->num_splits);
  UVMI_REQUIRE(a->window >= 0, UVMI_EINVAL, "uvmi_decode_attn: negative window");
  UVMI_REQUIRE(a->hd <= 256 && a->H / a->KH <= 16, UVMI_EUNSUPPORTED, "uvmi_decode_attn: head_dim %d / group %d beyond 256 / 16", a->hd,
               a->H / a->KH);
  return UVMI_OK;
}

static bool mfma_ok(const uvmi_attn_args* a) {
  const int G = a->H / a->KH;
  if (a->hd != 64 || a->kv_dtype != UVMI_I8 || G > 8) return false;
  if (a->ring && (a->S % 16 != 0)) return false;
  if (a->S % 4 != 0 || a->S < 4) return false;
  auto al = [](const void* p, int n) { return ((uintptr_t)p % n) == 0; };
  if (!al(a->q, 16) || a->sqb % 8 || a->sqh % 8) return false;
  if (!al(a->k_cache, 16) || a->skb % 16 || a->skh % 16 || a->sks % 16) return false;
  if (!al(a->v_cache, 4) || a->svb % 4 || a->svh % 4 || a->svs % 4) return false;
  if (!al(a->k_scale, 8) || a->ssb % 4 || a->ssh % 4) return false;
  if (!al(a->v_scale, 8) || a->stb % 4 || a->sth % 4) return false;
  const int ob = a->out_dtype == UVMI_F32 ? 4 : 2;
  if (!al(a->out, 16) || (a->sob * ob) % 16 || (a->soh * ob) % 16) return false;
  return true;
}

}  // namespace uvmi

using namespace uvmi;

extern "C" size_t uvmi_decode_attn_workspace_bytes(int B, int H, int KH, int hd, int num_splits) {
  if (num_splits <= 1 || B <= 0 || H <= 0 || KH <= 0 || hd <= 0) return 0;
  const size_t rows = (size_t)B * H * num_splits;  // B*KH*splits*G
  return rows * (size_t)hd * 4 + 2 * rows * 4 + 256;
}

extern "C" int uvmi_default_splits(int64_t n_bk, int ctx, int n_cus) {
  if (n_cus <= 0) n_cus = uvmi_device_cus();
  if (n_cus <= 0) n_cus = 256;
  if (n_bk < 1) n_bk = 1;
  // 16 resident waves per CU hide HBM latency with one 4 KB super-tile in flight each; chunks stay >= 64 keys
  const int64_t want = (16LL * n_cus + n_bk - 1) / n_bk;
  int64_t cap = ctx / 64;
  if (cap < 1) cap = 1;
  int64_t s = want < cap ? want : cap;
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

extern "C" int uvmi_decode_attn_path(const uvmi_attn_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  return mfma_ok(a) ? 1 : 0;
}

extern "C" int uvmi_decode_attn(const uvmi_attn_args* a, void* stream) {
  int rc = check_common(a);
  if (rc) return rc;
  if (a->B == 0) return UVMI_OK;
  hipStream_t st = (hipStream_t)stream;
  AttnParams P;
  P.q = a->q; P.kc = a->k_cache; P.vc = a->v_cache; P.ks = a->k_scale; P.vs = a->v_scale;
  P.pos = a->pos; P.starts = a->starts; P.out = a->out;
  P.sqb = a->sqb; P.sqh = a->sqh; P.skb = a->skb; P.skh = a->skh; P.sks = a->sks; P.svb = a->svb; P.svh = a->svh; P.svs = a->svs;
  P.ssb = a->ssb; P.ssh = a->ssh; P.stb = a->stb; P.sth = a->sth; P.sob = a->sob; P.soh = a->soh;
  P.B = a->B; P.H = a->H; P.KH = a->KH; P.G = a->H / a->KH; P.S = a->S; P.hd = a->hd;
  P.window = a->window; P.ring = a->ring ? 1 : 0; P.splits = a->num_splits; P.idx64 = a->idx_dtype == UVMI_I64;
  P.n_items = (int64_t)a->B * a->KH * a->num_splits;
  P.scale_log2 = a->scale * LOG2E;
  P.ws_o = P.ws_m = P.ws_l = nullptr;
  if (a->num_splits > 1) {
    const size_t need = uvmi_decode_attn_workspace_bytes(a->B, a->H, a->KH, a->hd, a->num_splits);
    UVMI_REQUIRE(a->workspace && a->workspace_bytes >= need, UVMI_EWORKSPACE,
                 "uvmi_decode_attn: workspace of %zu bytes needed, %zu given", need, a->workspace_bytes);
    UVMI_REQUIRE(((uintptr_t)a->workspace % 16) == 0, UVMI_EWORKSPACE, "uvmi_decode_attn: workspace must be 16-byte aligned");
    const size_t rows = (size_t)a->B * a->H * a->num_splits;
    P.ws_o = (float*)a->workspace;
    P.ws_m = P.ws_o + rows * a->hd;
    P.ws_l = P.ws_m + rows;
  }
  UVMI_REQUIRE(P.n_items < (1LL << 31), UVMI_EUNSUPPORTED, "uvmi_decode_attn: too many work items");
  if (mfma_ok(a)) {
    const dim3 grid((unsigned)((P.n_items + 3) / 4)), blk(256);
#define UVMI_L(QD, OD) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD>), grid, blk, 0, st, P)
    const int od = a->num_splits > 1 ? UVMI_F32 : a->out_dtype;  // partials are fp32; ODT only matters for splits == 1
    if (a->q_dtype == UVMI_F16) {
      if (od == UVMI_F16) UVMI_L(UVMI_F16, UVMI_F16); else if (od == UVMI_BF16) UVMI_L(UVMI_F16, UVMI_BF16); else UVMI_L(UVMI_F16, UVMI_F32);
    } else {
      if (od == UVMI_F16) UVMI_L(UVMI_BF16, UVMI_F16); else if (od == UVMI_BF16) UVMI_L(UVMI_BF16, UVMI_BF16); else UVMI_L(UVMI_BF16, UVMI_F32);
    }
#undef UVMI_L
  } else {
    const dim3 grid((unsigned)P.n_items), blk(64);
    const size_t sh = ((size_t)P.G * a->hd + (size_t)P.G * 64) * 4;
    const int od = a->num_splits > 1 ? UVMI_F32 : a->out_dtype;
#define UVMI_L(QD, KD, OD) hipLaunchKernelGGL((attn_generic<QD, KD, OD>), grid, blk, sh, st, P)
#define UVMI_LO(QD, KD) do { if (od == UVMI_F16) UVMI_L(QD, KD, UVMI_F16); else if (od == UVMI_BF16) UVMI_L(QD, KD, UVMI_BF16); else UVMI_L(QD, KD, UVMI_F32); } while (0)
#define UVMI_LK(QD) do { if (a->kv_dtype == UVMI_I8) UVMI_LO(QD, UVMI_I8); else if (a->kv_dtype == UVMI_F16) UVMI_LO(QD, UVMI_F16); else UVMI_LO(QD, UVMI_BF16); } while (0)
    if (a->q_dtype == UVMI_F16) UVMI_LK(UVMI_F16); else UVMI_LK(UVMI_BF16);
#undef UVMI_LK
#undef UVMI_LO
#undef UVMI_L
  }
  UVMI_CHECK_LAUNCH("uvmi_decode_attn");
  if (a->num_splits > 1) {
    const int64_t rows = (int64_t)a->B * a->H;
    const dim3 grid((unsigned)((rows + 3) / 4)), blk(256);
    if (a->out_dtype == UVMI_F16) hipLaunchKernelGGL((attn_combine<UVMI_F16>), grid, blk, 0, st, P);
    else if (a->out_dtype == UVMI_BF16) hipLaunchKernelGGL((attn_combine<UVMI_BF16>), grid, blk, 0, st, P);
    else hipLaunchKernelGGL((attn_combine<UVMI_F32>), grid, blk, 0, st, P);
    UVMI_CHECK_LAUNCH("uvmi_decode_attn(combine)");
  }
  return UVMI_OK;
}
