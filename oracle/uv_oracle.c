/*
 * Plain-C twin of the numpy oracle (checker only; see oracle/__init__.py).  Built by oracle/build.py into
 * oracle/libuv_oracle.so and called through ctypes by tests and by bench.py's cpu_baseline leg.
 *
 * Functions follow the reference files cited at each definition (paths relative to the reference checkout).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- fp16 <-> fp32 (IEEE, round-to-nearest-even, subnormals kept) ---------------------------------------- */
static float h2f(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 0x1f, m = h & 0x3ff, u;
  if (e == 0) {
    if (m == 0) u = s;
    else {
      int sh = 0;
      while (!(m & 0x400)) { m <<= 1; sh++; }
      u = s | ((uint32_t)(127 - 15 - sh + 1) << 23) | ((m & 0x3ff) << 13);
    }
  } else if (e == 31) u = s | 0x7f800000u | (m << 13);
  else u = s | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint16_t f2h(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t s = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return (uint16_t)(s | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0));
  if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00u);            /* rounds to >= 65520 -> inf */
  if (a < 0x33000001u) return (uint16_t)s;                         /* < 2^-25 (or exactly 2^-25: ties to even 0) */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13;
  uint32_t q = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  if (e < -14) return (uint16_t)(s | q);                           /* subnormal (q may carry into the normal range) */
  return (uint16_t)(s | (((uint32_t)(e + 15) << 10) + (q - 0x400u)));
}
uint16_t uvo_f2h(float f) { return f2h(f); }
float uvo_h2f(uint16_t h) { return h2f(h); }

/* ---- quantize_kv: ultraviolet/kernels/kv_quant.py:12-19 --------------------------------------------------- */
void uvo_quantize_rows(const float* x, int64_t n_rows, int hd, int8_t* q, uint16_t* scale) {
  for (int64_t r = 0; r < n_rows; r++) {
    const float* xr = x + r * hd;
    float am = 0.f;
    for (int d = 0; d < hd; d++) { float a = fabsf(xr[d]); if (a > am) am = a; }
    uint16_t s16 = f2h(am / 127.0f);
    float sf = h2f(s16);
    if (sf < 1e-30f) sf = 1e-30f;
    for (int d = 0; d < hd; d++) {
      float v = nearbyintf(xr[d] / sf);  /* default rounding mode: half to even */
      if (v > 127.f) v = 127.f;
      if (v < -127.f) v = -127.f;
      q[r * hd + d] = (int8_t)v;
    }
    scale[r] = s16;
  }
}

/* kv_write: ultraviolet/kernels/kv_quant.py:26-36 */
void uvo_kv_write(int8_t* cache, uint16_t* scale, const int64_t* flat_idx, const float* x, int64_t n_rows, int hd) {
  for (int64_t r = 0; r < n_rows; r++) uvo_quantize_rows(x + r * hd, 1, hd, cache + flat_idx[r] * hd, scale + flat_idx[r]);
}

/* ---- decode attention, per row over its own keys: decode_attn.py:233-263 (semantics), :37-44 (key range) ---
 * q (B, H, hd) fp32; caches (B, KH, S, hd) int8 contiguous; scales (B, KH, S) fp16; out (B, H, hd) fp32.
 * rows [b0, b1) are processed (so callers can thread over rows). */
void uvo_decode_attn_i8(const float* q, const int8_t* kc, const int8_t* vc, const uint16_t* ks, const uint16_t* vs,
                        const int64_t* pos, const int64_t* starts, float* out, int B, int H, int KH, int S, int hd,
                        float scale, int window, int ring, int b0, int b1) {
  int G = H / KH;
  float* sc = (float*)malloc(sizeof(float) * (size_t)S);
  double* acc = (double*)malloc(sizeof(double) * (size_t)hd);
  (void)B;
  for (int b = b0; b < b1; b++) {
    int64_t p = pos[b], lo = starts[b] > 0 ? starts[b] : 0;
    if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
    int64_t n = p - lo + 1;
    for (int h = 0; h < H; h++) {
      int kh = h / G;
      const float* qh = q + ((int64_t)b * H + h) * hd;
      float* o = out + ((int64_t)b * H + h) * hd;
      if (n <= 0) { memset(o, 0, sizeof(float) * hd); continue; }
      const int8_t* kb = kc + ((int64_t)b * KH + kh) * S * hd;
      const int8_t* vb = vc + ((int64_t)b * KH + kh) * S * hd;
      const uint16_t* ksb = ks + ((int64_t)b * KH + kh) * S;
      const uint16_t* vsb = vs + ((int64_t)b * KH + kh) * S;
      float mx = -INFINITY;
      for (int64_t i = 0; i < n; i++) {
        int64_t t = lo + i, sl = ring ? t % S : t;
        float d = 0.f;
        for (int e = 0; e < hd; e++) d += qh[e] * (float)kb[sl * hd + e];
        sc[i] = d * h2f(ksb[sl]) * scale;
        if (sc[i] > mx) mx = sc[i];
      }
      double den = 0.0;
      for (int e = 0; e < hd; e++) acc[e] = 0.0;
      for (int64_t i = 0; i < n; i++) {
        int64_t t = lo + i, sl = ring ? t % S : t;
        float w = expf(sc[i] - mx);
        den += w;
        float wv = w * h2f(vsb[sl]);
        for (int e = 0; e < hd; e++) acc[e] += (double)wv * (double)vb[sl * hd + e];
      }
      for (int e = 0; e < hd; e++) o[e] = (float)(acc[e] / den);
    }
  }
  free(sc);
  free(acc);
}

/* ---- fused_sample_ref: ultraviolet/kernels/fused_sample.py:79-91 ------------------------------------------- */
void uvo_fused_sample(const float* x, const float* u, int B, int V, float a, float b, float c, float T, int64_t* tok,
                      float* logp) {
  float* cs = (float*)malloc(sizeof(float) * (size_t)V);
  float* z = (float*)malloc(sizeof(float) * (size_t)V);
  for (int r = 0; r < B; r++) {
    const float* xr = x + (int64_t)r * V;
    float run = 0.f;
    for (int i = 0; i < V; i++) {
      z[i] = a / (1.0f + expf(-((xr[i] + b) / c)));
      run += expf((z[i] - a) / T);
      cs[i] = run;
    }
    float S = cs[V - 1], target = (1.0f - u[r]) * S;
    int lo = 0, hi = V;  /* first index with cs >= target */
    while (lo < hi) { int mid = (lo + hi) / 2; if (cs[mid] < target) lo = mid + 1; else hi = mid; }
    if (lo > V - 1) lo = V - 1;
    tok[r] = lo;
    logp[r] = (z[lo] - a) / T - logf(S);
  }
  free(cs);
  free(z);
}

/* ---- Philox4x32-10 (Random123) ----------------------------------------------------------------------------- */
void uvo_philox4x32_10(const uint32_t* ctr, const uint32_t* key, uint32_t* out) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
