// Backward of the packed (cu_seqlens) causal attention with an optional sliding window: dq, dk, dv from the output
// gradient (reference: mathk::varlen_attn_bwd, ultraviolet/kernels/varlen_attn.py:56-66, which calls
// aten._efficient_attention_backward on K / V expanded to the query heads and sums their gradients back over a group).
//
// With s_ij = scale q_i . k_j over the keys j query i sees (same segment, i - window < j <= i), p_ij = exp(s_ij - lse_i),
// D_i = go_i . o_i:   dv_j = sum_i p_ij go_i,   ds_ij = p_ij (go_i . v_j - D_i),   dq_i = scale sum_j ds_ij k_j,
// dk_j = scale sum_i ds_ij q_i  (dk, dv also summed over the query heads of the group).
//
// Two forms.  The matrix-core form (bwd_dq_mfma, bwd_dkv_mfma, described where they are defined) serves up to 8 query heads
// per kv head.  The plain form below it serves the rest: fp32 arithmetic on the vector units, no atomics, no
// cross-workgroup state.
//   bwd_dq_kernel   lane = query token (64 per wave), one query head per workgroup: the wave walks the union of its
//                   queries' key ranges; a key / value row is the same address in every lane.  Pass 1 recomputes the
//                   row's log-sum-exp (the forward does not keep it), pass 2 accumulates dq in registers.  Writes
//                   lse and D for the second kernel.
//   bwd_dkv_kernel  two lanes per key (32 head dims each, 32 keys per wave), one kv head per workgroup: the wave walks
//                   the queries that see its keys and the heads of the group; dk and dv stay in registers.
#include "common.h"
#include "attn_mfma_util.h"

#include <climits>

namespace uvmi {

struct BwdParams {
  const void* q; const void* k; const void* v; const void* o; const void* go;
  void* dq; void* dk; void* dv;
  float* lse; float* dsum;   // (N, H) each
  const void* cu; int idx64, n_seg, N, H, KH, G, window;
  float scale;
};

template <int DT>
__device__ __forceinline__ void bld8(const void* p, int64_t i, float* o) {  // 8 consecutive 16-bit elements from element i
  const uint4 w = *(const uint4*)((const uint16_t*)p + i);
  const uint32_t r[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if (DT == UVMI_BF16) {
      o[2 * j] = __uint_as_float(r[j] << 16);
      o[2 * j + 1] = __uint_as_float(r[j] & 0xffff0000u);
    } else {
      o[2 * j] = half_bits_to_float((uint16_t)(r[j] & 0xffff));
      o[2 * j + 1] = half_bits_to_float((uint16_t)(r[j] >> 16));
    }
  }
}
template <int DT>
__device__ __forceinline__ void bst8(void* p, int64_t i, const float* v) {
  uint32_t r[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if (DT == UVMI_BF16) r[j] = float2_to_bf16x2(v[2 * j], v[2 * j + 1]);
    else r[j] = (uint32_t)float_to_half_bits(v[2 * j]) | ((uint32_t)float_to_half_bits(v[2 * j + 1]) << 16);
  }
  *(uint4*)((uint16_t*)p + i) = uint4{r[0], r[1], r[2], r[3]};
}

__device__ __forceinline__ int wave_min_i(int v) {
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_max_i(int v) {
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}

// index s of the segment that holds token t: the last s < n_seg with cu[s] <= t (empty segments are skipped)
__device__ __forceinline__ int segment_of(const BwdParams& P, int t) {
  int lo = 0, hi = P.n_seg;  // invariant: cu[lo] <= t, and hi == n_seg or cu[hi] > t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (load_index(P.cu, P.idx64, mid) <= t) lo = mid; else hi = mid;
  }
  return lo;
}

template <int DT>
__global__ __launch_bounds__(64) void bwd_dq_kernel(BwdParams P) {
  const int lane = threadIdx.x, h = blockIdx.y, kh = h / P.G;
  const int i = blockIdx.x * 64 + lane;
  int n_end = (int)load_index(P.cu, P.idx64, P.n_seg);   // tokens at or after it are padding
  n_end = n_end < 0 ? 0 : (n_end > P.N ? P.N : n_end);
  const bool live = i < n_end;
  int lo = 0x7fffffff, hi = -1;   // keys lo..hi (inclusive)
  if (live) {
    int seg0 = (int)load_index(P.cu, P.idx64, segment_of(P, i));
    if (seg0 < 0) seg0 = 0;
    lo = P.window > 0 && i - P.window + 1 > seg0 ? i - P.window + 1 : seg0;
    hi = i;
  }
  const int jmin = __builtin_amdgcn_readfirstlane(wave_min_i(lo)), jmax = __builtin_amdgcn_readfirstlane(wave_max_i(hi));
  const int64_t qrow = ((int64_t)(live ? i : 0) * P.H + h) * 64;
  float q[64], g[64], dq[64];
  float D = 0.f;
#pragma unroll
  for (int c = 0; c < 8; c++) {
    float o8[8];
    bld8<DT>(P.q, qrow + 8 * c, q + 8 * c);
    bld8<DT>(P.go, qrow + 8 * c, g + 8 * c);
    bld8<DT>(P.o, qrow + 8 * c, o8);
#pragma unroll
    for (int d = 0; d < 8; d++) {
      D = fmaf(g[8 * c + d], o8[d], D);
      dq[8 * c + d] = 0.f;
    }
  }
  auto score = [&](int j) {
    const int64_t kr = ((int64_t)j * P.KH + kh) * 64;
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 8; c++) {
      float k8[8];
      bld8<DT>(P.k, kr + 8 * c, k8);
#pragma unroll
      for (int d = 0; d < 8; d++) s = fmaf(q[8 * c + d], k8[d], s);
    }
    return s * P.scale;
  };
  // ---- pass 1: log-sum-exp of the row
  float m = -INFINITY, l = 0.f;
  for (int j = jmin; j <= jmax; j++) {
    const float s = score(j);
    if (j >= lo && j <= hi) {
      const float mn = fmaxf(m, s);
      l = l * __expf(m - mn) + __expf(s - mn);
      m = mn;
    }
  }
  const float lse = live ? m + __logf(l) : 0.f;   // (a live query sees at least itself)
  // ---- pass 2: dq
  for (int j = jmin; j <= jmax; j++) {
    const float s = score(j);
    const bool ok = j >= lo && j <= hi;
    const float p = ok ? __expf(s - lse) : 0.f;
    const int64_t kr = ((int64_t)j * P.KH + kh) * 64;
    float dp = 0.f;
#pragma unroll
    for (int c = 0; c < 8; c++) {
      float v8[8];
      bld8<DT>(P.v, kr + 8 * c, v8);
#pragma unroll
      for (int d = 0; d < 8; d++) dp = fmaf(g[8 * c + d], v8[d], dp);
    }
    const float ds = p * (dp - D);
#pragma unroll
    for (int c = 0; c < 8; c++) {
      float k8[8];
      bld8<DT>(P.k, kr + 8 * c, k8);
#pragma unroll
      for (int d = 0; d < 8; d++) dq[8 * c + d] = fmaf(ds, k8[d], dq[8 * c + d]);
    }
  }
  if (i < P.N) {
    const int64_t orow = ((int64_t)i * P.H + h) * 64;
#pragma unroll
    for (int c = 0; c < 8; c++) {
      float o8[8];
#pragma unroll
      for (int d = 0; d < 8; d++) o8[d] = live ? dq[8 * c + d] * P.scale : 0.f;
      bst8<DT>(P.dq, orow + 8 * c, o8);
    }
    P.lse[(int64_t)i * P.H + h] = lse;
    P.dsum[(int64_t)i * P.H + h] = live ? D : 0.f;
  }
}

template <int DT>
__global__ __launch_bounds__(64) void bwd_dkv_kernel(BwdParams P) {
  const int lane = threadIdx.x, jj = lane >> 1, half = lane & 1, kh = blockIdx.y;
  const int j = blockIdx.x * 32 + jj;
  int n_end = (int)load_index(P.cu, P.idx64, P.n_seg);
  n_end = n_end < 0 ? 0 : (n_end > P.N ? P.N : n_end);
  const bool live = j < n_end;
  int lo = 0x7fffffff, hi = 0;   // queries lo .. hi - 1 see key j
  if (live) {
    int se = (int)load_index(P.cu, P.idx64, segment_of(P, j) + 1);
    se = se > n_end ? n_end : se;
    lo = j;
    hi = P.window > 0 && j + P.window < se ? j + P.window : se;
  }
  const int imin = __builtin_amdgcn_readfirstlane(wave_min_i(lo)), imax = __builtin_amdgcn_readfirstlane(wave_max_i(hi)) - 1;
  const int64_t krow = ((int64_t)(live ? j : 0) * P.KH + kh) * 64 + 32 * half;
  float kk[32], vv[32], dk[32], dv[32];
#pragma unroll
  for (int c = 0; c < 4; c++) {
    bld8<DT>(P.k, krow + 8 * c, kk + 8 * c);
    bld8<DT>(P.v, krow + 8 * c, vv + 8 * c);
#pragma unroll
    for (int d = 0; d < 8; d++) { dk[8 * c + d] = 0.f; dv[8 * c + d] = 0.f; }
  }
  for (int i = imin; i <= imax; i++) {
    const bool ok = live && i >= lo && i < hi;
    for (int hh = 0; hh < P.G; hh++) {
      const int h = kh * P.G + hh;
      const int64_t qrow = ((int64_t)i * P.H + h) * 64 + 32 * half;
      float qh[32], gh[32];
      float s = 0.f, dp = 0.f;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        bld8<DT>(P.q, qrow + 8 * c, qh + 8 * c);
        bld8<DT>(P.go, qrow + 8 * c, gh + 8 * c);
#pragma unroll
        for (int d = 0; d < 8; d++) {
          s = fmaf(qh[8 * c + d], kk[8 * c + d], s);
          dp = fmaf(gh[8 * c + d], vv[8 * c + d], dp);
        }
      }
      s += __shfl_xor(s, 1, 64);
      dp += __shfl_xor(dp, 1, 64);
      const float p = ok ? __expf(s * P.scale - P.lse[(int64_t)i * P.H + h]) : 0.f;
      const float ds = p * (dp - P.dsum[(int64_t)i * P.H + h]);
#pragma unroll
      for (int d = 0; d < 32; d++) {
        dv[d] = fmaf(p, gh[d], dv[d]);
        dk[d] = fmaf(ds, qh[d], dk[d]);
      }
    }
  }
  if (j < P.N) {
    const int64_t orow = ((int64_t)j * P.KH + kh) * 64 + 32 * half;
#pragma unroll
    for (int c = 0; c < 4; c++) {
      float a8[8], b8[8];
#pragma unroll
      for (int d = 0; d < 8; d++) { a8[d] = live ? dk[8 * c + d] * P.scale : 0.f; b8[d] = live ? dv[8 * c + d] : 0.f; }
      bst8<DT>(P.dk, orow + 8 * c, a8);
      bst8<DT>(P.dv, orow + 8 * c, b8);
    }
  }
}

// ------------------------------------------------------------------------------------------------ the MFMA form
// Same mathematics on the matrix cores, on the forward kernel's operand layouts (prefill_attn.hip):
//   * the forward kernel is run once more without storing an output, for the rows' log-sum-exp (log2 domain);
//   * bwd_dq_mfma: a workgroup owns 16 query rows of one kv head, wave w the query heads 2w, 2w+1 of the group.  K and V
//     super-tiles (32 keys) are staged once per workgroup in LDS.  S^T = K Q^T and dP^T = V dO^T have the same shape: a lane
//     of either accumulator holds 4 consecutive keys of one query row for two 16-key tiles, so p = exp2(c s - lse) and
//     ds = p (dp - D) are lane-local, and the 8 values of ds, rounded to the input type, are the lane's slice of the B
//     operand of dQ^T += K^T dS^T (K^T operands from 8-byte LDS reads regrouped with v_perm_b32, as V^T in the forward);
//   * bwd_dkv_mfma: the transposed problem.  A workgroup owns 64 keys of one kv head (16 per wave) and walks (query tile of
//     32, query head): the tile's Q and dO rows are staged in LDS; S = Q K^T and dP = dO V^T leave 4 consecutive queries
//     of one key in a lane for two 16-query tiles, exactly the B-operand slices of dV^T += dO^T P and dK^T += Q^T dS, which
//     accumulate over the tiles and over the heads of the group in registers.
// Probabilities and ds are rounded to the input type for their second products; everything else is fp32.
struct BwdMParams {
  const void* q; const void* k; const void* v; const void* o; const void* go;
  void* dq; void* dk; void* dv;
  const float* lse; float* dsum; int64_t ls;   // (H, ls) each: log2-domain log-sum-exp of a row, and D = go . o
  const int32_t* seg_start;                     // (ls,) first token of each token's sequence (entries >= N unused)
  const void* cu; int idx64, n_seg;
  int N, H, KH, G, window, n_wg;
  float scale, scale_log2;
};

template <int DT>
__device__ __forceinline__ float dot2w(uint32_t a, uint32_t b, float acc) {  // acc + a.lo b.lo + a.hi b.hi of two packed 16-bit pairs
  float a0, a1, b0, b1;
  if constexpr (DT == UVMI_BF16) {
    a0 = __uint_as_float(a << 16); a1 = __uint_as_float(a & 0xffff0000u); b0 = __uint_as_float(b << 16); b1 = __uint_as_float(b & 0xffff0000u);
  } else {
    a0 = half_bits_to_float((uint16_t)(a & 0xffff)); a1 = half_bits_to_float((uint16_t)(a >> 16));
    b0 = half_bits_to_float((uint16_t)(b & 0xffff)); b1 = half_bits_to_float((uint16_t)(b >> 16));
  }
  return fmaf(a1, b1, fmaf(a0, b0, acc));
}

// Four transposed operands from eight 8-byte reads: r[j] holds dims 4m..4m+3 of contraction slot j's row; operand t, row m is
// dim 4m + t, dword p of an operand holds slots 2p, 2p+1.
__device__ __forceinline__ void transpose_ops(const pu2* r, pu4* op) {
  constexpr uint32_t LO = 0x05040100u, HI = 0x07060302u;
#pragma unroll
  for (int p = 0; p < 4; p++) {
    op[0][p] = __builtin_amdgcn_perm(r[2 * p + 1].x, r[2 * p].x, LO);
    op[1][p] = __builtin_amdgcn_perm(r[2 * p + 1].x, r[2 * p].x, HI);
    op[2][p] = __builtin_amdgcn_perm(r[2 * p + 1].y, r[2 * p].y, LO);
    op[3][p] = __builtin_amdgcn_perm(r[2 * p + 1].y, r[2 * p].y, HI);
  }
}

// LDS reads of a staged 32-row tile (rows of 128 bytes, chunk-swizzled): the A-operand form (lane = row m of tile A / B,
// dims 8g.. of each half) and the rows for the transposed form (rows 4g+j of tile A / B, dims 4m..4m+3).
__device__ __forceinline__ void read_rows_a(const unsigned char* s, int m, int g, pu4* a) {
  const uint32_t o0 = lds_chunk_off(m, g), o1 = lds_chunk_off(m, 4 + g);   // (rows m and 16 + m swizzle alike)
  a[0] = *(const pu4*)(s + o0);
  a[1] = *(const pu4*)(s + o1);
  a[2] = *(const pu4*)(s + 2048 + o0);
  a[3] = *(const pu4*)(s + 2048 + o1);
}
__device__ __forceinline__ void read_rows_t(const unsigned char* s, int m, int g, pu2* r) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint32_t o = lds_chunk_off(4 * g + j, m >> 1) + 8 * (m & 1);
    r[j] = *(const pu2*)(s + o);
    r[4 + j] = *(const pu2*)(s + 2048 + o);
  }
}

template <int DT>
__device__ __forceinline__ void store_dims16(void* base, int64_t off, const pf4* acc, float mul) {  // acc[t][i] is dim 4 i + t of the lane's 16
  float o[16];
#pragma unroll
  for (int t = 0; t < 4; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) o[4 * i + t] = acc[t][i] * mul;
  uint32_t w[8];
#pragma unroll
  for (int i = 0; i < 8; i++) w[i] = pack2<DT>(o[2 * i], o[2 * i + 1]);
  uint16_t* p = (uint16_t*)base + off;
  *(uint4*)p = uint4{w[0], w[1], w[2], w[3]};
  *(uint4*)(p + 8) = uint4{w[4], w[5], w[6], w[7]};
}

template <int DT>
__global__ __launch_bounds__(256) void bwd_dq_mfma(BwdMParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2][2][4096];  // [half][K, V][32 keys x 128 B]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int per = gridDim.x >> 3;
  const int bid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);   // an XCD (ids congruent mod 8) gets a contiguous range
  if (bid >= P.n_wg) return;
  const int kvh = bid % P.KH, qb = bid / P.KH;
  const int m = lane & 15, g = lane >> 4;
  const int G = P.G;
  const float c = P.scale_log2;
  int n_end = (int)load_index(P.cu, P.idx64, P.n_seg);   // tokens at or after it are padding
  n_end = n_end < 0 ? 0 : (n_end > P.N ? P.N : n_end);
  const int r0 = qb * 16, row = r0 + m;
  const bool row_ok = row < n_end;
  const int rowc = row < P.N ? row : P.N - 1;
  int lo_n = P.seg_start[rowc];
  if (P.window > 0 && row - P.window + 1 > lo_n) lo_n = row - P.window + 1;
  if (!row_ok) lo_n = INT_MAX;
  // the block's key range: from its first live row's lower bound to its last live row (none: no tile)
  const int rl = min(r0 + 15, n_end - 1);
  const bool any = r0 < n_end;
  const int lo_first = __builtin_amdgcn_readfirstlane(lo_n);
  const int lo_last = __builtin_amdgcn_readfirstlane(__shfl(lo_n, any ? rl - r0 : 0, 64));
  const int kbeg = any ? lo_first & ~31 : 0, kend = any ? rl + 1 : 0;
  const int nk = (kend - kbeg + 31) >> 5;

  // ---- Q^T and dO^T operands (lane = row m, dims 32 s + 8 g ..), D = dO . O, the row's log-sum-exp
  pu4 Q[2][2], GO[2][2];
  float lse2[2], Dr[2];
  bool hok[2];
#pragma unroll
  for (int hh = 0; hh < 2; hh++) {
    const int hq = 2 * wave + hh;
    hok[hh] = hq < G;
    const int head = kvh * G + (hok[hh] ? hq : G - 1);
    const int64_t base = ((int64_t)rowc * P.H + head) * 64 + 8 * g;
    Q[hh][0] = *(const pu4*)((const uint16_t*)P.q + base);
    Q[hh][1] = *(const pu4*)((const uint16_t*)P.q + base + 32);
    GO[hh][0] = *(const pu4*)((const uint16_t*)P.go + base);
    GO[hh][1] = *(const pu4*)((const uint16_t*)P.go + base + 32);
    const pu4 o0 = *(const pu4*)((const uint16_t*)P.o + base), o1 = *(const pu4*)((const uint16_t*)P.o + base + 32);
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) d = dot2w<DT>(GO[hh][1][i], o1[i], dot2w<DT>(GO[hh][0][i], o0[i], d));
    d = psum32(psum16(d));
    Dr[hh] = d;
    lse2[hh] = row_ok ? P.lse[(int64_t)head * P.ls + row] : INFINITY;
    if (hok[hh] && g == 0 && row < P.N) P.dsum[(int64_t)head * P.ls + row] = row_ok ? d : 0.f;
  }
  pf4 dQ[2][4];
#pragma unroll
  for (int hh = 0; hh < 2; hh++)
#pragma unroll
    for (int t = 0; t < 4; t++) dQ[hh][t] = pf4{0.f, 0.f, 0.f, 0.f};

  // ---- K / V tiles: global -> registers -> LDS, one tile ahead of the arithmetic
  const uint16_t* kbase = (const uint16_t*)P.k + (int64_t)kvh * 64;
  const uint16_t* vbase = (const uint16_t*)P.v + (int64_t)kvh * 64;
  const int64_t rstride = (int64_t)P.KH * 64;
  const int lkey = tid >> 3, lch = tid & 7;
  const uint32_t st_off = lds_chunk_off(lkey, lch);
  pu4 rk, rv;
  auto fetch = [&](int kt) {
    const int tb = kbeg + 32 * min(kt, max(nk - 1, 0));
    const int64_t r = (int64_t)min(tb + lkey, P.N - 1) * rstride + 8 * lch;
    rk = *(const pu4*)(kbase + r);
    rv = *(const pu4*)(vbase + r);
  };
  auto park = [&](int half) {
    *(pu4*)(&smem[half][0][st_off]) = rk;
    *(pu4*)(&smem[half][1][st_off]) = rv;
  };
  const bool work = hok[0];   // (wave-uniform: a wave without a head only helps with the loads)
  auto step = [&](int half, int tb) {
    pu4 KA[4], VA[4], KT[4];
    pu2 kt[8];
    read_rows_a(smem[half][0], m, g, KA);
    read_rows_a(smem[half][1], m, g, VA);
    read_rows_t(smem[half][0], m, g, kt);
    transpose_ops(kt, KT);
    const bool edge = !(tb >= lo_last && tb + 31 <= r0);
    const int kA = tb + 4 * g, kB = kA + 16;
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      if (!hok[hh]) continue;
      pf4 sA = pf4{0.f, 0.f, 0.f, 0.f}, sB = sA, pA = sA, pB = sA;
      sA = mfma16<DT>(KA[0], Q[hh][0], sA);
      sB = mfma16<DT>(KA[2], Q[hh][0], sB);
      pA = mfma16<DT>(VA[0], GO[hh][0], pA);
      pB = mfma16<DT>(VA[2], GO[hh][0], pB);
      sA = mfma16<DT>(KA[1], Q[hh][1], sA);
      sB = mfma16<DT>(KA[3], Q[hh][1], sB);
      pA = mfma16<DT>(VA[1], GO[hh][1], pA);
      pB = mfma16<DT>(VA[3], GO[hh][1], pB);
      float ds[8];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float p0 = __builtin_amdgcn_exp2f(fmaf(sA[i], c, -lse2[hh])), p1 = __builtin_amdgcn_exp2f(fmaf(sB[i], c, -lse2[hh]));
        if (edge) {
          if (kA + i < lo_n || kA + i > row) p0 = 0.f;
          if (kB + i < lo_n || kB + i > row) p1 = 0.f;
        }
        ds[i] = p0 * (pA[i] - Dr[hh]);
        ds[4 + i] = p1 * (pB[i] - Dr[hh]);
      }
      const pu4 dsB = pu4{pack2<DT>(ds[0], ds[1]), pack2<DT>(ds[2], ds[3]), pack2<DT>(ds[4], ds[5]), pack2<DT>(ds[6], ds[7])};
#pragma unroll
      for (int t = 0; t < 4; t++) dQ[hh][t] = mfma16<DT>(KT[t], dsB, dQ[hh][t]);
    }
  };
  if (nk > 0) {
    fetch(0);
    park(0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
      fetch(kt + 1);
      if (work) step(kt & 1, kbeg + 32 * kt);
      park((kt + 1) & 1);
      __syncthreads();
    }
  }
  // ---- dq = scale dQ; lane (row m, group g) holds head dims 16g .. 16g+15 (zeros for padding rows)
  if (row < P.N) {
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      if (!hok[hh]) continue;
      const int head = kvh * G + 2 * wave + hh;
      store_dims16<DT>(P.dq, ((int64_t)row * P.H + head) * 64 + 16 * g, dQ[hh], P.scale);
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void bwd_dkv_mfma(BwdMParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2][2][4096];  // [half][Q, dO][32 queries x 128 B]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int per = gridDim.x >> 3;
  const int bid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (bid >= P.n_wg) return;
  const int kvh = bid % P.KH, kb = bid / P.KH;
  const int n = lane & 15, g = lane >> 4;   // accumulator column n = key, group g = queries 4g .. 4g+3 of a 16-query tile
  const int G = P.G;
  const float c = P.scale_log2;
  int n_end = (int)load_index(P.cu, P.idx64, P.n_seg);
  n_end = n_end < 0 ? 0 : (n_end > P.N ? P.N : n_end);
  const int jw0 = kb * 64, jw_last = min(jw0 + 63, n_end - 1);
  const int key = jw0 + 16 * wave + n;
  const bool key_ok = key < n_end;
  const int keyc = key < P.N ? key : P.N - 1;
  // ---- K^T / V^T operands (B side: lane = key n, dims 32 s + 8 g ..)
  pu4 Kb[2], Vb[2];
  {
    const int64_t base = ((int64_t)keyc * P.KH + kvh) * 64 + 8 * g;
    Kb[0] = *(const pu4*)((const uint16_t*)P.k + base);
    Kb[1] = *(const pu4*)((const uint16_t*)P.k + base + 32);
    Vb[0] = *(const pu4*)((const uint16_t*)P.v + base);
    Vb[1] = *(const pu4*)((const uint16_t*)P.v + base + 32);
  }
  pf4 dK[4], dV[4];
#pragma unroll
  for (int t = 0; t < 4; t++) dK[t] = dV[t] = pf4{0.f, 0.f, 0.f, 0.f};
  // queries that may see a key of this workgroup: jw0 .. qend - 1 (its keys' segment may end earlier: checked per tile)
  int qend = n_end;
  if (P.window > 0 && jw_last + P.window < qend) qend = jw_last + P.window;
  const int n_tiles = jw0 < n_end ? (qend - jw0 + 31) >> 5 : 0;
  const int n_it = n_tiles * G;
  const int lrow = tid >> 3, lch = tid & 7;
  const uint32_t st_off = lds_chunk_off(lrow, lch);
  pu4 rq, rg;
  auto fetch = [&](int it) {
    const int itc = min(it, max(n_it - 1, 0));
    const int tq = jw0 + 32 * (itc / G), head = kvh * G + itc % G;
    const int64_t r = ((int64_t)min(tq + lrow, P.N - 1) * P.H + head) * 64 + 8 * lch;
    rq = *(const pu4*)((const uint16_t*)P.q + r);
    rg = *(const pu4*)((const uint16_t*)P.go + r);
  };
  auto park = [&](int half) {
    *(pu4*)(&smem[half][0][st_off]) = rq;
    *(pu4*)(&smem[half][1][st_off]) = rg;
  };
  auto step = [&](int half, int tq, int head, bool interior) {
    pu4 QA[4], GA[4], QT[4], GT[4];
    pu2 rt[8];
    read_rows_a(smem[half][0], n, g, QA);
    read_rows_a(smem[half][1], n, g, GA);
    read_rows_t(smem[half][0], n, g, rt);
    transpose_ops(rt, QT);
    read_rows_t(smem[half][1], n, g, rt);
    transpose_ops(rt, GT);
    pf4 sA = pf4{0.f, 0.f, 0.f, 0.f}, sB = sA, pA = sA, pB = sA;
    sA = mfma16<DT>(QA[0], Kb[0], sA);
    sB = mfma16<DT>(QA[2], Kb[0], sB);
    pA = mfma16<DT>(GA[0], Vb[0], pA);
    pB = mfma16<DT>(GA[2], Vb[0], pB);
    sA = mfma16<DT>(QA[1], Kb[1], sA);
    sB = mfma16<DT>(QA[3], Kb[1], sB);
    pA = mfma16<DT>(GA[1], Vb[1], pA);
    pB = mfma16<DT>(GA[3], Vb[1], pB);
    // statistics of this lane's queries tq + 4g + i (tile A) and tq + 16 + 4g + i (tile B)
    const float* lp = P.lse + (int64_t)head * P.ls + tq + 4 * g;
    const float* dp = P.dsum + (int64_t)head * P.ls + tq + 4 * g;
    const float4 la = *(const float4*)lp, lb = *(const float4*)(lp + 16), da = *(const float4*)dp, db = *(const float4*)(dp + 16);
    const float lA[4] = {la.x, la.y, la.z, la.w}, lB[4] = {lb.x, lb.y, lb.z, lb.w};
    const float dA[4] = {da.x, da.y, da.z, da.w}, dB[4] = {db.x, db.y, db.z, db.w};
    float p[8], ds[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      p[i] = __builtin_amdgcn_exp2f(fmaf(sA[i], c, -lA[i]));
      p[4 + i] = __builtin_amdgcn_exp2f(fmaf(sB[i], c, -lB[i]));
      ds[i] = p[i] * (pA[i] - dA[i]);
      ds[4 + i] = p[4 + i] * (pB[i] - dB[i]);
    }
    if (!interior) {   // (selects, not products: the statistics of a query past the last token are whatever the workspace held)
      const int4 sa = *(const int4*)(P.seg_start + tq + 4 * g), sb = *(const int4*)(P.seg_start + tq + 16 + 4 * g);
      const int sA_[4] = {sa.x, sa.y, sa.z, sa.w}, sB_[4] = {sb.x, sb.y, sb.z, sb.w};
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int ia = tq + 4 * g + i, ib = ia + 16;
        const bool va = key_ok && ia < n_end && key <= ia && (P.window == 0 || ia - key < P.window) && sA_[i] <= key;
        const bool vb = key_ok && ib < n_end && key <= ib && (P.window == 0 || ib - key < P.window) && sB_[i] <= key;
        if (!va) { p[i] = 0.f; ds[i] = 0.f; }
        if (!vb) { p[4 + i] = 0.f; ds[4 + i] = 0.f; }
      }
    }
    const pu4 PB = pu4{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7])};
    const pu4 SB = pu4{pack2<DT>(ds[0], ds[1]), pack2<DT>(ds[2], ds[3]), pack2<DT>(ds[4], ds[5]), pack2<DT>(ds[6], ds[7])};
#pragma unroll
    for (int t = 0; t < 4; t++) {
      dV[t] = mfma16<DT>(GT[t], PB, dV[t]);
      dK[t] = mfma16<DT>(QT[t], SB, dK[t]);
    }
  };
  if (n_it > 0) {
    fetch(0);
    park(0);
    __syncthreads();
    bool interior = false;
    for (int it = 0; it < n_it; it++) {
      const int tq = jw0 + 32 * (it / G), hh = it % G;
      if (hh == 0) {   // workgroup-uniform: the first query of the tile starts a later sequence than the last key's - done
        if (P.seg_start[min(tq, P.N - 1)] > jw_last) break;
        // no mask needed when every query of the tile follows every key, in the first key's sequence and window
        interior = tq >= jw0 + 63 && tq + 31 < n_end && jw0 + 63 < n_end && P.seg_start[tq + 31] <= jw0 &&
                   (P.window == 0 || tq + 31 - jw0 < P.window);
      }
      fetch(it + 1);
      step(it & 1, tq, kvh * G + hh, interior);
      park((it + 1) & 1);
      __syncthreads();
    }
  }
  if (key < P.N) {   // (zeros for padding tokens)
    const int64_t off = ((int64_t)key * P.KH + kvh) * 64 + 16 * g;
    store_dims16<DT>(P.dk, off, dK, P.scale);
    store_dims16<DT>(P.dv, off, dV, 1.0f);
  }
}

}  // namespace uvmi

using namespace uvmi;

static int64_t bwd_row_stride(int N) { return (((int64_t)(N > 0 ? N : 0) + 31) & ~31LL) + 32; }   // statistics rows, padded for whole-tile reads

extern "C" size_t uvmi_prefill_attn_bwd_workspace_bytes(int N, int H) {
  const size_t ls = (size_t)bwd_row_stride(N);
  return ((size_t)2 * (size_t)(H > 0 ? H : 0) * ls + 2 * ls) * 4 + 256;   // lse, D (H, ls); segment table, scratch (ls)
}

extern "C" int uvmi_prefill_attn_bwd(const uvmi_prefill_attn_bwd_args* a, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_prefill_attn_bwd: null arguments");
  UVMI_REQUIRE(a->N >= 0 && a->H > 0 && a->KH > 0 && a->H % a->KH == 0 && a->n_seg >= 0, UVMI_EINVAL, "uvmi_prefill_attn_bwd: bad sizes");
  UVMI_REQUIRE(a->hd == 64, UVMI_EUNSUPPORTED, "uvmi_prefill_attn_bwd: head_dim %d (only 64)", a->hd);
  UVMI_REQUIRE(a->dtype == UVMI_F16 || a->dtype == UVMI_BF16, UVMI_EUNSUPPORTED, "uvmi_prefill_attn_bwd: q / k / v / o / go must be fp16 or bf16");
  UVMI_REQUIRE(a->idx_dtype == UVMI_I32 || a->idx_dtype == UVMI_I64, UVMI_EINVAL, "uvmi_prefill_attn_bwd: cu_seqlens must be int32 or int64");
  UVMI_REQUIRE(a->window >= 0 && a->N < (1 << 30), UVMI_EINVAL, "uvmi_prefill_attn_bwd: bad window / N");
  if (a->N == 0) return UVMI_OK;
  UVMI_REQUIRE(a->q && a->k && a->v && a->o && a->go && a->dq && a->dk && a->dv && a->cu_seqlens, UVMI_EINVAL, "uvmi_prefill_attn_bwd: null pointer");
  const void* ptrs[] = {a->q, a->k, a->v, a->o, a->go, a->dq, a->dk, a->dv};
  for (const void* p : ptrs) UVMI_REQUIRE(((uintptr_t)p % 16) == 0, UVMI_EINVAL, "uvmi_prefill_attn_bwd: tensors must be 16-byte aligned");
  UVMI_REQUIRE(a->workspace && ((uintptr_t)a->workspace % 16) == 0 && a->workspace_bytes >= uvmi_prefill_attn_bwd_workspace_bytes(a->N, a->H),
               UVMI_EWORKSPACE, "uvmi_prefill_attn_bwd: workspace of %zu bytes needed", uvmi_prefill_attn_bwd_workspace_bytes(a->N, a->H));
  hipStream_t st = (hipStream_t)stream;
  const int64_t ls = bwd_row_stride(a->N);
  float* lse = (float*)a->workspace;
  float* dsum = lse + (size_t)a->H * ls;
  int32_t* seg = (int32_t*)(dsum + (size_t)a->H * ls);
  int32_t* pidx = seg + ls;
  const int G = a->H / a->KH;
  if (G <= 8 && (int64_t)a->N * a->H * 64 < (1LL << 30)) {
    // the MFMA form: statistics from a forward pass without output, then dq and dk / dv
    uvmi_prefill_attn_args f = {};
    f.q = a->q; f.q_dtype = a->dtype; f.sqn = (int64_t)a->H * 64; f.sqh = 64;
    f.k = a->k; f.v = a->v; f.kv_dtype = a->dtype; f.skn = f.svn = (int64_t)a->KH * 64; f.skh = f.svh = 64;
    f.cu_seqlens = a->cu_seqlens; f.idx_dtype = a->idx_dtype; f.n_seg = a->n_seg;
    f.N = a->N; f.H = a->H; f.KH = a->KH; f.hd = a->hd; f.scale = a->scale; f.window = a->window;
    UVMI_REQUIRE(a->scale > 0.f, UVMI_EUNSUPPORTED, "uvmi_prefill_attn_bwd: scale must be positive");
    int rc = prefill_attn_stats(&f, seg, pidx, lse, ls, stream);
    if (rc) return rc;
    BwdMParams M;
    M.q = a->q; M.k = a->k; M.v = a->v; M.o = a->o; M.go = a->go; M.dq = a->dq; M.dk = a->dk; M.dv = a->dv;
    M.lse = lse; M.dsum = dsum; M.ls = ls; M.seg_start = seg;
    M.cu = a->cu_seqlens; M.idx64 = a->idx_dtype == UVMI_I64 ? 1 : 0; M.n_seg = a->n_seg;
    M.N = a->N; M.H = a->H; M.KH = a->KH; M.G = G; M.window = a->window;
    M.scale = a->scale; M.scale_log2 = a->scale * 1.4426950408889634f;
    M.n_wg = ((a->N + 15) / 16) * a->KH;
    const dim3 blk4(256), gq((unsigned)((M.n_wg + 7) / 8 * 8));
    if (a->dtype == UVMI_F16) hipLaunchKernelGGL((bwd_dq_mfma<UVMI_F16>), gq, blk4, 0, st, M);
    else hipLaunchKernelGGL((bwd_dq_mfma<UVMI_BF16>), gq, blk4, 0, st, M);
    UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(dq)");
    M.n_wg = ((a->N + 63) / 64) * a->KH;
    const dim3 gk((unsigned)((M.n_wg + 7) / 8 * 8));
    if (a->dtype == UVMI_F16) hipLaunchKernelGGL((bwd_dkv_mfma<UVMI_F16>), gk, blk4, 0, st, M);
    else hipLaunchKernelGGL((bwd_dkv_mfma<UVMI_BF16>), gk, blk4, 0, st, M);
    UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(dkv)");
    return UVMI_OK;
  }
  // more than 8 query heads per kv head: the plain kernels
  BwdParams P;
  P.q = a->q; P.k = a->k; P.v = a->v; P.o = a->o; P.go = a->go; P.dq = a->dq; P.dk = a->dk; P.dv = a->dv;
  P.lse = lse;
  P.dsum = P.lse + (size_t)a->N * a->H;
  P.cu = a->cu_seqlens; P.idx64 = a->idx_dtype == UVMI_I64 ? 1 : 0; P.n_seg = a->n_seg; P.N = a->N; P.H = a->H; P.KH = a->KH; P.G = a->H / a->KH;
  P.window = a->window; P.scale = a->scale;
  const dim3 blk(64), g1((unsigned)((a->N + 63) / 64), (unsigned)a->H), g2((unsigned)((a->N + 31) / 32), (unsigned)a->KH);
  if (a->dtype == UVMI_F16) hipLaunchKernelGGL((bwd_dq_kernel<UVMI_F16>), g1, blk, 0, st, P);
  else hipLaunchKernelGGL((bwd_dq_kernel<UVMI_BF16>), g1, blk, 0, st, P);
  UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(dq)");
  if (a->dtype == UVMI_F16) hipLaunchKernelGGL((bwd_dkv_kernel<UVMI_F16>), g2, blk, 0, st, P);
  else hipLaunchKernelGGL((bwd_dkv_kernel<UVMI_BF16>), g2, blk, 0, st, P);
  UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(dkv)");
  return UVMI_OK;
}
