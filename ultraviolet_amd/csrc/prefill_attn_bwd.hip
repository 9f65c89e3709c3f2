// Backward of the packed (cu_seqlens) causal attention with an optional sliding window: dq, dk, dv from the output
// gradient (reference: mathk::varlen_attn_bwd, ultraviolet/kernels/varlen_attn.py:56-66, which calls
// aten._efficient_attention_backward on K / V expanded to the query heads and sums their gradients back over a group).
//
// With s_ij = scale q_i . k_j over the keys j query i sees (same segment, i - window < j <= i), p_ij = exp(s_ij - lse_i),
// D_i = go_i . o_i:   dv_j = sum_i p_ij go_i,   ds_ij = p_ij (go_i . v_j - D_i),   dq_i = scale sum_j ds_ij k_j,
// dk_j = scale sum_i ds_ij q_i  (dk, dv also summed over the query heads of the group).
//
// A first, plain form of it: fp32 arithmetic on the vector units, no matrix cores, no atomics, no cross-workgroup state.
//   bwd_dq_kernel   lane = query token (64 per wave), one query head per workgroup: the wave walks the union of its
//                   queries' key ranges; a key / value row is the same address in every lane.  Pass 1 recomputes the
//                   row's log-sum-exp (the forward does not keep it), pass 2 accumulates dq in registers.  Writes
//                   lse and D for the second kernel.
//   bwd_dkv_kernel  two lanes per key (32 head dims each, 32 keys per wave), one kv head per workgroup: the wave walks
//                   the queries that see its keys and the heads of the group; dk and dv stay in registers.
// Both are O(pairs x head_dim) fused multiply-adds per lane: functional, an order of magnitude below what an MFMA form
// would reach.
#include "common.h"

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

}  // namespace uvmi

using namespace uvmi;

extern "C" size_t uvmi_prefill_attn_bwd_workspace_bytes(int N, int H) { return (size_t)2 * (size_t)(N > 0 ? N : 0) * (size_t)(H > 0 ? H : 0) * 4 + 256; }

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
  BwdParams P;
  P.q = a->q; P.k = a->k; P.v = a->v; P.o = a->o; P.go = a->go; P.dq = a->dq; P.dk = a->dk; P.dv = a->dv;
  P.lse = (float*)a->workspace;
  P.dsum = P.lse + (size_t)a->N * a->H;
  P.cu = a->cu_seqlens; P.idx64 = a->idx_dtype == UVMI_I64 ? 1 : 0; P.n_seg = a->n_seg; P.N = a->N; P.H = a->H; P.KH = a->KH; P.G = a->H / a->KH;
  P.window = a->window; P.scale = a->scale;
  hipStream_t st = (hipStream_t)stream;
  const dim3 blk(64), g1((unsigned)((a->N + 63) / 64), (unsigned)a->H), g2((unsigned)((a->N + 31) / 32), (unsigned)a->KH);
  if (a->dtype == UVMI_F16) hipLaunchKernelGGL((bwd_dq_kernel<UVMI_F16>), g1, blk, 0, st, P);
  else hipLaunchKernelGGL((bwd_dq_kernel<UVMI_BF16>), g1, blk, 0, st, P);
  UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(dq)");
  if (a->dtype == UVMI_F16) hipLaunchKernelGGL((bwd_dkv_kernel<UVMI_F16>), g2, blk, 0, st, P);
  else hipLaunchKernelGGL((bwd_dkv_kernel<UVMI_BF16>), g2, blk, 0, st, P);
  UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(dkv)");
  return UVMI_OK;
}
