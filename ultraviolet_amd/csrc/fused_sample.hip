// Fused softcap + categorical draw (inverse CDF, one uniform per row) + behaviour log-prob, and greedy argmax.
//
// Contract (ultraviolet/kernels/fused_sample.py:31-77 of the reference): with z = a*sigmoid((x+b)/c) and
// e = exp((z-a)/T) in (exp(-a/T), 1] (the softcap bounds z, so there is no max pass), S = sum(e),
// target = (1-u)*S; the token is the first index whose running sum reaches target (clamped to V-1) and
// logp = (z_tok - a)/T - log S.  The running sum is hierarchical here (512-element chunks, then lanes, then the
// lane's 8 elements), so the token equals the flat-cumsum one up to fp32 summation order.
//
// e is evaluated as exp2(-(a/T)*log2(e) / (1 + exp2(t*log2(e)))), t = (x+b)/c: algebraically the same as above
// (z - a = -a*sigmoid(-t)) without the cancellation of z - a near the cap.
//
// One workgroup of 256 threads per row streams the row once (HBM-bound: 2 B per logit for bf16/fp16), keeps only
// the 64 chunk sums in LDS, then one wave re-reads the chosen 1 KB chunk (cache-hot).  When u is not supplied it is
// drawn from Philox4x32-10 keyed by the seed with counter (token index, request id lo, request id hi, "SAMP"), so a
// request's stream does not depend on the slot it occupies.
#include "common.h"
#include "sched_commit.h"

namespace uvmi {

constexpr int CHUNK = 512;          // elements per wave pass: 64 lanes x 8
constexpr uint32_t DOMAIN_SAMPLE = 0x53414D50u;

__host__ __device__ inline void philox4x32_10(const uint32_t c_in[4], const uint32_t k_in[2], uint32_t out[4]) {
  uint32_t c0 = c_in[0], c1 = c_in[1], c2 = c_in[2], c3 = c_in[3], k0 = k_in[0], k1 = k_in[1];
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

struct SampleParams {
  const void* x; int64_t stride; const float* u; uint64_t seed; const int64_t* req_id; const int64_t* tok_idx;
  int64_t* tok; float* logp; float* u_out;
  int V;
  float inv_c_l2, b_over_c_l2;  // t*log2(e) = x*inv_c_l2 + b_over_c_l2
  float neg_a_over_t_l2;        // -(a/T)*log2(e)
  float neg_a_over_t;           // -(a/T)
  float cap_a, cap_b, cap_c, inv_c;
  int top_k; float top_p; float* thr_out;
  // optional: commit the drawn token to the slot table in the same launch (row = dense row of a decode step)
  int commit; float retire_p; uint64_t commit_seed; uvmi_sched_state S; DenseArrays D;
};

// The row's result; with P.commit also what uvmi_sched_commit_dense does for the row (one thread per row calls this).
__device__ __forceinline__ void emit(const SampleParams P, int row, int tok, float logp) {
  P.tok[row] = tok;
  P.logp[row] = logp;
  if (P.commit) commit_row<true>(P.S, P.D, row, tok, logp, P.retire_p, P.commit_seed);
}

template <int DT>
__device__ __forceinline__ void load8(const void* row, int i, float (&o)[8]) {  // elements 8i .. 8i+7
  if (DT == UVMI_F32) {
    const float4 a = ((const float4*)row)[2 * i], b = ((const float4*)row)[2 * i + 1];
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
    const uint4 w = ((const uint4*)row)[i];
    const uint32_t r[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (DT == UVMI_BF16) {
        o[2 * j] = __uint_as_float(r[j] << 16);
        o[2 * j + 1] = __uint_as_float(r[j] & 0xffff0000u);
      } else {
        o[2 * j] = half_bits_to_float(r[j] & 0xffff);
        o[2 * j + 1] = half_bits_to_float(r[j] >> 16);
      }
    }
  }
}

__device__ __forceinline__ float e_of(float x, const SampleParams& P) {
  const float E = __builtin_amdgcn_exp2f(fmaf(x, P.inv_c_l2, P.b_over_c_l2));  // exp(t), may be +inf (then e = 1)
  return __builtin_amdgcn_exp2f(P.neg_a_over_t_l2 * __builtin_amdgcn_rcpf(1.0f + E));
}

// (the row pointer's ingredients lead the argument list: leading scalar arguments are preloaded into SGPRs with the wave,
// so the first loads of the row do not wait for a load of the kernel arguments)
// NT threads per row: 256 when there are rows enough to fill the device, 1024 for small batches (the row's exponentials are
// the work of the launch; with one small workgroup per row and fewer rows than compute units most of the device would idle)
template <int DT, int NT>
__global__ __launch_bounds__(NT) void sample_kernel(const void* a_x, int64_t a_stride, int a_V, float a_inv_c_l2, float a_b_over_c_l2,
                                                    float a_neg_a_over_t_l2, SampleParams P) {
  P.x = a_x; P.stride = a_stride; P.V = a_V; P.inv_c_l2 = a_inv_c_l2; P.b_over_c_l2 = a_b_over_c_l2; P.neg_a_over_t_l2 = a_neg_a_over_t_l2;
  __shared__ float csum[64 + 4];
  __shared__ int sh_chunk;
  __shared__ float sh_before, sh_total, sh_target;
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const char* xr = (const char*)P.x + (int64_t)row * P.stride * (DT == UVMI_F32 ? 4 : 2);
  const int nchunks = P.V / CHUNK;  // host guarantees V % 512 == 0 and nchunks <= 64
  for (int c = wave; c < nchunks; c += NT / 64) {
    float v[8];
    load8<DT>(xr, c * 64 + lane, v);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) s += e_of(v[j], P);
    s = wave_sum(s);
    if (lane == 0) csum[c] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  // ---- wave 0: pick the chunk, then the lane, then the element
  float mine = lane < nchunks ? csum[lane] : 0.f;
  float incl = mine;  // inclusive scan over chunks in lane order
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  const float S = __shfl(incl, 63, 64);
  float u;
  if (P.u) {
    u = P.u[row];
  } else {
    const uint64_t rid = (uint64_t)P.req_id[row], ti = (uint64_t)P.tok_idx[row];
    const uint32_t ctr[4] = {(uint32_t)ti, (uint32_t)rid, (uint32_t)(rid >> 32), DOMAIN_SAMPLE};
    const uint32_t key[2] = {(uint32_t)P.seed, (uint32_t)(P.seed >> 32)};
    uint32_t o[4];
    philox4x32_10(ctr, key, o);
    u = (float)(o[0] >> 8) * 5.9604644775390625e-08f;  // 2^-24
  }
  const float target = (1.0f - u) * S;
  const unsigned long long below = __ballot(lane < nchunks && incl < target);
  int ck = __popcll(below);  // first chunk whose inclusive sum reaches target
  if (ck > nchunks - 1) ck = nchunks - 1;
  const float before = ck > 0 ? __shfl(incl, ck - 1, 64) : 0.f;
  float v[8], e[8];
  load8<DT>(xr, ck * 64 + lane, v);
  float ls = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    e[j] = e_of(v[j], P);
    ls += e[j];
  }
  float linc = ls;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(linc, o, 64);
    if (lane >= o) linc += t;
  }
  linc += before;
  const unsigned long long lb = __ballot(linc < target);
  int ln = __popcll(lb);
  if (ln > 63) ln = 63;
  // every lane recomputes the winner lane's walk from broadcast values (uniform control flow)
  float run = ln > 0 ? __shfl(linc, ln - 1, 64) : before;
  int jsel = 7;
  bool found = false;
  float xsel = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const float ej = __shfl(e[j], ln, 64), xj = __shfl(v[j], ln, 64);
    run += ej;
    if (!found && run >= target) { found = true; jsel = j; xsel = xj; }
    if (j == 7 && !found) xsel = xj;
  }
  if (lane == 0) {
    const int tok = ck * CHUNK + ln * 8 + jsel;
    // logp = (z_tok - a)/T - log S, with (z - a)/T = -(a/T) / (1 + exp(t))
    const float E = __builtin_amdgcn_exp2f(fmaf(xsel, P.inv_c_l2, P.b_over_c_l2));
    if (P.u_out) P.u_out[row] = u;
    emit(P, row, tok, P.neg_a_over_t * __builtin_amdgcn_rcpf(1.0f + E) - __logf(S));
  }
}

// Top-k / nucleus sampling (sample() of the reference, ultraviolet/model.py:1194-1211): keep the tokens whose value is at
// least the k-th largest, then of those the smallest prefix by probability whose mass reaches top_p (the token that
// crosses it included, ties of the last kept value all kept), and draw from what is kept by inverse CDF in index order.
// Everything is decided on e = exp((z - a)/T), which is positive and monotone in the logit, so its fp32 bit pattern
// orders the tokens: both thresholds are found by a radix select over those 32 bits, 8 bits per sweep of the row (the row
// stays in cache between sweeps).  The nucleus select walks the digits by probability mass; masses are summed as 32.32
// fixed point in 64-bit integers, so the histogram does not depend on the order in which lanes add to it.  The behaviour
// log-prob is that of the unfiltered softmax, as the reference records it (model.py:1161-1169).
template <int DT>
__global__ __launch_bounds__(256) void sample_filtered_kernel(SampleParams P) {
  __shared__ float csum[64 + 4];
  __shared__ unsigned int hcnt[256];
  __shared__ unsigned long long hmass[256];
  __shared__ unsigned int sh_prefix, sh_krem;
  __shared__ unsigned long long sh_mhi, sh_zk;
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tid = threadIdx.x;
  const char* xr = (const char*)P.x + (int64_t)row * P.stride * (DT == UVMI_F32 ? 4 : 2);
  const int nchunks = P.V / CHUNK;
  const int nvec = P.V / 8;
  auto fix = [](float e) -> unsigned long long { return (unsigned long long)((double)e * 4294967296.0); };

  // ---- unfiltered sum S (for the log-prob), in the order of the unfiltered kernel
  for (int c = wave; c < nchunks; c += 4) {
    float v[8];
    load8<DT>(xr, c * 64 + lane, v);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) s += e_of(v[j], P);
    s = wave_sum(s);
    if (lane == 0) csum[c] = s;
  }
  __syncthreads();
  float S = 0.f;
  for (int c = 0; c < nchunks; c++) S += csum[c];
  __syncthreads();

  // ---- top-k: the k-th largest key
  unsigned int thr = 0;  // keep keys >= thr
  if (P.top_k > 0 && P.top_k < P.V) {
    unsigned int prefix = 0, mask = 0, krem = (unsigned int)P.top_k;
    for (int shift = 24; shift >= 0; shift -= 8) {
      hcnt[tid] = 0;
      __syncthreads();
      for (int i = tid; i < nvec; i += 256) {
        float v[8];
        load8<DT>(xr, i, v);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const unsigned int key = __float_as_uint(e_of(v[j], P));
          if ((key & mask) == prefix) atomicAdd(&hcnt[(key >> shift) & 255u], 1u);
        }
      }
      __syncthreads();
      if (tid == 0) {
        unsigned int c = 0;
        int d = 255;
        for (; d > 0; d--) {
          if (c + hcnt[d] >= krem) break;
          c += hcnt[d];
        }
        sh_prefix = prefix | ((unsigned int)d << shift);
        sh_krem = krem - c;
      }
      __syncthreads();
      prefix = sh_prefix; krem = sh_krem;
      mask |= 255u << shift;
      __syncthreads();
    }
    thr = prefix;
  }

  // ---- nucleus: the smallest key whose mass of strictly larger keys is below top_p * (mass of the top-k set)
  if (P.top_p < 1.0f) {
    if (tid == 0) sh_zk = 0;
    __syncthreads();
    unsigned long long part = 0;
    for (int i = tid; i < nvec; i += 256) {
      float v[8];
      load8<DT>(xr, i, v);
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const float e = e_of(v[j], P);
        if (__float_as_uint(e) >= thr) part += fix(e);
      }
    }
    atomicAdd(&sh_zk, part);
    __syncthreads();
    const double tp = P.top_p > 0.f ? (double)P.top_p : 0.0;
    const unsigned long long target = (unsigned long long)(tp * (double)sh_zk);
    unsigned int prefix = 0, mask = 0;
    unsigned long long mhi = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
      hcnt[tid] = 0;
      hmass[tid] = 0;
      __syncthreads();
      for (int i = tid; i < nvec; i += 256) {
        float v[8];
        load8<DT>(xr, i, v);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const float e = e_of(v[j], P);
          const unsigned int key = __float_as_uint(e);
          if (key >= thr && (key & mask) == prefix) {
            const unsigned int d = (key >> shift) & 255u;
            atomicAdd(&hcnt[d], 1u);
            atomicAdd(&hmass[d], fix(e));
          }
        }
      }
      __syncthreads();
      if (tid == 0) {
        // walk the digits downwards; `run` is the mass above the digit.  The last non-empty digit reached while run <
        // target holds the cut; when even the largest key fails (top_p = 0) it is kept anyway, as the first token is.
        unsigned long long run = mhi, above = mhi;
        int dsel = -1;
        for (int d = 255; d >= 0; d--) {
          if (hcnt[d] == 0) continue;
          if (dsel >= 0 && run >= target) break;
          dsel = d; above = run;
          run += hmass[d];
        }
        if (dsel < 0) dsel = 0;
        sh_prefix = prefix | ((unsigned int)dsel << shift);
        sh_mhi = above;
      }
      __syncthreads();
      prefix = sh_prefix; mhi = sh_mhi;
      mask |= 255u << shift;
      __syncthreads();
    }
    thr = prefix;  // (a key of the top-k set, so >= the top-k threshold)
  }
  auto e_kept = [&](float x) -> float {
    const float e = e_of(x, P);
    return __float_as_uint(e) >= thr ? e : 0.f;
  };

  // ---- draw from the kept tokens: chunk sums, then the chunk, the lane, the element (as the unfiltered kernel)
  for (int c = wave; c < nchunks; c += 4) {
    float v[8];
    load8<DT>(xr, c * 64 + lane, v);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) s += e_kept(v[j]);
    s = wave_sum(s);
    if (lane == 0) csum[c] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  float incl = lane < nchunks ? csum[lane] : 0.f;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  const float Sk = __shfl(incl, 63, 64);
  float u;
  if (P.u) {
    u = P.u[row];
  } else {
    const uint64_t rid = (uint64_t)P.req_id[row], ti = (uint64_t)P.tok_idx[row];
    const uint32_t ctr[4] = {(uint32_t)ti, (uint32_t)rid, (uint32_t)(rid >> 32), DOMAIN_SAMPLE};
    const uint32_t key[2] = {(uint32_t)P.seed, (uint32_t)(P.seed >> 32)};
    uint32_t o[4];
    philox4x32_10(ctr, key, o);
    u = (float)(o[0] >> 8) * 5.9604644775390625e-08f;  // 2^-24
  }
  const float target = (1.0f - u) * Sk;
  const unsigned long long below = __ballot(lane < nchunks && incl < target);
  int ck = __popcll(below);
  if (ck > nchunks - 1) ck = nchunks - 1;
  // (a chunk without kept tokens has the inclusive sum of its predecessor, which is < target whenever it is chosen over,
  // so the chosen chunk always holds a kept token unless rounding pushed target past the total: then walk back)
  while (ck > 0 && (ck > 0 ? __shfl(incl, ck - 1, 64) : 0.f) >= Sk) ck--;
  const float before = ck > 0 ? __shfl(incl, ck - 1, 64) : 0.f;
  float v[8], e[8];
  load8<DT>(xr, ck * 64 + lane, v);
  float ls = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    e[j] = e_kept(v[j]);
    ls += e[j];
  }
  float linc = ls;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(linc, o, 64);
    if (lane >= o) linc += t;
  }
  linc += before;
  // the lane: the first one whose inclusive sum reaches target and that holds a kept token; when rounding pushed target
  // past the chunk's total, the last lane that holds one
  const unsigned long long has = __ballot(ls > 0.f);
  int ln = __popcll(__ballot(linc < target));
  {
    const unsigned long long hi = ln < 64 ? has & ~((1ull << ln) - 1ull) : 0ull;
    ln = hi ? __ffsll((long long)hi) - 1 : (has ? 63 - __clzll((long long)has) : 0);
  }
  // every lane recomputes that lane's walk from broadcast values: the first kept element whose running sum reaches
  // target, else the lane's last kept element
  float run = ln > 0 ? __shfl(linc, ln - 1, 64) : before;
  int sel = ln * 8;
  float xsel = __shfl(v[0], ln, 64);
  bool found = false;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const float ej = __shfl(e[j], ln, 64), xj = __shfl(v[j], ln, 64);
    if (ej > 0.f && !found) {
      run += ej;
      sel = ln * 8 + j; xsel = xj;
      if (run >= target) found = true;
    }
  }
  if (lane == 0) {
    const float E = __builtin_amdgcn_exp2f(fmaf(xsel, P.inv_c_l2, P.b_over_c_l2));
    if (P.u_out) P.u_out[row] = u;
    if (P.thr_out) P.thr_out[row] = __uint_as_float(thr);
    emit(P, row, ck * CHUNK + sel, P.neg_a_over_t * __builtin_amdgcn_rcpf(1.0f + E) - __logf(S));
  }
}

// Greedy: argmax of the raw head output (the softcap is strictly increasing, so argmax z = argmax x), first maximal
// index; logp = log softmax(z)[tok] at T = 1.
template <int DT>
__global__ __launch_bounds__(256) void argmax_kernel(SampleParams P) {
  __shared__ float smax[4];
  __shared__ int sidx[4];
  __shared__ float ssum[4];
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const char* xr = (const char*)P.x + (int64_t)row * P.stride * (DT == UVMI_F32 ? 4 : 2);
  const int nvec = P.V / 8;
  float best = -INFINITY, esum = 0.f;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < nvec; i += 256) {
    float v[8];
    load8<DT>(xr, i, v);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      if (v[j] > best) { best = v[j]; bi = i * 8 + j; }
      // softmax(z) with T = 1: e = exp(z - a)
      const float E = __builtin_amdgcn_exp2f(fmaf(v[j], P.inv_c_l2, P.b_over_c_l2));
      esum += __builtin_amdgcn_exp2f(-P.cap_a * 1.4426950408889634f * __builtin_amdgcn_rcpf(1.0f + E));
    }
  }
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
  }
  esum = wave_sum(esum);
  if (lane == 0) { smax[wave] = best; sidx[wave] = bi; ssum[wave] = esum; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float tot = 0.f;
    for (int w = 0; w < 4; w++) {
      tot += ssum[w];
      if (smax[w] > best || (smax[w] == best && sidx[w] < bi)) { best = smax[w]; bi = sidx[w]; }
    }
    const float E = __builtin_amdgcn_exp2f(fmaf(best, P.inv_c_l2, P.b_over_c_l2));
    if (P.u_out) P.u_out[row] = 0.f;
    emit(P, row, bi, -P.cap_a * __builtin_amdgcn_rcpf(1.0f + E) - __logf(tot));
  }
}

}  // namespace uvmi

using namespace uvmi;

extern "C" void uvmi_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) { philox4x32_10(ctr, key, out); }

extern "C" int uvmi_fused_sample(const uvmi_sample_args* a, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_fused_sample: null args");
  UVMI_REQUIRE(a->x && a->tok && a->logp, UVMI_EINVAL, "uvmi_fused_sample: null pointer");
  UVMI_REQUIRE(is_float_dtype(a->x_dtype), UVMI_EINVAL, "uvmi_fused_sample: x_dtype must be a float type");
  UVMI_REQUIRE(a->B >= 0 && a->V > 0 && a->stride >= a->V, UVMI_EINVAL, "uvmi_fused_sample: bad sizes");
  UVMI_REQUIRE(a->V % CHUNK == 0 && a->V / CHUNK <= 64, UVMI_EUNSUPPORTED,
               "uvmi_fused_sample: V=%d must be a multiple of 512 and at most 32768", a->V);
  UVMI_REQUIRE(a->cap_c != 0.f, UVMI_EINVAL, "uvmi_fused_sample: softcap c must be non-zero");
  const int eb = a->x_dtype == UVMI_F32 ? 4 : 2;
  UVMI_REQUIRE(((uintptr_t)a->x % 16) == 0 && (a->stride * eb) % 16 == 0, UVMI_EUNSUPPORTED,
               "uvmi_fused_sample: rows of x must be 16-byte aligned");
  const bool greedy = !(a->temperature > 0.f);
  if (!greedy) {
    UVMI_REQUIRE(a->cap_a / a->temperature <= 80.0f, UVMI_EUNSUPPORTED, "uvmi_fused_sample: a/T = %g exceeds 80 (fp32 underflow)",
                 (double)(a->cap_a / a->temperature));
    UVMI_REQUIRE(a->u || (a->req_id && a->tok_idx), UVMI_EINVAL, "uvmi_fused_sample: need u or (req_id, tok_idx)");
  }
  if (a->B == 0) return UVMI_OK;
  SampleParams P;
  P.x = a->x; P.stride = a->stride; P.u = a->u; P.seed = a->seed; P.req_id = a->req_id; P.tok_idx = a->tok_idx;
  P.tok = a->tok; P.logp = a->logp; P.u_out = a->u_out; P.V = a->V;
  const float l2e = 1.4426950408889634f;
  P.inv_c = 1.0f / a->cap_c;
  P.inv_c_l2 = l2e / a->cap_c;
  P.b_over_c_l2 = a->cap_b / a->cap_c * l2e;
  const float T = greedy ? 1.0f : a->temperature;
  P.neg_a_over_t = -a->cap_a / T;
  P.neg_a_over_t_l2 = P.neg_a_over_t * l2e;
  P.cap_a = a->cap_a; P.cap_b = a->cap_b; P.cap_c = a->cap_c;
  P.top_k = a->top_k > 0 && a->top_k < a->V ? a->top_k : 0;
  P.top_p = a->top_p > 0.f && a->top_p < 1.0f ? a->top_p : 1.0f;
  P.thr_out = a->thr_out;
  P.commit = 0;
  if (a->commit) {
    const uvmi_sample_commit* c = a->commit;
    UVMI_REQUIRE(c->state && c->act_slot && c->tok_c && c->pos_c && c->starts_c && c->req_c && c->cnt_c, UVMI_EINVAL,
                 "uvmi_fused_sample: null pointer in commit");
    const uvmi_sched_state* t = c->state;
    UVMI_REQUIRE(t->slot_req && t->slot_cnt && t->slot_limit && t->slot_tok && t->pos && t->starts && t->out_tok && t->counters && t->done_req &&
                     t->done_slot && t->done_cnt && t->B > 0 && t->max_new > 0 && t->done_cap > 0, UVMI_EINVAL,
                 "uvmi_fused_sample: bad slot table in commit");
    // the kernel reads req_id / tok_idx of a row before it rewrites the row's dense entries, so they may be the same arrays
    P.commit = 1; P.retire_p = c->retire_p; P.commit_seed = c->seed; P.S = *t;
    P.D = DenseArrays{c->act_slot, c->tok_c, c->pos_c, c->starts_c, c->req_c, c->cnt_c};
  }
  const bool filtered = !greedy && (P.top_k > 0 || P.top_p < 1.0f);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(a->B), blk(256);
#define UVMI_S(K)                                                                          \
  do {                                                                                     \
    if (a->x_dtype == UVMI_F16) hipLaunchKernelGGL((K<UVMI_F16>), grid, blk, 0, st, P);    \
    else if (a->x_dtype == UVMI_BF16) hipLaunchKernelGGL((K<UVMI_BF16>), grid, blk, 0, st, P); \
    else hipLaunchKernelGGL((K<UVMI_F32>), grid, blk, 0, st, P);                           \
  } while (0)
  if (greedy) UVMI_S(argmax_kernel);
  else if (filtered) UVMI_S(sample_filtered_kernel);
  else {
#define UVMI_SK(DT, NT) \
  hipLaunchKernelGGL((sample_kernel<DT, NT>), grid, dim3(NT), 0, st, P.x, P.stride, P.V, P.inv_c_l2, P.b_over_c_l2, P.neg_a_over_t_l2, P)
    // 1024 threads per row are faster up to ~640 rows (measured: 12.0 against 14.5 us at 384 rows), slower from 1024 on; the
    // chunk sums are formed per chunk whatever the width, so the draw does not depend on it
    const bool wide = a->B <= 640;
    if (a->x_dtype == UVMI_F16) { if (wide) UVMI_SK(UVMI_F16, 1024); else UVMI_SK(UVMI_F16, 256); }
    else if (a->x_dtype == UVMI_BF16) { if (wide) UVMI_SK(UVMI_BF16, 1024); else UVMI_SK(UVMI_BF16, 256); }
    else { if (wide) UVMI_SK(UVMI_F32, 1024); else UVMI_SK(UVMI_F32, 256); }
#undef UVMI_SK
  }
#undef UVMI_S
  UVMI_CHECK_LAUNCH("uvmi_fused_sample");
  return UVMI_OK;
}
