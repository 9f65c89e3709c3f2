// On-device continuous-batching bookkeeping: the slot table of the reference's host loop
// (generate_continuous, ultraviolet/model.py:1283-1350; StreamGen, scripts/rl_stream.py:55-146) kept in HBM and
// advanced by a few tiny kernels per decode step, so a step needs no host synchronisation:
//
//   sched_expand   per-token position / cache-row tables of the prompts admitted with a step, from their cu_seqlens;
//   sched_compact  scan the slot table, list the active slots first (ascending), gather their token / position /
//                  request id / token index into dense arrays of a fixed bucket length (padding rows get slot -1);
//   sched_commit   scatter the sampled token and its log-prob into the slot's output row, advance count and position,
//                  retire on EOS / length limit / seeded Bernoulli(p), park retired rows at position 0 and append a
//                  completion record for the host to harvest asynchronously; its dense form also carries the step's dense
//                  arrays to the next step (retired rows become padding where they stand), so that only the first
//                  step after an admission or a change of bucket needs a compaction;
//   sched_harvest  pack new completion records and their output rows for the host's copy.
//
// Both are integer bookkeeping on <= a few thousand slots: latency-bound, one workgroup / one thread per row.
#include "common.h"
#include "sched_commit.h"

namespace uvmi {

// One workgroup of 1024 threads; slots are handled in tiles of 1024 with a running base (ordered compaction).
__device__ __forceinline__ void compact_phase(const uvmi_sched_state& S, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c,
                                              int64_t* starts_c, int64_t* req_c, int64_t* cnt_c, int* wsum, int& base_sh) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) base_sh = 0;
  __syncthreads();
  for (int t0 = 0; t0 < S.B; t0 += 1024) {
    const int slot = t0 + tid;
    const bool act = slot < S.B && S.slot_req[slot] >= 0;
    const unsigned long long bal = __ballot(act);
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wsum[wave] = __popcll(bal);
    __syncthreads();
    int woff = 0;
    for (int w = 0; w < wave; w++) woff += wsum[w];
    const int base = base_sh;
    if (act) {
      const int i = base + woff + before;
      if (i < n_bucket) {
        act_slot[i] = slot;
        tok_c[i] = S.slot_tok[slot];
        pos_c[i] = S.pos[slot];
        starts_c[i] = S.starts[slot];
        req_c[i] = S.slot_req[slot];
        cnt_c[i] = S.slot_cnt[slot];
      }
    }
    __syncthreads();
    if (tid == 0) {
      int tot = 0;
      for (int w = 0; w < 16; w++) tot += wsum[w];
      base_sh = base + tot;
    }
    __syncthreads();
  }
  const int n_act = base_sh;
  for (int i = n_act + tid; i < n_bucket; i += 1024) {
    act_slot[i] = -1; tok_c[i] = 0; pos_c[i] = 0; starts_c[i] = 0; req_c[i] = 0; cnt_c[i] = 0;
  }
  if (tid == 0) {
    S.counters[0] = n_act;                              // active slots seen by this step
    if (n_act > n_bucket) S.counters[2] = 1;            // bucket too small: the overflow slots idle this step
  }
  __syncthreads();
}

__global__ __launch_bounds__(1024) void sched_compact_kernel(uvmi_sched_state S, int n_bucket, int64_t* act_slot, int64_t* tok_c,
                                                             int64_t* pos_c, int64_t* starts_c, int64_t* req_c, int64_t* cnt_c) {
  __shared__ int wsum[16];
  __shared__ int base_sh;
  compact_phase(S, n_bucket, act_slot, tok_c, pos_c, starts_c, req_c, cnt_c, wsum, base_sh);
}

// One thread per dense row (see commit_row).
template <bool DENSE>
__global__ __launch_bounds__(256) void sched_commit_kernel(uvmi_sched_state S, int n_bucket, DenseArrays D, const int64_t* new_tok,
                                                           const float* new_lp, float retire_p, uint64_t seed) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n_bucket) return;
  commit_row<DENSE>(S, D, i, new_tok[i], new_lp ? new_lp[i] : 0.f, retire_p, seed);
}

// Admission after a prefill: bind request ids to slots and record the first sampled token (it counts as token 0 of
// the request: model.py:1306-1313, rl_stream.py:86-92).  pos / starts were set by the prefill.
__global__ __launch_bounds__(256) void sched_admit_kernel(uvmi_sched_state S, int n, const int64_t* slots, const int64_t* req_ids,
                                                          const int64_t* limits, const int64_t* first_tok, const float* first_lp) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int64_t slot = slots[i];
  if (slot < 0 || slot >= S.B) return;
  S.slot_req[slot] = req_ids[i];
  S.slot_limit[slot] = limits[i];
  S.slot_tok[slot] = first_tok[i];
  S.slot_cnt[slot] = 1;
  S.out_tok[slot * S.max_new] = (int32_t)first_tok[i];
  if (S.out_lp) S.out_lp[slot * S.max_new] = first_lp ? first_lp[i] : 0.f;
  const bool fin = limits[i] <= 1 || (S.eos_id >= 0 && first_tok[i] == S.eos_id);
  if (fin) {
    const int k = atomicAdd(&S.counters[1], 1) % S.done_cap;
    S.done_req[k] = req_ids[i]; S.done_slot[k] = slot; S.done_cnt[k] = 1;
    S.slot_req[slot] = -1;
    if (S.slot_hold) S.slot_hold[slot] = 1;
    S.pos[slot] = 0;
    S.starts[slot] = 0;
  }
}

// The admission of a step planned on the device (see uvmi_sched_plan_admit): one workgroup of 1024 threads.  Phase 1 lists
// the first admit_cap reusable slots in ascending order (ballot / popcount prefix over tiles of 1024 slots, as the
// compaction does); phase 2 (one thread) walks the staged ring from its head while slots, the prompt cap and the token
// budget last; phase 3 (all threads) writes the tables and copies the admitted prompts' tokens back to back.
constexpr int PLAN_MAXA = 256;
struct PlanShared {
  int wsum[16];
  int base, na, tmax;
  int free_slot[PLAN_MAXA];
  int cu[PLAN_MAXA + 1];
};

__device__ __forceinline__ void plan_phase(const uvmi_sched_state& S, int A, int n_tokens, int left_pad, int64_t* adm_cu, int64_t* adm_slot,
                                           int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req, int64_t* tok_packed, PlanShared& sh) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) sh.base = 0;
  __syncthreads();
  for (int t0 = 0; t0 < S.B && sh.base < A; t0 += 1024) {
    const int slot = t0 + tid;
    const bool fr = slot < S.B && S.slot_req[slot] < 0 && !(S.slot_hold && S.slot_hold[slot]);
    const unsigned long long bal = __ballot(fr);
    const int before = __popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) sh.wsum[wave] = __popcll(bal);
    __syncthreads();
    int woff = 0;
    for (int w = 0; w < wave; w++) woff += sh.wsum[w];
    const int base = sh.base;
    if (fr && base + woff + before < A) sh.free_slot[base + woff + before] = slot;
    __syncthreads();
    if (tid == 0) {
      int tot = 0;
      for (int w = 0; w < 16; w++) tot += sh.wsum[w];
      sh.base = base + tot;
    }
    __syncthreads();
  }
  const int64_t head = S.q_ctl[1], tail = S.q_ctl[0];
  __syncthreads();   // (every thread has read the head before one thread moves it)
  if (tid == 0) {
    const int nfree = sh.base < A ? sh.base : A;
    int na = 0, ntok = 0, tmax = 0;
    sh.cu[0] = 0;
    while (na < nfree && head + na < tail) {
      const int64_t* row = S.q_buf + ((head + na) % S.q_cap) * (int64_t)S.q_stride;
      int len = (int)row[0];
      len = len < 0 ? 0 : (len > S.q_stride - 3 ? S.q_stride - 3 : len);
      if (ntok + len > n_tokens) break;
      ntok += len;
      tmax = len > tmax ? len : tmax;
      sh.cu[++na] = ntok;
    }
    sh.na = na;
    sh.tmax = tmax;
    S.q_ctl[1] = head + na;
    S.q_ctl[2] = na;
  }
  __syncthreads();
  const int na = sh.na, total = sh.cu[na];
  for (int a = tid; a <= A; a += 1024) adm_cu[a] = a <= na ? sh.cu[a] : total;
  for (int a = tid; a < A; a += 1024) {
    const bool ok = a < na;
    const int64_t* row = S.q_buf + ((head + (ok ? a : 0)) % S.q_cap) * (int64_t)S.q_stride;
    adm_slot[a] = ok ? sh.free_slot[a] : -1;
    adm_start[a] = ok && left_pad ? sh.tmax - (sh.cu[a + 1] - sh.cu[a]) : 0;
    adm_limit[a] = ok ? row[2] : 0;
    adm_req[a] = ok ? row[1] : 0;
  }
  // tokens: packed token i belongs to the prompt a with cu[a] <= i < cu[a + 1] (binary search, na <= 256)
  for (int i = tid; i < n_tokens; i += 1024) {
    int64_t v = 0;
    if (i < total) {
      int lo = 0, hi = na;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (sh.cu[mid] <= i) lo = mid; else hi = mid;
      }
      v = S.q_buf[((head + lo) % S.q_cap) * (int64_t)S.q_stride + 3 + (i - sh.cu[lo])];
    }
    tok_packed[i] = v;
  }
  __syncthreads();
}

__global__ __launch_bounds__(1024) void sched_plan_admit_kernel(uvmi_sched_state S, int A, int n_tokens, int left_pad, int64_t* adm_cu,
                                                                int64_t* adm_slot, int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req,
                                                                int64_t* tok_packed) {
  __shared__ PlanShared sh;
  plan_phase(S, A, n_tokens, left_pad, adm_cu, adm_slot, adm_start, adm_limit, adm_req, tok_packed, sh);
}

// The whole bookkeeping ahead of a step that admits prompts, in one launch of one workgroup: the compaction of the active
// slots, the admission plan, and the per-token tables of the admitted prompts (what uvmi_sched_compact, uvmi_sched_plan_admit
// and uvmi_sched_expand do in three).
__global__ __launch_bounds__(1024) void sched_step_plan_kernel(uvmi_sched_state S, int n_bucket, int64_t* act_slot, int64_t* tok_c,
                                                               int64_t* pos_c, int64_t* starts_c, int64_t* req_c, int64_t* cnt_c, int A,
                                                               int n_tokens, int left_pad, int64_t* adm_cu, int64_t* adm_slot,
                                                               int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req, int64_t* tok_packed,
                                                               int64_t* pos_t, int64_t* row_t, int64_t* last_t, int64_t* last_idx, int64_t* last_c) {
  __shared__ PlanShared sh;
  compact_phase(S, n_bucket, act_slot, tok_c, pos_c, starts_c, req_c, cnt_c, sh.wsum, sh.base);
  if (last_c)   // a decode row's own position is the last position it may attend (and append at)
    for (int i = threadIdx.x; i < n_bucket; i += 1024) last_c[i] = pos_c[i];
  plan_phase(S, A, n_tokens, left_pad, adm_cu, adm_slot, adm_start, adm_limit, adm_req, tok_packed, sh);
  const int tid = threadIdx.x, na = sh.na;
  for (int a = tid; a < A; a += 1024) {
    const bool ok = a < na && sh.cu[a + 1] > sh.cu[a];
    last_idx[a] = ok ? sh.cu[a + 1] - 1 : 0;
    if (ok) {
      const int slot = sh.free_slot[a], st = left_pad ? sh.tmax - (sh.cu[a + 1] - sh.cu[a]) : 0;
      S.starts[slot] = st;
      S.pos[slot] = st + (sh.cu[a + 1] - sh.cu[a]);
    }
  }
  const int total = sh.cu[na];
  for (int i = tid; i < n_tokens; i += 1024) {
    int64_t p = 0, r = -1, l = 0;
    if (i < total) {
      int lo = 0, hi = na;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (sh.cu[mid] <= i) lo = mid; else hi = mid;
      }
      const int st = left_pad ? sh.tmax - (sh.cu[lo + 1] - sh.cu[lo]) : 0;
      p = st + (i - sh.cu[lo]);
      r = sh.free_slot[lo];
      l = st + (sh.cu[lo + 1] - sh.cu[lo]) - 1;
    }
    pos_t[i] = p; row_t[i] = r; last_t[i] = l;
  }
}

// Per-token tables of a packed prefill built on the device from its cu_seqlens (the reference builds them on the host
// for every refill: prefill_packed_host, ultraviolet/kernels/fast_decode.py:210-269).  One thread per packed token:
// binary search of its prompt, then position / cache row / last position; tokens past cu[n_adm] are padding (row -1).
// The first n_adm threads also record the packed index of their prompt's last token and point the slot at its prompt
// (starts = first position, pos = next position to write).
__global__ __launch_bounds__(256) void sched_expand_kernel(uvmi_sched_state S, int n_adm, int n_tokens, const int64_t* cu,
                                                           const int64_t* adm_slot, const int64_t* adm_start, int64_t* pos_t,
                                                           int64_t* row_t, int64_t* last_t, int64_t* last_idx) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n_adm) {
    const int64_t n = cu[i + 1] - cu[i], slot = adm_slot[i];
    const bool ok = n > 0 && slot >= 0 && slot < S.B;
    last_idx[i] = ok ? cu[i + 1] - 1 : 0;
    if (ok) {
      S.starts[slot] = adm_start[i];
      S.pos[slot] = adm_start[i] + n;
    }
  }
  if (i >= n_tokens) return;
  int lo = 0, hi = n_adm;  // invariant: cu[lo] <= i, and hi == n_adm or cu[hi] > i
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= i) lo = mid; else hi = mid;
  }
  const int64_t slot = adm_slot[lo];
  const bool real = i < cu[n_adm] && i < cu[lo + 1] && slot >= 0 && slot < S.B;
  pos_t[i] = real ? adm_start[lo] + (i - cu[lo]) : 0;
  row_t[i] = real ? slot : -1;
  last_t[i] = real ? adm_start[lo] + (cu[lo + 1] - cu[lo]) - 1 : 0;
}

// Completion records seen .. min(seen + max_rows, written) and their output rows, packed back to back for one small
// device->host copy of the header and one of exactly the finished tokens.  One workgroup per record.
__global__ __launch_bounds__(256) void sched_harvest_kernel(uvmi_sched_state S, int64_t seen, int max_rows, int64_t* hdr, int32_t* tok_dst,
                                                            float* lp_dst) {
  __shared__ int64_t wsum[4];
  const int j = blockIdx.x, tid = threadIdx.x;
  int64_t k = (int64_t)S.counters[1] - seen;
  k = k < 0 ? 0 : (k > max_rows ? max_rows : k);
  if (j == 0 && tid < 4) hdr[tid] = tid < 3 ? (int64_t)S.counters[tid] : k;
  if (j == gridDim.x - 1) {   // the last workgroup (never one with a long copy ahead of it) counts the active slots
    int64_t n = 0;
    for (int s0 = tid; s0 < S.B; s0 += 256) n += S.slot_req[s0] >= 0;
    for (int o = 32; o > 0; o >>= 1) n += __shfl_xor(n, o, 64);
    if ((tid & 63) == 0) wsum[tid >> 6] = n;
    __syncthreads();
    if (tid == 0) {
      int64_t* x = hdr + 4 + 4 * (int64_t)max_rows;
      x[0] = wsum[0] + wsum[1] + wsum[2] + wsum[3];
      x[1] = S.q_ctl ? S.q_ctl[1] : 0;
      x[2] = S.q_ctl ? S.q_ctl[2] : 0;
      x[3] = 0;
    }
    __syncthreads();
  }
  if (j >= k) return;
  auto count_of = [&](int64_t rec) {
    const int64_t c = S.done_cnt[rec % S.done_cap];
    return c < 0 ? 0 : (c > S.max_new ? S.max_new : c);
  };
  int64_t part = 0;
  for (int i = tid; i < j; i += 256) part += count_of(seen + i);
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
  if ((tid & 63) == 0) wsum[tid >> 6] = part;
  __syncthreads();
  const int64_t off = wsum[0] + wsum[1] + wsum[2] + wsum[3];
  const int64_t e = (seen + j) % S.done_cap;
  const int64_t slot = S.done_slot[e];
  const bool ok = slot >= 0 && slot < S.B;
  const int64_t cnt = ok ? count_of(seen + j) : 0;
  if (tid == 0) {
    int64_t* h = hdr + 4 + 4 * j;
    h[0] = S.done_req[e];
    h[1] = slot;
    h[2] = cnt;
    h[3] = off;
  }
  const int32_t* src_t = S.out_tok + slot * S.max_new;
  const float* src_l = S.out_lp ? S.out_lp + slot * S.max_new : nullptr;
  for (int64_t t = tid; t < cnt; t += 256) {
    tok_dst[off + t] = src_t[t];
    if (lp_dst && src_l) lp_dst[off + t] = src_l[t];
  }
  if (S.slot_hold && ok) {   // the row is packed: the slot may be handed out again
    __syncthreads();
    if (tid == 0) S.slot_hold[slot] = 0;
  }
}

static int check_state(const uvmi_sched_state* s, const char* who) {
  UVMI_REQUIRE(s, UVMI_EINVAL, "%s: null state", who);
  UVMI_REQUIRE(s->slot_req && s->slot_cnt && s->slot_limit && s->slot_tok && s->pos && s->starts && s->out_tok && s->counters &&
                   s->done_req && s->done_slot && s->done_cnt, UVMI_EINVAL, "%s: null pointer in state", who);
  UVMI_REQUIRE(s->B > 0 && s->B <= (1 << 20) && s->max_new > 0 && s->done_cap > 0, UVMI_EINVAL, "%s: bad sizes", who);
  return UVMI_OK;
}

}  // namespace uvmi

using namespace uvmi;

extern "C" int uvmi_sched_compact(const uvmi_sched_state* s, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c,
                                  int64_t* starts_c, int64_t* req_c, int64_t* cnt_c, void* stream) {
  int rc = check_state(s, "uvmi_sched_compact");
  if (rc) return rc;
  UVMI_REQUIRE(n_bucket > 0 && act_slot && tok_c && pos_c && starts_c && req_c && cnt_c, UVMI_EINVAL, "uvmi_sched_compact: bad arguments");
  hipLaunchKernelGGL(sched_compact_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, *s, n_bucket, act_slot, tok_c, pos_c, starts_c, req_c, cnt_c);
  UVMI_CHECK_LAUNCH("uvmi_sched_compact");
  return UVMI_OK;
}

extern "C" int uvmi_sched_commit(const uvmi_sched_state* s, int n_bucket, const int64_t* act_slot, const int64_t* new_tok,
                                 const float* new_lp, float retire_p, uint64_t seed, void* stream) {
  int rc = check_state(s, "uvmi_sched_commit");
  if (rc) return rc;
  UVMI_REQUIRE(n_bucket > 0 && act_slot && new_tok, UVMI_EINVAL, "uvmi_sched_commit: bad arguments");
  const DenseArrays D{const_cast<int64_t*>(act_slot), nullptr, nullptr, nullptr, nullptr, nullptr};
  hipLaunchKernelGGL(sched_commit_kernel<false>, dim3((n_bucket + 255) / 256), dim3(256), 0, (hipStream_t)stream, *s, n_bucket, D, new_tok,
                     new_lp, retire_p, seed);
  UVMI_CHECK_LAUNCH("uvmi_sched_commit");
  return UVMI_OK;
}

extern "C" int uvmi_sched_commit_dense(const uvmi_sched_state* s, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c,
                                       int64_t* starts_c, int64_t* req_c, int64_t* cnt_c, const int64_t* new_tok, const float* new_lp,
                                       float retire_p, uint64_t seed, void* stream) {
  int rc = check_state(s, "uvmi_sched_commit_dense");
  if (rc) return rc;
  UVMI_REQUIRE(n_bucket > 0 && act_slot && tok_c && pos_c && starts_c && req_c && cnt_c && new_tok, UVMI_EINVAL,
               "uvmi_sched_commit_dense: bad arguments");
  const DenseArrays D{act_slot, tok_c, pos_c, starts_c, req_c, cnt_c};
  hipLaunchKernelGGL(sched_commit_kernel<true>, dim3((n_bucket + 255) / 256), dim3(256), 0, (hipStream_t)stream, *s, n_bucket, D, new_tok,
                     new_lp, retire_p, seed);
  UVMI_CHECK_LAUNCH("uvmi_sched_commit_dense");
  return UVMI_OK;
}

extern "C" int uvmi_sched_admit(const uvmi_sched_state* s, int n, const int64_t* slots, const int64_t* req_ids, const int64_t* limits,
                                const int64_t* first_tok, const float* first_lp, void* stream) {
  int rc = check_state(s, "uvmi_sched_admit");
  if (rc) return rc;
  UVMI_REQUIRE(n >= 0 && (n == 0 || (slots && req_ids && limits && first_tok)), UVMI_EINVAL, "uvmi_sched_admit: bad arguments");
  if (n == 0) return UVMI_OK;
  hipLaunchKernelGGL(sched_admit_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, *s, n, slots, req_ids, limits, first_tok, first_lp);
  UVMI_CHECK_LAUNCH("uvmi_sched_admit");
  return UVMI_OK;
}

extern "C" int uvmi_sched_expand(const uvmi_sched_state* s, int n_adm, int n_tokens, const int64_t* cu_seqlens, const int64_t* adm_slot,
                                 const int64_t* adm_start, int64_t* pos_t, int64_t* row_t, int64_t* last_t, int64_t* last_idx, void* stream) {
  int rc = check_state(s, "uvmi_sched_expand");
  if (rc) return rc;
  UVMI_REQUIRE(n_adm > 0 && n_tokens >= 0 && cu_seqlens && adm_slot && adm_start && pos_t && row_t && last_t && last_idx, UVMI_EINVAL,
               "uvmi_sched_expand: bad arguments");
  const int n = n_tokens > n_adm ? n_tokens : n_adm;
  hipLaunchKernelGGL(sched_expand_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, *s, n_adm, n_tokens, cu_seqlens, adm_slot,
                     adm_start, pos_t, row_t, last_t, last_idx);
  UVMI_CHECK_LAUNCH("uvmi_sched_expand");
  return UVMI_OK;
}

extern "C" int uvmi_sched_plan_admit(const uvmi_sched_state* s, int admit_cap, int n_tokens, int left_pad, int64_t* adm_cu, int64_t* adm_slot,
                                     int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req, int64_t* tok_packed, void* stream) {
  int rc = check_state(s, "uvmi_sched_plan_admit");
  if (rc) return rc;
  UVMI_REQUIRE(s->q_buf && s->q_ctl && s->q_cap > 0 && s->q_stride > 3, UVMI_EINVAL, "uvmi_sched_plan_admit: the state has no admission queue");
  UVMI_REQUIRE(admit_cap > 0 && admit_cap <= 256 && n_tokens > 0 && adm_cu && adm_slot && adm_start && adm_limit && adm_req && tok_packed,
               UVMI_EINVAL, "uvmi_sched_plan_admit: bad arguments (admit_cap 1..256)");
  hipLaunchKernelGGL(sched_plan_admit_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, *s, admit_cap, n_tokens, left_pad ? 1 : 0, adm_cu,
                     adm_slot, adm_start, adm_limit, adm_req, tok_packed);
  UVMI_CHECK_LAUNCH("uvmi_sched_plan_admit");
  return UVMI_OK;
}

extern "C" int uvmi_sched_step_plan(const uvmi_sched_state* s, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c, int64_t* starts_c,
                                    int64_t* req_c, int64_t* cnt_c, int admit_cap, int n_tokens, int left_pad, int64_t* adm_cu, int64_t* adm_slot,
                                    int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req, int64_t* tok_packed, int64_t* pos_t,
                                    int64_t* row_t, int64_t* last_t, int64_t* last_idx, int64_t* last_c, void* stream) {
  int rc = check_state(s, "uvmi_sched_step_plan");
  if (rc) return rc;
  UVMI_REQUIRE(s->q_buf && s->q_ctl && s->q_cap > 0 && s->q_stride > 3, UVMI_EINVAL, "uvmi_sched_step_plan: the state has no admission queue");
  UVMI_REQUIRE(n_bucket > 0 && act_slot && tok_c && pos_c && starts_c && req_c && cnt_c && admit_cap > 0 && admit_cap <= 256 && n_tokens > 0 &&
                   adm_cu && adm_slot && adm_start && adm_limit && adm_req && tok_packed && pos_t && row_t && last_t && last_idx,
               UVMI_EINVAL, "uvmi_sched_step_plan: bad arguments (admit_cap 1..256)");
  hipLaunchKernelGGL(sched_step_plan_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, *s, n_bucket, act_slot, tok_c, pos_c, starts_c, req_c,
                     cnt_c, admit_cap, n_tokens, left_pad ? 1 : 0, adm_cu, adm_slot, adm_start, adm_limit, adm_req, tok_packed, pos_t, row_t,
                     last_t, last_idx, last_c);
  UVMI_CHECK_LAUNCH("uvmi_sched_step_plan");
  return UVMI_OK;
}

extern "C" int uvmi_sched_harvest(const uvmi_sched_state* s, int64_t seen, int max_rows, int64_t* hdr, int32_t* tok_dst, float* lp_dst,
                                  void* stream) {
  int rc = check_state(s, "uvmi_sched_harvest");
  if (rc) return rc;
  UVMI_REQUIRE(seen >= 0 && max_rows > 0 && max_rows <= 65535 && hdr && tok_dst, UVMI_EINVAL, "uvmi_sched_harvest: bad arguments");
  hipLaunchKernelGGL(sched_harvest_kernel, dim3(max_rows), dim3(256), 0, (hipStream_t)stream, *s, seen, max_rows, hdr, tok_dst, lp_dst);
  UVMI_CHECK_LAUNCH("uvmi_sched_harvest");
  return UVMI_OK;
}
