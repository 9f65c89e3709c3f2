// One row of the slot table's commit step, shared by the commit kernel and by the sampler kernels that commit the token
// they drew in the same launch (reference: buf.scatter_ / cnt.add_ and the harvest test of scripts/rl_stream.py:120-143,
// ultraviolet/model.py:1321-1350).
#pragma once
#include "common.h"

namespace uvmi {

constexpr uint32_t DOMAIN_RETIRE = 0x52455452u;

__device__ inline void philox_round10(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1, n3 = (uint32_t)p0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

// The dense arrays of a step (uvmi_sched_compact's outputs); all null: the step's arrays are not carried on.
struct DenseArrays {
  int64_t* act_slot; int64_t* tok; int64_t* pos; int64_t* starts; int64_t* req; int64_t* cnt;
};

// Dense row i drew token tok with log-prob lp: scatter both into the slot's output row, advance count and position, retire
// on EOS / length limit / the seeded Bernoulli(retire_p) draw keyed by (seed, request, token index), park a retired row
// at position 0 and append its completion record.  DENSE: the row's dense entries become the next step's - the new
// token, position + 1, index + 1 - or padding (slot -1, zeros) when the row retires.
template <bool DENSE>
__device__ __forceinline__ void commit_row(const uvmi_sched_state S, const DenseArrays D, int i, int64_t tok, float lp, float retire_p,
                                           uint64_t seed) {
  const int64_t slot = D.act_slot[i];
  if (slot < 0) return;
  const int64_t c = S.slot_cnt[slot];
  const int64_t col = c < S.max_new ? c : S.max_new - 1;   // clamp like the reference's buffers (rl_stream.py:122)
  S.out_tok[slot * S.max_new + col] = (int32_t)tok;
  if (S.out_lp) S.out_lp[slot * S.max_new + col] = lp;
  S.slot_cnt[slot] = c + 1;
  S.slot_tok[slot] = tok;
  S.pos[slot] += 1;
  bool fin = (c + 1 >= S.slot_limit[slot]) || (S.eos_id >= 0 && tok == S.eos_id);
  const int64_t req = S.slot_req[slot];
  if (!fin && retire_p > 0.f) {
    uint32_t ctr[4] = {(uint32_t)c, (uint32_t)req, (uint32_t)((uint64_t)req >> 32), DOMAIN_RETIRE};
    philox_round10(ctr, (uint32_t)seed, (uint32_t)(seed >> 32));
    fin = (float)(ctr[0] >> 8) * 5.9604644775390625e-08f < retire_p;
  }
  if (fin) {
    const int k = atomicAdd(&S.counters[1], 1) % S.done_cap;  // ring: the host must poll before done_cap more rows finish
    S.done_req[k] = req;
    S.done_slot[k] = slot;
    S.done_cnt[k] = c + 1;
    S.slot_req[slot] = -1;
    if (S.slot_hold) S.slot_hold[slot] = 1;   // its output row is not harvested yet: not reusable by a device-side admission
    S.pos[slot] = 0;      // parked: never overruns the cache (model.py:1345-1350)
    S.starts[slot] = 0;
  }
  if (DENSE) {
    D.act_slot[i] = fin ? -1 : slot;
    D.tok[i] = fin ? 0 : tok;
    D.pos[i] = fin ? 0 : D.pos[i] + 1;
    D.cnt[i] = fin ? 0 : c + 1;
    if (fin) { D.starts[i] = 0; D.req[i] = 0; }
  }
}

}  // namespace uvmi
