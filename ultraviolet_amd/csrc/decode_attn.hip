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
//         v_perm_b32 only (u = x ^ 0x80 = x + 128): K' = fp16 0x64uu = 1024 + u keeps a +1152 bias that is
//         cancelled by the accumulator's initial value -1152 * sum(q); V'' = fp16 0x00uu = u * 2^-24 (a subnormal,
//         which the f16 MFMA honours) keeps a +128 bias that is removed at the end with 128 * sum(P'), P' being the
//         fp16-rounded probabilities (accumulated with v_dot2_f32_f16);
//       - all addressing in the loop is scalar (wave-uniform tile base) plus lane-invariant 32-bit offsets;
//       - online softmax per (stream, head) column, rescaling only when some column's maximum grew; the two
//         streams are merged once at the end.
//   * attn_generic: any head_dim <= 256, G <= 16, int8 / fp16 / bf16 caches, arbitrary alignment: plain fp32 VALU.
//
// Split partials (acc, m, l) go to a caller-provided workspace; attn_combine merges them.
#include "common.h"

#include <cstdlib>
#include <type_traits>
#include <mutex>

namespace uvmi {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));

constexpr float LOG2E = 1.4426950408889634f;

struct AttnParams {
  const void* q; const void* kc; const void* vc; const void* ks; const void* vs;
  const void* pos; const void* starts; const void* rows;
  void* out; float* ws_o; float* ws_m; float* ws_l;
  int64_t sqb, sqh, skb, skh, sks, svb, svh, svs, ssb, ssh, stb, sth, sob, soh;
  int B, H, KH, G, S, hd, window, ring, splits, idx64, chunk_keys, gran;  // gran: chunk granularity (keys)
  int64_t n_items;
  float scale_log2;
  // optional fused epilogue (Attention.post of the reference, model.py:321-333)
  const float* post_vhat; const float* post_gate; const float* post_xsa; int post_dt;
  // optional fused QKV post-processing of the row's own token (model.py:302-319, fast_decode.py:291-294, 315-317)
  const void* f_qkv; const void* f_tok; const void* f_ve; const float* f_rope_tab;
  int64_t f_sqkv, f_vocab;
  int f_ext, f_rope, f_rope_n, f_has_ve, f_has_gate;
  float f_eps, f_xsa_eps;
};

// Key range of a row and how it is cut.  The span starts at lo rounded down to 32 so tiles stay aligned to the
// slot grid; each work item gets `chunk` keys (a multiple of 32, at least chunk_keys, and large enough that at most
// `splits` items cover the span).  A row with a single chunk is written directly, without partials.
struct RowPlan { int lo, p, a0, chunk, nsplit, cb, pc; };  // p: last streamed position; pc: the row's own position
// Low 32 bits of element i of an I32 / I64 index array (positions, starts and row ids fit 31 bits; -1 keeps its sign),
// for a wave-uniform i: one 4-byte scalar load whatever the width (constant address space: the arrays are inputs of the
// launch), so the three loads of a plan have no branches between them and go out together.
__device__ __forceinline__ int load_idx32(const void* p, int is64, int64_t i) {
  typedef const int32_t __attribute__((address_space(4))) * cptr32;
  return *(cptr32)((uintptr_t)p + (uintptr_t)(i * (is64 ? 8 : 4)));
}
// own_key_apart: the key at the row's own position is not in the cache yet (the kernel forms it itself), so the streamed
// range ends one position earlier.
__device__ __forceinline__ RowPlan plan_row(const AttnParams& P, int b, bool own_key_apart = false, bool uncut = false) {
  RowPlan r;
  const int pv = load_idx32(P.pos, P.idx64, b);
  const int st = load_idx32(P.starts, P.idx64, b);
  const int rv = load_idx32(P.rows ? P.rows : P.pos, P.idx64, b);
  r.cb = P.rows ? rv : b;               // cache row of this query row
  const int pc = r.cb < 0 ? -1 : pv;    // padding row of a compacted batch: no keys, output zeros
  if (r.cb < 0) r.cb = 0;               // (dead rows have no keys; keep addresses valid)
  int lo = st > 0 ? st : 0;
  if (P.window > 0 && pc - P.window + 1 > lo) lo = pc - P.window + 1;
  const int p = own_key_apart ? pc - 1 : pc;
  r.pc = pc;
  r.lo = lo;
  r.p = p;
  r.a0 = lo & ~31;
  int span = p + 1 - r.a0;
  if (span < 0) span = 0;
  if (uncut) {  // (known at compile time where it is set: the whole row is one chunk)
    r.chunk = 0x3fffffff;
    r.nsplit = 1;
    return r;
  }
  // (integer divisions by run-time values cost a few dozen instructions each, here on the way to the row's first tile
  // request: the granule is a power of two, and an uncut row - every decode step of the engine - divides by nothing)
  const int gr = P.gran;  // 32, 64 or 128
  const int per = P.splits == 1 ? span : (int)(((uint32_t)span + (uint32_t)P.splits - 1u) / (uint32_t)P.splits);
  int chunk = (per + gr - 1) & ~(gr - 1);
  if (chunk < P.chunk_keys) chunk = P.chunk_keys;
  if (chunk < gr) chunk = gr;
  r.chunk = chunk;
  r.nsplit = span > chunk ? (int)(((uint32_t)span + (uint32_t)chunk - 1u) / (uint32_t)chunk) : 1;
  return r;
}

// Cache slot of position t >= 0: t itself, or t mod S on a ring (a mask when S is a power of two, as every window is).
__device__ __forceinline__ int ring_slot(const AttnParams& P, int t) {
  if (!P.ring) return t;
  return (P.S & (P.S - 1)) == 0 ? (t & (P.S - 1)) : (int)((uint32_t)t % (uint32_t)P.S);
}

// ---------------------------------------------------------------------------------------------------- MFMA kernel
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

__device__ __forceinline__ h8 as_h8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uint32_t r[4] = {a, b, c, d};
  h8 v;
  __builtin_memcpy(&v, r, 16);
  return v;
}

// (the lane exchanges and the 64-lane butterflies - pairing lane ^ 32, 16, 8, 4, 2, 1, the order every kernel of this library
// reduces in - live in common.h)
__device__ __forceinline__ float bfly_sum(float v) { return wave_sum(v); }
__device__ __forceinline__ float bfly_max(float v) { return wave_max(v); }

struct Tile {             // one 32-key super-tile as loaded from HBM (26 dwords per lane)
  uint4 kA, kB;           // key m of stream A / B, bytes 16g..16g+15
  uint32_t vA[4], vB[4];  // keys 4g+j of stream A / B, bytes 4m..4m+3
  uint2 ksc, vsc;         // fp16 scales of keys 4g..4g+3 of this lane's stream
};

struct Tile16 {           // the same super-tile of a 16-bit cache (32 dwords per lane)
  u4 kA[2], kB[2];        // key m of stream A / B, dims 16g..16g+7 and 16g+8..16g+15
  u2 vA[4], vB[4];        // keys 4g+j of stream A / B, dims 4m..4m+3
};

// 16x16x32 MFMA on operand words of the 16-bit type DT (the int8 path always multiplies in fp16)
template <int DT>
__device__ __forceinline__ f4 mfma_kv(const h8& a, const h8& b, f4 acc) {
  if constexpr (DT == UVMI_BF16) {
    typedef __bf16 b8 __attribute__((ext_vector_type(8)));
    b8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
  }
}

struct AttnState {
  f4 O[4];                // O''^T tiles: 2^-24 * sum (v + 128) P'
  float mrun, lrun, psum; // reference point of the exponentials (score units before scale), sum p, sum of the fp16-rounded P'
  float mthr;             // mrun + the slack a score may exceed it by before the reference point moves
};

// WPR waves of a workgroup share one work item (row, kv head, split): wave w takes super-tiles w, w + WPR, ... of the
// chunk, so the workgroup streams 32 * WPR consecutive keys (2 KB * WPR of K and of V) per step, which keeps many more
// DRAM pages open-and-hit than one wave per row does; the WPR online-softmax states are merged through LDS at the end.

// FUSE: the row's own token is taken from the projection output (q, k, v, gate logits) instead of from q and the cache:
// the kernel normalises and rotates q and k, adds the value embedding to v, quantises k and v into the cache, and attends
// the streamed cache range lo..pos-1 plus the own key from registers; the XSA / gate epilogue uses the own v directly.
// The arguments ahead of the parameter block are what a wave needs before it can request anything - the index arrays of
// the row's plan, the q (or projection) pointer and the item arithmetic: as leading scalar arguments they are preloaded
// into SGPRs with the wave, so the plan's loads go out without first waiting for a load of the kernel arguments.
// KV16: the cache holds K / V unquantized in the q dtype (no scales): the same work split, plan, online softmax, merge and
// epilogue around tiles that go into the MFMAs as they are loaded - no conversion, no bias terms, probabilities rounded to
// the cache type (a tile is 32 dwords per lane, still 4 waves per SIMD).  With FUSE the own token's k and v are appended
// as they are (on the cache type's grid already) and the own key's score is q . k in fp32.
// FAST: the shape of the engine's decode step as compile-time constants - one kv head, 8 query heads, uncut rows, 64-bit
// indices - so that the item arithmetic, the head masks, the split bookkeeping and the partial-result path fold away
// (the fixed part of a wave's life is as long as its streaming loop on rows of a few hundred keys).
// PROBE (uvmi_decode_attn_probe; measurement only, the output is meaningless): 1 - the kernel's memory stream without its
// arithmetic: every tile is loaded exactly as in the real kernel and folded into the state with a few xors; 2 - its
// arithmetic without the stream: tiles are made up in registers, nothing is loaded from the cache.
template <int QDT, int ODT, int WPR, bool FUSE, bool KV16 = false, bool FAST = false, int PROBE = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4)))
void attn_mfma_i8_hd64(const void* a_pos, const void* a_starts, const void* a_rows, const void* a_q, int64_t a_items, int a_idx64,
                       int a_splits, int a_kh, AttnParams P) {
  P.pos = a_pos; P.starts = a_starts; P.rows = a_rows; P.n_items = a_items; P.idx64 = a_idx64; P.splits = a_splits; P.KH = a_kh;
  if constexpr (FAST) { P.idx64 = 1; P.splits = 1; P.KH = 1; P.G = 8; P.H = 8; P.hd = 64; P.chunk_keys = 0; }
  if (FUSE) P.f_qkv = a_q; else P.q = a_q;
  constexpr int IPB = 4 / WPR;  // items per block
  __shared__ __attribute__((aligned(16))) float sh_o[4][16][68];
  __shared__ __attribute__((aligned(16))) float sh_ml[4][16][4];
  __shared__ float sh_post[4][80];  // epilogue operands of the item whose first wave this is: v_hat[64], gate[8], xsa[8]
  __shared__ float sh_cur[FUSE ? 4 : 1][72];  // own key of that item: score per head [8], dequantised v [64]
  __shared__ __attribute__((aligned(16))) uint16_t sh_q[FUSE ? 4 : 1][8][64];  // the item's q as fp16 operand words
  __shared__ float sh_qs[FUSE ? 4 : 1][8];                                      // and their sum per head
  __shared__ float sh_kq[FUSE ? 4 : 1][64];   // the own key's int8 codes (as floats), for its score against every head
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wsub = wave % WPR;
  int64_t item = (int64_t)blockIdx.x * IPB + wave / WPR;  // wave-uniform
  const bool live_item = item < P.n_items;
  if (!live_item) {
    if (WPR == 1) return;
    item = P.n_items - 1;  // keep the wave for the barrier below; it does no work
  }
  // (items fit 31 bits, host-checked; one split and one kv head - the engine's shape - need no division)
  const uint32_t it32 = (uint32_t)item;
  const int sid = P.splits == 1 ? 0 : (int)(it32 % (uint32_t)P.splits);
  const uint32_t bk = P.splits == 1 ? it32 : it32 / (uint32_t)P.splits;
  const int b = __builtin_amdgcn_readfirstlane((int)(P.KH == 1 ? bk : bk / (uint32_t)P.KH));
  const int h = __builtin_amdgcn_readfirstlane((int)(P.KH == 1 ? 0u : bk % (uint32_t)P.KH));
  const int m = lane & 15, g = lane >> 4;  // A/B operand (row, group) == accumulator (column, group)
  const int strm = m >> 3, head = m & 7;
  const int G = P.G;
  const float c = P.scale_log2;
  // The q loads depend only on the row index: they go out first, then the row's plan (three scalar loads issued
  // together), then the first K/V tile; q is converted while that tile is in flight.
  // (no branch around the loads: lanes of absent heads read head G-1 and are masked to zero when the operands are
  // formed, which keeps the control flow, and with it every row-derived scalar, wave-uniform)
  const uint32_t qmask = head < G ? 0xffffffffu : 0u;
  // (FUSE: q is normalised and rotated once per item, by its first wave, eight dims per lane - lane (hh, cc) = dims
  // 8cc..8cc+7 of head hh, the standalone post-processing kernel's layout and reduction order - and reaches the operand
  // layout of every wave of the item through LDS)
  const int hh = lane >> 3, cc = lane & 7;
  const uint16_t* qp = FUSE ? (const uint16_t*)P.f_qkv + (int64_t)b * P.f_sqkv + (h * G + (hh < G ? hh : G - 1)) * 64 + 8 * cc
                            : (const uint16_t*)P.q + (int64_t)b * P.sqb + (int64_t)(h * G + (head < G ? head : G - 1)) * P.sqh + 16 * g;
  const uint4 qw0 = *(const uint4*)qp, qw1 = FUSE ? qw0 : *(const uint4*)(qp + 8);
  // FUSE: the row's gate logits and its raw k / v go out with q.  k and v are read one dim per lane: the item's first wave
  // takes k, its second wave v (a lone wave takes both)
  constexpr int VW = WPR > 1 ? 1 : 0;  // the wave of an item that forms the own value (the first wave forms the own key)
  uint16_t glog = 0, vlog = 0, raw_a = 0, raw_v = 0;
  int64_t own_tok = 0;
  if constexpr (FUSE) {
    const uint16_t* rowp = (const uint16_t*)P.f_qkv + (int64_t)b * P.f_sqkv;
    glog = rowp[P.f_ext + (P.f_has_gate ? h * G + (head < G ? head : G - 1) : 0)];
    vlog = rowp[P.f_ext + P.H + h];
    raw_a = rowp[(P.H + (WPR > 1 && wsub == VW ? P.KH : 0) + h) * 64 + lane];
    if (WPR == 1) raw_v = rowp[(P.H + P.KH + h) * 64 + lane];
    own_tok = P.f_has_ve ? (int64_t)load_idx32(P.f_tok, P.idx64, b) : 0;
    own_tok = own_tok < 0 ? 0 : (own_tok >= P.f_vocab ? P.f_vocab - 1 : own_tok);
  }
  // Operands of the fused epilogue are requested now, with q, and parked in LDS once q has arrived, so that the
  // epilogue at the end of the workgroup's life does not start with a round trip to memory.  Unconditional loads (from
  // q when there is no epilogue) keep the control flow uniform.
  const bool has_post = FUSE || P.post_vhat != nullptr;
  const int hsafe = h * G + (head < G ? head : G - 1);
  const float* anyf = FUSE ? (const float*)P.f_qkv : (const float*)P.q;  // a readable address for the unused cases
  const float* pv_src = !FUSE && has_post ? P.post_vhat + ((int64_t)b * P.KH + h) * 64 + lane : anyf + lane;
  const float* pg_src = !FUSE && has_post && P.post_gate ? P.post_gate + (int64_t)b * P.H + hsafe : anyf;
  const float* px_src = has_post && P.post_xsa ? P.post_xsa + hsafe : anyf;
  const float pv_val = *pv_src, pg_val = *pg_src, px_val = *px_src;
  const RowPlan rp = plan_row(P, b, FUSE, FAST);
  // FUSE: the row of the rotation table (cos / sin of the row's position per frequency, already rounded to the activation
  // type): prep_q reads its 32 values as scalars, the lane that owns dim d of the own key reads its own pair
  const int rope_row = rp.pc < 0 ? 0 : (rp.pc < P.f_rope_n ? rp.pc : P.f_rope_n - 1);
  const bool live = live_item && sid < rp.nsplit;
  if (WPR == 1 && !live) return;
  const int s0 = rp.a0 + sid * rp.chunk;
  const int s1 = live ? min(s0 + rp.chunk, rp.p + 1) : s0;
  const int lo_eff = max(rp.lo, s0);

  // ---- Q^T operands: lane (n, g) holds q[head][16g + 8s + j] as fp16 (bf16 inputs are converted; exact for
  // 2^-14 <= |q| <= 65504).  The K operand carries a +1152 bias, cancelled by starting the accumulator at
  // -1152 * sum_d q[head][d].
  const uint32_t mA = strm == 0 ? qmask : 0u, mB = strm == 0 ? 0u : qmask;
  h8 QA0, QA1, QB0, QB1;
  float cinit;
  auto rq = [&](float v) -> float { return QDT == UVMI_BF16 ? bf16_to_float(float_to_bf16(v)) : (float)(half_t)v; };
  const int iw = wave - wsub;  // LDS slot of the item: its first wave
  uint32_t qr[8];
  float qsum;
  auto set_q = [&]() {
    QA0 = as_h8(qr[0] & mA, qr[1] & mA, qr[2] & mA, qr[3] & mA); QA1 = as_h8(qr[4] & mA, qr[5] & mA, qr[6] & mA, qr[7] & mA);
    QB0 = as_h8(qr[0] & mB, qr[1] & mB, qr[2] & mB, qr[3] & mB); QB1 = as_h8(qr[4] & mB, qr[5] & mB, qr[6] & mB, qr[7] & mB);
    cinit = !KV16 && qmask ? -1152.0f * qsum : 0.f;
  };
  // unfused: q arrives normalised and rotated, 16 dims per lane in the operand layout
  auto prep_q = [&]() {
    const uint32_t w[8] = {qw0.x, qw0.y, qw0.z, qw0.w, qw1.x, qw1.y, qw1.z, qw1.w};
    qsum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      float f0, f1;
      if (QDT == UVMI_BF16) { f0 = __uint_as_float(w[i] << 16); f1 = __uint_as_float(w[i] & 0xffff0000u); }
      else { f0 = half_bits_to_float(w[i] & 0xffff); f1 = half_bits_to_float(w[i] >> 16); }
      if constexpr (KV16) {
        qr[i] = w[i];   // the product runs in the q dtype itself
      } else {
        const uint16_t l16 = float_to_half_bits(f0), h16 = float_to_half_bits(f1);
        qr[i] = (uint32_t)l16 | ((uint32_t)h16 << 16);
        qsum += half_bits_to_float(l16) + half_bits_to_float(h16);
      }
    }
    qsum = xsum32(xsum16(qsum));  // all 64 dims of this head
    set_q();
  };
  // FUSE, first wave of the item: QK-norm and partial rotation of the 8 heads (uvmi_qkv_post's arithmetic: RMS over the
  // head's 8 lanes by xor 1, 2, 4; rotation partner dims 8cc.. <-> 8(cc ^ 2)..), then the fp16 operand words and their
  // sum per head go to LDS
  auto prep_q_item = [&](const float4& c0, const float4& c1, const float4& s0, const float4& s1) {
    const uint32_t w[4] = {qw0.x, qw0.y, qw0.z, qw0.w};
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (QDT == UVMI_BF16) { x[2 * i] = __uint_as_float(w[i] << 16); x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
      else { x[2 * i] = half_bits_to_float(w[i] & 0xffff); x[2 * i + 1] = half_bits_to_float(w[i] >> 16); }
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) ss += x[j] * x[j];
    ss += dpp_mov<0xb1>(ss); ss += dpp_mov<0x4e>(ss); ss += lane_xor4(ss);
    const float rs = rsqrtf(ss * (1.0f / 64.0f) + P.f_eps);
#pragma unroll
    for (int j = 0; j < 8; j++) x[j] = rq(x[j] * rs);
    if (P.f_rope) {  // 16 pairs: dims 0..15 (cc 0, 1) with 16..31 (cc 2, 3); frequency index of dim 8cc + j is 8(cc & 1) + j
      const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w}, sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
      const bool first = cc < 2, rot = cc < 4;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const float v = rope_rot(x[j], dpp_mov<0x4e>(x[j]), cs[j], sn[j], first, rq);
        x[j] = rot ? v : x[j];
      }
    }
    uint32_t o[4];
    float qs = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if constexpr (KV16 && QDT == UVMI_BF16) {   // the product runs in the q dtype itself (x is on its grid already)
        o[i] = (uint32_t)float_to_bf16(x[2 * i]) | ((uint32_t)float_to_bf16(x[2 * i + 1]) << 16);
      } else {
        const uint16_t l16 = float_to_half_bits(x[2 * i]), h16 = float_to_half_bits(x[2 * i + 1]);
        o[i] = (uint32_t)l16 | ((uint32_t)h16 << 16);
        qs += half_bits_to_float(l16) + half_bits_to_float(h16);
      }
    }
    qs += dpp_mov<0xb1>(qs); qs += dpp_mov<0x4e>(qs); qs += lane_xor4(qs);
    *(uint4*)&sh_q[iw][hh][8 * cc] = uint4{o[0], o[1], o[2], o[3]};
    if (cc == 0) sh_qs[iw][hh] = qs;
  };
  // FUSE, every wave of the item, after the barrier that follows prep_q_item: its operand words from LDS
  auto fetch_q = [&]() {
    const uint4 o0 = *(const uint4*)&sh_q[iw][head][16 * g], o1 = *(const uint4*)&sh_q[iw][head][16 * g + 8];
    qr[0] = o0.x; qr[1] = o0.y; qr[2] = o0.z; qr[3] = o0.w; qr[4] = o1.x; qr[5] = o1.y; qr[6] = o1.z; qr[7] = o1.w;
    qsum = sh_qs[iw][head];
    set_q();
  };

  // FUSE, the row's own token.  The item's first wave forms k (norm, rotation), its second wave v (value embedding); both
  // work one dim per lane with the arithmetic, roundings and reduction order of the standalone post-processing kernel
  // (uvmi_qkv_post), append the int8 row at the row's position, and park in LDS what the end of the kernel needs: the own
  // key's score per head and dequantised value (merged into the softmax after the streamed range), v_hat and the gates.
  auto cvt_in = [&](uint16_t w) -> float { return QDT == UVMI_BF16 ? bf16_to_float(w) : half_bits_to_float(w); };
  // int8 code (as a float) of this lane's element of a 64-dim row, and the row's fp16 scale: fp16 scale, IEEE division,
  // round half to even, clamp - the standalone quantizer's arithmetic
  auto quant1 = [&](float x, uint16_t& sb) -> float {
    const float am = bfly_max(fabsf(x));
    sb = float_to_half_bits(__fdiv_rn(am, 127.0f));
    const float sf = fmaxf(half_bits_to_float(sb), 1e-30f);
    return fminf(fmaxf(__builtin_rintf(__fdiv_rn(x, sf)), -127.0f), 127.0f);
  };
  auto own_k = [&](uint16_t raw, float kcs, float ksn) {
    float k = cvt_in(raw);
    const float rs = rsqrtf(bfly_sum(k * k) * (1.0f / 64.0f) + P.f_eps);
    k = rq(k * rs);
    if (P.f_rope) {
      const float kr = rope_rot(k, lane_xor16(k), kcs, ksn, lane < 16, rq);
      k = lane < 32 ? kr : k;
    }
    uint16_t sbk = 0;
    float kq;   // what the cache holds for this lane's dim: the int8 code, or (16-bit cache) k itself
    const int slot = ring_slot(P, rp.pc);
    if constexpr (KV16) {
      kq = k;   // on the cache type's grid already
      if (slot < P.S)
        ((uint16_t*)P.kc)[(int64_t)rp.cb * P.skb + (int64_t)h * P.skh + (int64_t)slot * P.sks + lane] =
            QDT == UVMI_BF16 ? float_to_bf16(k) : float_to_half_bits(k);
    } else {
      kq = quant1(k, sbk);
      if (slot < P.S) {
        ((int8_t*)P.kc)[(int64_t)rp.cb * P.skb + (int64_t)h * P.skh + (int64_t)slot * P.sks + lane] = (int8_t)(int)kq;
        if (lane == 0) ((uint16_t*)P.ks)[(int64_t)rp.cb * P.ssb + (int64_t)h * P.ssh + slot] = sbk;
      }
    }
    // score of the own key against every head: q as the operand holds it (lane (head, g): dims 16g..16g+15) . the int8
    // codes * k scale (16-bit cache: . k), in the units of the streamed scores
    sh_kq[iw][lane] = kq;
    __builtin_amdgcn_wave_barrier();
    auto qlo = [&](uint32_t w) -> float { return KV16 && QDT == UVMI_BF16 ? __uint_as_float(w << 16) : half_bits_to_float(w & 0xffff); };
    auto qhi = [&](uint32_t w) -> float { return KV16 && QDT == UVMI_BF16 ? __uint_as_float(w & 0xffff0000u) : half_bits_to_float(w >> 16); };
    float dq = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float4 c4 = *(const float4*)&sh_kq[iw][16 * g + 4 * i];
      dq += qlo(qr[2 * i]) * c4.x + qhi(qr[2 * i]) * c4.y;
      dq += qlo(qr[2 * i + 1]) * c4.z + qhi(qr[2 * i + 1]) * c4.w;
    }
    dq = xsum32(xsum16(dq));
    if constexpr (!KV16) dq *= half_bits_to_float(sbk);
    if (lane < 8) {
      sh_cur[iw][lane] = dq;
      sh_post[iw][64 + lane] = P.f_has_gate ? rq(2.0f * rq(1.0f / (1.0f + __expf(-cvt_in(glog))))) : 1.0f;
    }
    if (lane >= 8 && lane < 16) sh_post[iw][64 + lane] = px_val;
  };
  auto own_v = [&](uint16_t raw, uint16_t raw_ve) {
    float v = cvt_in(raw);
    if (P.f_has_ve) {
      const float gv = rq(2.0f * rq(1.0f / (1.0f + __expf(-cvt_in(vlog)))));
      v = ve_add(v, gv, cvt_in(raw_ve), rq);
    }
    const float nv = fmaxf(sqrtf(bfly_sum(v * v)), P.f_xsa_eps);
    const int slot = ring_slot(P, rp.pc);
    if constexpr (KV16) {
      if (slot < P.S)
        ((uint16_t*)P.vc)[(int64_t)rp.cb * P.svb + (int64_t)h * P.svh + (int64_t)slot * P.svs + lane] =
            QDT == UVMI_BF16 ? float_to_bf16(v) : float_to_half_bits(v);
      sh_cur[iw][8 + lane] = v;
    } else {
      uint16_t sbv;
      const float vq = quant1(v, sbv);
      if (slot < P.S) {
        ((int8_t*)P.vc)[(int64_t)rp.cb * P.svb + (int64_t)h * P.svh + (int64_t)slot * P.svs + lane] = (int8_t)(int)vq;
        if (lane == 0) ((uint16_t*)P.vs)[(int64_t)rp.cb * P.stb + (int64_t)h * P.sth + slot] = sbv;
      }
      sh_cur[iw][8 + lane] = half_bits_to_float(sbv) * vq;
    }
    sh_post[iw][lane] = v / nv;
  };

  AttnState st;
#pragma unroll
  for (int t = 0; t < 4; t++) st.O[t] = f4{0.f, 0.f, 0.f, 0.f};
  st.mrun = -INFINITY;
  st.mthr = -INFINITY;
  st.lrun = 0.f;
  st.psum = 0.f;
  constexpr float LAZY = 4.0f;           // log2 of the largest probability relative to the reference point
  const float lazy_pre = LAZY / c;       // in score units before the softmax scale (c > 0, host-checked)

  // ---- addressing: wave-uniform row base + wave-uniform tile offset (scalar) + lane-invariant 32-bit offsets
  const int64_t cb = rp.cb;
  constexpr int ES = KV16 ? 2 : 1;   // bytes per cache element
  const int8_t* kbase = (const int8_t*)P.kc + (cb * P.skb + (int64_t)h * P.skh) * ES;
  const int8_t* vbase = (const int8_t*)P.vc + (cb * P.svb + (int64_t)h * P.svh) * ES;
  const uint16_t* ksb = (const uint16_t*)P.ks + cb * P.ssb + (int64_t)h * P.ssh;
  const uint16_t* vsb = (const uint16_t*)P.vs + cb * P.stb + (int64_t)h * P.sth;
  const int S = P.S;
  const uint32_t sks = (uint32_t)P.sks * ES, svs = (uint32_t)P.svs * ES;   // row strides in bytes
  const uint32_t usks = __builtin_amdgcn_readfirstlane(sks), usvs = __builtin_amdgcn_readfirstlane(svs);
  const uint32_t koA = m * sks + 16 * ES * g, koB = koA + 16 * sks;  // K: key m of stream A / B, dims 16g..
  const uint32_t voA = 4 * g * svs + 4 * ES * m;     // V: key 4g (+j via the scalar offset), dims 4m..
  const uint32_t so = 16 * strm + 4 * g;  // scale offset (elements) inside the super-tile

  // Buffer descriptors (wave-uniform, one per row stream): a load is descriptor base + lane-invariant VGPR offset +
  // scalar tile offset, so the loop spends no VALU work on addresses.  num_records covers exactly the row's bytes.
  const __amdgpu_buffer_rsrc_t rK = __builtin_amdgcn_make_buffer_rsrc((void*)kbase, 0, (S - 1) * (int)sks + 64 * ES, 0x00020000);
  const __amdgpu_buffer_rsrc_t rV = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, (S - 1) * (int)svs + 64 * ES, 0x00020000);
  const __amdgpu_buffer_rsrc_t rKS = __builtin_amdgcn_make_buffer_rsrc((void*)ksb, 0, S * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t rVS = __builtin_amdgcn_make_buffer_rsrc((void*)vsb, 0, S * 2, 0x00020000);
  const uint32_t so2 = so * 2;

  // slot0: cache slot of absolute position tb (a multiple of 32).  Ring caches have S % 32 == 0 (host-checked), so a
  // super-tile never wraps.  load_tile needs slot0 + 32 <= S; a linear cache that ends inside its last super-tile
  // takes load_tail (per-lane clamped rows) for that one tile, outside the pipelined loop.
  using TileX = std::conditional_t<KV16, Tile16, Tile>;
  auto load_tile = [&](int slot_in, TileX& T) {
    const int slot0 = __builtin_amdgcn_readfirstlane(slot_in);  // wave-uniform by construction
    const uint32_t ok = (uint32_t)slot0 * usks, ov = (uint32_t)slot0 * usvs, os = (uint32_t)slot0 * 2;
    if constexpr (KV16) {
      T.kA[0] = __builtin_amdgcn_raw_buffer_load_b128(rK, koA, ok, 0);
      T.kA[1] = __builtin_amdgcn_raw_buffer_load_b128(rK, koA + 16, ok, 0);
      T.kB[0] = __builtin_amdgcn_raw_buffer_load_b128(rK, koB, ok, 0);
      T.kB[1] = __builtin_amdgcn_raw_buffer_load_b128(rK, koB + 16, ok, 0);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        T.vA[j] = __builtin_amdgcn_raw_buffer_load_b64(rV, voA, ov + j * usvs, 0);
        T.vB[j] = __builtin_amdgcn_raw_buffer_load_b64(rV, voA, ov + (16 + j) * usvs, 0);
      }
    } else if constexpr (PROBE == 2) {
      const uint32_t w = (uint32_t)slot0 * 0x9E3779B1u + (uint32_t)lane * 0x85EBCA6Bu;
      T.kA = uint4{w, w ^ 0x01234567u, w * 3u, w * 5u};
      T.kB = uint4{~w, w ^ 0x76543210u, w * 7u, w * 9u};
#pragma unroll
      for (int j = 0; j < 4; j++) { T.vA[j] = w + 0x01010101u * j; T.vB[j] = ~w + 0x01010101u * j; }
      T.ksc = uint2{0x21202120u, 0x21202120u};   // fp16 0.0100 four times
      T.vsc = uint2{0x21202120u, 0x21202120u};
    } else {
    u4 ka = __builtin_amdgcn_raw_buffer_load_b128(rK, koA, ok, 0);
    u4 kb = __builtin_amdgcn_raw_buffer_load_b128(rK, koB, ok, 0);
    T.kA = uint4{ka.x, ka.y, ka.z, ka.w};
    T.kB = uint4{kb.x, kb.y, kb.z, kb.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      T.vA[j] = __builtin_amdgcn_raw_buffer_load_b32(rV, voA, ov + j * usvs, 0);
      T.vB[j] = __builtin_amdgcn_raw_buffer_load_b32(rV, voA, ov + (16 + j) * usvs, 0);
    }
    u2 a = __builtin_amdgcn_raw_buffer_load_b64(rKS, so2, os, 0);
    u2 c2 = __builtin_amdgcn_raw_buffer_load_b64(rVS, so2, os, 0);
    T.ksc = uint2{a.x, a.y};
    T.vsc = uint2{c2.x, c2.y};
    }
  };
  auto load_tail = [&](int slot0, TileX& T) {
    const int smax = S - 1;
    if constexpr (KV16) {
      const int8_t* ka = kbase + (int64_t)min(slot0 + m, smax) * sks + 32 * g;
      const int8_t* kb = kbase + (int64_t)min(slot0 + 16 + m, smax) * sks + 32 * g;
      T.kA[0] = *(const u4*)ka; T.kA[1] = *(const u4*)(ka + 16);
      T.kB[0] = *(const u4*)kb; T.kB[1] = *(const u4*)(kb + 16);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        T.vA[j] = *(const u2*)(vbase + (int64_t)min(slot0 + 4 * g + j, smax) * svs + 8 * m);
        T.vB[j] = *(const u2*)(vbase + (int64_t)min(slot0 + 16 + 4 * g + j, smax) * svs + 8 * m);
      }
    } else {
    T.kA = *(const uint4*)(kbase + (int64_t)min(slot0 + m, smax) * P.sks + 16 * g);
    T.kB = *(const uint4*)(kbase + (int64_t)min(slot0 + 16 + m, smax) * P.sks + 16 * g);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      T.vA[j] = *(const uint32_t*)(vbase + (int64_t)min(slot0 + 4 * g + j, smax) * P.svs + 4 * m);
      T.vB[j] = *(const uint32_t*)(vbase + (int64_t)min(slot0 + 16 + 4 * g + j, smax) * P.svs + 4 * m);
    }
    const int ss = min(slot0 + (int)so, S - 4);  // S % 4 == 0: a clamped group is entirely past the cache end
    T.ksc = *(const uint2*)(ksb + ss);
    T.vsc = *(const uint2*)(vsb + ss);
    }
  };

  auto step = [&](const TileX& T, int tb, bool edge) {
    if constexpr (PROBE == 1 && !KV16) {
      const uint32_t x = T.kA.x ^ T.kA.y ^ T.kA.z ^ T.kA.w ^ T.kB.x ^ T.kB.y ^ T.kB.z ^ T.kB.w ^ T.vA[0] ^ T.vA[1] ^ T.vA[2] ^ T.vA[3] ^
                         T.vB[0] ^ T.vB[1] ^ T.vB[2] ^ T.vB[3] ^ T.ksc.x ^ T.ksc.y ^ T.vsc.x ^ T.vsc.y;
      st.psum = __uint_as_float(__float_as_uint(st.psum) ^ x);
      return;
    }
    // ---- S^T = K' . Q^T - 1152 sum(q), K' = 1024 + (k ^ 0x80) as fp16 0x64uu (16-bit cache: K as loaded, no bias)
    f4 acc = f4{cinit, cinit, cinit, cinit};
    if constexpr (KV16) {
      // An accumulator column sums one stream's products and the other stream's products with zeros, so on an edge tile
      // the rows of keys outside the range are cleared first: a slot never written may hold a NaN or Inf pattern, and
      // 0 x NaN would reach the score of the other stream's valid key.
      u4 a0 = T.kA[0], a1 = T.kA[1], b0 = T.kB[0], b1 = T.kB[1];
      if (edge) {
        const u4 z = u4{0u, 0u, 0u, 0u};
        if (tb + m < lo_eff || tb + m >= s1) { a0 = z; a1 = z; }
        if (tb + 16 + m < lo_eff || tb + 16 + m >= s1) { b0 = z; b1 = z; }
      }
      acc = mfma_kv<QDT>(as_h8(a0.x, a0.y, a0.z, a0.w), QA0, acc);
      acc = mfma_kv<QDT>(as_h8(a1.x, a1.y, a1.z, a1.w), QA1, acc);
      acc = mfma_kv<QDT>(as_h8(b0.x, b0.y, b0.z, b0.w), QB0, acc);
      acc = mfma_kv<QDT>(as_h8(b1.x, b1.y, b1.z, b1.w), QB1, acc);
    } else {
      const uint32_t a0 = T.kA.x ^ 0x80808080u, a1 = T.kA.y ^ 0x80808080u, a2 = T.kA.z ^ 0x80808080u, a3 = T.kA.w ^ 0x80808080u;
      const uint32_t b0 = T.kB.x ^ 0x80808080u, b1 = T.kB.y ^ 0x80808080u, b2 = T.kB.z ^ 0x80808080u, b3 = T.kB.w ^ 0x80808080u;
      constexpr uint32_t C64 = 0x64646464u, LO = 0x04010400u, HI = 0x04030402u;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(perm(C64, a0, LO), perm(C64, a0, HI), perm(C64, a1, LO), perm(C64, a1, HI)), QA0, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(perm(C64, a2, LO), perm(C64, a2, HI), perm(C64, a3, LO), perm(C64, a3, HI)), QA1, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(perm(C64, b0, LO), perm(C64, b0, HI), perm(C64, b1, LO), perm(C64, b1, HI)), QB0, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_h8(perm(C64, b2, LO), perm(C64, b2, HI), perm(C64, b3, LO), perm(C64, b3, HI)), QB1, acc, 0, 0, 0);
    }
    // ---- t_i = (q.k_int) * kscale_i for the lane's keys 4g+i of its stream (softmax scale applied inside exp2)
    float t[4], vsf[4];
    if constexpr (KV16) {
#pragma unroll
      for (int i = 0; i < 4; i++) { t[i] = acc[i]; vsf[i] = 1.f; }
    } else {
      h2 ks01, ks23, vs01, vs23;
      __builtin_memcpy(&ks01, &T.ksc.x, 4); __builtin_memcpy(&ks23, &T.ksc.y, 4);
      __builtin_memcpy(&vs01, &T.vsc.x, 4); __builtin_memcpy(&vs23, &T.vsc.y, 4);
      t[0] = acc[0] * (float)ks01[0]; t[1] = acc[1] * (float)ks01[1]; t[2] = acc[2] * (float)ks23[0]; t[3] = acc[3] * (float)ks23[1];
      vsf[0] = (float)vs01[0]; vsf[1] = (float)vs01[1]; vsf[2] = (float)vs23[0]; vsf[3] = (float)vs23[1];
    }
    if (edge) {  // keys outside [lo_eff, s1): no score, and their (possibly stale, non-finite) V scale must not meet p = 0
      const int t0 = tb + 16 * strm + 4 * g;
#pragma unroll
      for (int i = 0; i < 4; i++)
        if (t0 + i < lo_eff || t0 + i >= s1) { t[i] = -INFINITY; vsf[i] = 0.f; }
    }
    // The reference point of a column's exponentials only has to stay within 2^LAZY of its true maximum (probabilities up
    // to 2^LAZY are as exact in fp16 / fp32 as those below 1), so the common tile compares each lane's own scores with
    // the column's threshold and skips both the cross-lane maximum and the rescale.
    float mx = fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3]));
    if (__builtin_amdgcn_ballot_w64(mx > st.mthr) != 0) {  // some column outgrew its reference point: move it (alpha = 1 elsewhere)
      mx = xmax32(xmax16(mx));
      const float mnew = fmaxf(st.mrun, mx);
      const float alpha = mnew == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f((st.mrun - mnew) * c);
#pragma unroll
      for (int tt = 0; tt < 4; tt++) st.O[tt] *= alpha;
      st.lrun *= alpha;
      st.psum *= alpha;
      st.mrun = mnew;
      st.mthr = mnew + lazy_pre;   // (-inf stays -inf)
    }
    const float mc = st.mrun == -INFINITY ? 0.f : st.mrun * c;
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; i++) p[i] = __builtin_amdgcn_exp2f(fmaf(t[i], c, -mc));
    st.lrun += (p[0] + p[1]) + (p[2] + p[3]);
    // ---- P' = fp16(p * vscale) (16-bit cache: p rounded to the cache type), placed in this stream's half of the
    // contraction slots
    uint32_t u01, u23;
    [[maybe_unused]] uint32_t l01 = 0, l23 = 0;
    if constexpr (KV16 && QDT == UVMI_BF16) {
      // a bf16 cache: p goes in as two bf16 terms, p = hi + lo (16 significant bits, where a single bf16 has 8), and P V is
      // two MFMAs per operand - the matrix pipe has the room, and the result stays within the fp16 path's error
      typedef __bf16 b2 __attribute__((ext_vector_type(2)));
      const b2 p01 = b2{(__bf16)p[0], (__bf16)p[1]}, p23 = b2{(__bf16)p[2], (__bf16)p[3]};
      const b2 q01 = b2{(__bf16)(p[0] - (float)p01[0]), (__bf16)(p[1] - (float)p01[1])};
      const b2 q23 = b2{(__bf16)(p[2] - (float)p23[0]), (__bf16)(p[3] - (float)p23[1])};
      __builtin_memcpy(&u01, &p01, 4);
      __builtin_memcpy(&u23, &p23, 4);
      __builtin_memcpy(&l01, &q01, 4);
      __builtin_memcpy(&l23, &q23, 4);
    } else {
      const h2 p01 = h2{(_Float16)(p[0] * vsf[0]), (_Float16)(p[1] * vsf[1])};
      const h2 p23 = h2{(_Float16)(p[2] * vsf[2]), (_Float16)(p[3] * vsf[3])};
      if constexpr (!KV16) {
        const h2 ones = h2{(_Float16)1.0f, (_Float16)1.0f};
        st.psum = __builtin_amdgcn_fdot2(p23, ones, __builtin_amdgcn_fdot2(p01, ones, st.psum, false), false);
      }
      __builtin_memcpy(&u01, &p01, 4);
      __builtin_memcpy(&u23, &p23, 4);
    }
    const h8 PB = as_h8(u01 & mA, u23 & mA, u01 & mB, u23 & mB);
    // ---- O''^T += V'' . P'^T with V'' = (v ^ 0x80) * 2^-24 (fp16 subnormal 0x00uu; the MFMA takes subnormals);
    // tile tt, operand row m is head dim 4m + tt
    if constexpr (KV16) {
      // V as loaded: dword pairs (dims 4m..4m+3) of 8 keys; operand tt takes half tt of each pair.  On an edge tile the
      // values of keys outside the range are cleared: a slot never written may hold a NaN pattern, and 0 x NaN is NaN.
      u2 va_[4], vb_[4];
#pragma unroll
      for (int j = 0; j < 4; j++) { va_[j] = T.vA[j]; vb_[j] = T.vB[j]; }
      if (edge) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const int ka = tb + 4 * g + j, kb = ka + 16;
          if (ka < lo_eff || ka >= s1) va_[j] = u2{0u, 0u};
          if (kb < lo_eff || kb >= s1) vb_[j] = u2{0u, 0u};
        }
      }
      constexpr uint32_t LO = 0x05040100u, HI = 0x07060302u;
#pragma unroll
      for (int tt = 0; tt < 4; tt++) {
        const uint32_t sel = (tt & 1) ? HI : LO;
        const int e = tt >> 1;
        const h8 va = as_h8(perm(va_[1][e], va_[0][e], sel), perm(va_[3][e], va_[2][e], sel), perm(vb_[1][e], vb_[0][e], sel), perm(vb_[3][e], vb_[2][e], sel));
        st.O[tt] = mfma_kv<QDT>(va, PB, st.O[tt]);
        if constexpr (QDT == UVMI_BF16) st.O[tt] = mfma_kv<QDT>(va, as_h8(l01 & mA, l23 & mA, l01 & mB, l23 & mB), st.O[tt]);
      }
    } else {
      uint32_t xa[4], xb[4];
#pragma unroll
      for (int j = 0; j < 4; j++) { xa[j] = T.vA[j] ^ 0x80808080u; xb[j] = T.vB[j] ^ 0x80808080u; }
#pragma unroll
      for (int tt = 0; tt < 4; tt++) {
        const uint32_t sel = 0x0c000c00u | ((4u + tt) << 16) | (uint32_t)tt;  // [0, S0.byte tt, 0, S1.byte tt]
        const h8 va = as_h8(perm(xa[1], xa[0], sel), perm(xa[3], xa[2], sel), perm(xb[1], xb[0], sel), perm(xb[3], xb[2], sel));
        st.O[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, PB, st.O[tt], 0, 0, 0);
      }
    }
  };

  {
    // Pipelined part: tiles that lie entirely inside the cache.  The next tile's loads are issued unconditionally
    // before the current tile is consumed (past the end the current tile is re-read, a cache hit), so that no
    // branch separates load issue from use and the wait counters stay exact.
    constexpr int STEP = 32 * WPR;
    const int s1f = P.ring ? s1 : min(s1, S & ~31);
    int tb = s0 + 32 * wsub;
    const bool has = tb < s1f;
    int slot = has ? ring_slot(P, tb) : 0;
    auto next_slot = [&](int sl, int t) {
      if (t + STEP >= s1f) return sl;
      sl += STEP;
      if (P.ring) while (sl >= S) sl -= S;
      return sl;
    };
    // What the fused prologue still needs from memory - the rotation table row (q: this lane's 8 frequencies; own key: the
    // lane's pair) and the value-embedding element - is requested before the tiles: loads complete in order, so anything
    // requested after a tile could only be used once that tile has arrived.
    // (unconditional loads from a select of addresses - the row itself when a feature is off - keep this stretch free of
    // branches, which would make the compiler wait for the loads before it requests the tiles)
    float kcs = 1.f, ksn = 0.f;
    uint16_t raw_ve = 0;
    float4 rc0 = float4{1.f, 1.f, 1.f, 1.f}, rc1 = rc0, rs0 = float4{0.f, 0.f, 0.f, 0.f}, rs1 = rs0;
    if constexpr (FUSE) {
      const uint16_t* own_row = (const uint16_t*)P.f_qkv + (int64_t)b * P.f_sqkv;
      const float* tr = P.f_rope ? P.f_rope_tab + (int64_t)rope_row * 32 : (const float*)own_row;
      const float* tq = tr + 8 * (cc & 1);
      rc0 = *(const float4*)tq; rc1 = *(const float4*)(tq + 4); rs0 = *(const float4*)(tq + 16); rs1 = *(const float4*)(tq + 20);
      kcs = tr[lane & 15]; ksn = tr[16 + (lane & 15)];
      raw_ve = (P.f_has_ve ? (const uint16_t*)P.f_ve + (own_tok * P.KH + h) * 64 : own_row)[lane];
    }
    // The first tile is requested unconditionally (a wave without a pipelined tile reads slot 0 and drops it; the
    // descriptor bounds the access), so that the q conversion - and, on the fused path, the forming of the row's own key -
    // follows it on every path and waits for q only.  (Requesting two tiles here was measured on the fused path, with no
    // spills: 20.5 us against 19.2 us per launch on ~2000 rows x ~215 keys - all waves' first two tiles then leave in
    // one burst of more than half the launch's bytes.)
    TileX TA, TB;
    load_tile(slot, TA);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!FUSE) {
      prep_q();
      if (wsub == 0) {
        sh_post[wave][lane] = pv_val;
        if (lane < 16) sh_post[wave][64 + lane] = lane < 8 ? pg_val : px_val;  // lanes 8..15 carry head lane - 8 too
      }
    } else {
      const bool own = live && rp.pc >= 0;
      if (wsub == 0) prep_q_item(rc0, rc1, rs0, rs1);
      else if (WPR > 1 && wsub == VW && own) own_v(raw_a, raw_ve);  // needs no q: done while the first wave prepares it
      if (WPR > 1) __syncthreads(); else __builtin_amdgcn_wave_barrier();
      fetch_q();
      if (own && wsub == 0) {
        own_k(raw_a, kcs, ksn);
        if (WPR == 1) own_v(raw_v, raw_ve);
      }
    }
    if (has) {
      while (true) {
        slot = next_slot(slot, tb);
        load_tile(slot, TB);
        step(TA, tb, tb < lo_eff || tb + 32 > s1);
        tb += STEP;
        if (tb >= s1f) break;
        slot = next_slot(slot, tb);
        load_tile(slot, TA);
        step(TB, tb, tb < lo_eff || tb + 32 > s1);
        tb += STEP;
        if (tb >= s1f) break;
      }
    }
    if (tb < s1) {  // linear cache ending inside this super-tile (at most one wave of the item gets here)
      TileX TT;
      load_tail(tb, TT);
      step(TT, tb, true);
    }
  }
  // ---- reduce l and sum P' over the 4 lane groups of a column
  const float lsum = xsum32(xsum16(st.lrun)), ps = xsum32(xsum16(st.psum));
  const float m2 = st.mrun == -INFINITY ? -INFINITY : st.mrun * c;  // exp2 domain
  if (!FAST && rp.nsplit > 1) {
    // ---- a chunk of a cut row: stream B is merged into stream A (lanes n and n ^ 8: a rotation by 8 inside a row of 16
    // lanes, a DPP move), the WPR waves of the item through LDS, and the item's first wave writes the partial state
    const float m_o = dpp_mov<0x128>(m2), l_o = dpp_mov<0x128>(lsum), ps_o = dpp_mov<0x128>(ps);
    const float mm = fmaxf(m2, m_o);
    const float ms = mm == -INFINITY ? 0.f : mm;
    const float w_s = __builtin_amdgcn_exp2f(m2 - ms), w_o = __builtin_amdgcn_exp2f(m_o - ms);
    const float lm = lsum * w_s + l_o * w_o;
    const float pm = KV16 ? 0.f : 128.0f * (ps * w_s + ps_o * w_o);
    const float w_s24 = KV16 ? w_s : w_s * 16777216.0f, w_o24 = KV16 ? w_o : w_o * 16777216.0f;
    float o[16];  // head dims 16g .. 16g+15: O[t][i] is dim 16g + 4i + t
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float mine = st.O[t][i];
        const float oth = dpp_mov<0x128>(mine);
        o[4 * i + t] = (mine * w_s24 + oth * w_o24) - pm;
      }
    float mfin = mm, lfin = lm;
    if (WPR > 1) {
      if (strm == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) *(float4*)&sh_o[wave][head][16 * g + 4 * i] = float4{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
        if (g == 0) { sh_ml[wave][head][0] = mm; sh_ml[wave][head][1] = lm; }
      }
      __syncthreads();
      if (wsub != 0 || !live) return;
      if (strm == 0) {
        float mw[WPR];
        float mall = -INFINITY;
#pragma unroll
        for (int w = 0; w < WPR; w++) { mw[w] = sh_ml[wave + w][head][0]; mall = fmaxf(mall, mw[w]); }
        const float msf = mall == -INFINITY ? 0.f : mall;
        lfin = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) o[i] = 0.f;
#pragma unroll
        for (int w = 0; w < WPR; w++) {
          const float ww = __builtin_amdgcn_exp2f(mw[w] - msf);
          lfin += ww * sh_ml[wave + w][head][1];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const float4 x = *(const float4*)&sh_o[wave + w][head][16 * g + 4 * i];
            o[4 * i] += ww * x.x; o[4 * i + 1] += ww * x.y; o[4 * i + 2] += ww * x.z; o[4 * i + 3] += ww * x.w;
          }
        }
        mfin = mall;
      }
    }
    if (strm == 0 && head < G) {
      const int64_t r = item * G + head;
      float* op = P.ws_o + r * 64 + 16 * g;
#pragma unroll
      for (int i = 0; i < 4; i++) *(float4*)(op + 4 * i) = float4{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
      if (g == 0) {
        P.ws_m[r] = mfin;
        P.ws_l[r] = lfin;
      }
    }
    return;
  }
  // ---- an uncut row: every wave parks its raw state in LDS - both streams' accumulators and (m, l, sum P') per column -
  // and all lanes of the item's waves then share the merge and the epilogue: a thread owns NV consecutive dims of one head
  // (with one wave per row 8, with four waves 2), merges the 2 WPR partial states of its dims, applies the epilogue and
  // stores.  (Rows of sh_o are padded to 68 floats so that the 16 columns of a 16-byte access fall into different banks.)
#pragma unroll
  for (int i = 0; i < 4; i++) *(float4*)&sh_o[wave][m][16 * g + 4 * i] = float4{st.O[0][i], st.O[1][i], st.O[2][i], st.O[3][i]};
  if (g == 0) *(float4*)&sh_ml[wave][m][0] = float4{m2, lsum, ps, 0.f};
  if (WPR > 1) __syncthreads(); else __builtin_amdgcn_wave_barrier();
  if (!live) return;
  constexpr int NV = 8 / WPR, TPH = 64 / NV;       // values per thread, threads per head
  const int ti = wsub * 64 + lane;
  const int eh = ti / TPH, d0 = (ti % TPH) * NV;   // head and first dim of this thread
  float mw[2 * WPR], mall = -INFINITY;
#pragma unroll
  for (int w = 0; w < WPR; w++)
#pragma unroll
    for (int sx = 0; sx < 2; sx++) { mw[2 * w + sx] = sh_ml[iw + w][8 * sx + eh][0]; mall = fmaxf(mall, mw[2 * w + sx]); }
  const float msf = mall == -INFINITY ? 0.f : mall;
  float o[NV], lfin = 0.f, psf = 0.f;
#pragma unroll
  for (int j = 0; j < NV; j++) o[j] = 0.f;
#pragma unroll
  for (int w = 0; w < WPR; w++)
#pragma unroll
    for (int sx = 0; sx < 2; sx++) {
      const float ww = __builtin_amdgcn_exp2f(mw[2 * w + sx] - msf);
      lfin += ww * sh_ml[iw + w][8 * sx + eh][1];
      psf += ww * sh_ml[iw + w][8 * sx + eh][2];
      const float* src = &sh_o[iw + w][8 * sx + eh][d0];
      if constexpr (NV == 8) {
        const float4 x = *(const float4*)src, y = *(const float4*)(src + 4);
        o[0] += ww * x.x; o[1] += ww * x.y; o[2] += ww * x.z; o[3] += ww * x.w; o[4] += ww * y.x; o[5] += ww * y.y; o[6] += ww * y.z; o[7] += ww * y.w;
      } else if constexpr (NV == 4) {
        const float4 x = *(const float4*)src;
        o[0] += ww * x.x; o[1] += ww * x.y; o[2] += ww * x.z; o[3] += ww * x.w;
      } else {
        const float2 x = *(const float2*)src;
        o[0] += ww * x.x; o[1] += ww * x.y;
      }
    }
  if constexpr (!KV16) {  // undo the 2^-24 of the subnormal V operand and its +128 bias
    const float pm = 128.0f * psf;
#pragma unroll
    for (int j = 0; j < NV; j++) o[j] = o[j] * 16777216.0f - pm;
  }
  float mfin = mall;
  if constexpr (FUSE) {
    if (rp.pc >= 0) {  // the own key joins the softmax after the streamed range
      const float s2 = sh_cur[iw][eh] * c;
      const float mnew = fmaxf(mfin, s2);
      const float wa = mfin == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mfin - mnew), wb = __builtin_amdgcn_exp2f(s2 - mnew);
      lfin = lfin * wa + wb;
#pragma unroll
      for (int j = 0; j < NV; j++) o[j] = o[j] * wa + wb * sh_cur[iw][8 + d0 + j];
      mfin = mnew;
    }
  }
  const float inv = lfin > 0.f ? 1.0f / lfin : 0.f;
  if (has_post) {
    // z (rounded to the q dtype, as the attention output tensor would be) -> XSA -> gate, written in the output type.
    // The TPH threads of a head are consecutive lanes of one wave, all active, so the cross-lane sums are well defined.
    auto rnd = [&](float x, int dt) -> float {
      return dt == UVMI_F32 ? x : (dt == UVMI_BF16 ? bf16_to_float(float_to_bf16(x)) : (float)(half_t)x);
    };
    const bool dead = FUSE && rp.pc < 0;  // padding row of the fused path: nothing was parked for it, the output is zero
    float vv[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) vv[j] = dead ? 0.f : sh_post[iw][d0 + j];
    const float gate = dead ? 0.f : (FUSE || P.post_gate ? sh_post[iw][64 + eh] : 1.0f);
    float proj = 0.f;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      o[j] = rnd(o[j] * inv, QDT);
      proj += o[j] * vv[j];
    }
    if (P.post_xsa) {
      proj += lane_xor1(proj); proj += lane_xor2(proj); proj += lane_xor4(proj);
      if constexpr (TPH >= 16) proj += lane_xor8(proj);
      if constexpr (TPH >= 32) proj += lane_xor16(proj);
      const float ah = dead ? 0.f : sh_post[iw][72 + eh] * proj;
#pragma unroll
      for (int j = 0; j < NV; j++) o[j] = rnd(o[j] - ah * vv[j], QDT);
    }
#pragma unroll
    for (int j = 0; j < NV; j++) o[j] *= gate;
  } else {
#pragma unroll
    for (int j = 0; j < NV; j++) o[j] *= inv;
  }
  if (eh < G) {
    const int64_t off = (int64_t)b * P.sob + (int64_t)(h * G + eh) * P.soh + d0;
    if constexpr (ODT == UVMI_F32) {
      float* op = (float*)P.out + off;
      if constexpr (NV == 2) *(float2*)op = float2{o[0], o[1]};
      else
#pragma unroll
        for (int j = 0; j < NV; j += 4) *(float4*)(op + j) = float4{o[j], o[j + 1], o[j + 2], o[j + 3]};
    } else {
      uint32_t w[NV / 2];
#pragma unroll
      for (int j = 0; j < NV / 2; j++) {
        const uint32_t l16 = ODT == UVMI_BF16 ? float_to_bf16(o[2 * j]) : float_to_half_bits(o[2 * j]);
        const uint32_t h16 = ODT == UVMI_BF16 ? float_to_bf16(o[2 * j + 1]) : float_to_half_bits(o[2 * j + 1]);
        w[j] = l16 | (h16 << 16);
      }
      uint16_t* op = (uint16_t*)P.out + off;
      if constexpr (NV == 8) *(uint4*)op = uint4{w[0], w[1], w[2], w[3]};
      else if constexpr (NV == 4) *(uint2*)op = uint2{w[0], w[1]};
      else *(uint32_t*)op = w[0];
    }
  }
}

// ------------------------------------------------------------------------------------------------- generic kernel
// One wave per (row, kv head, split).  Lanes own keys for Q.K (64 keys per tile), then own head dims for P.V.
template <int KVDT>
__device__ __forceinline__ float kv_ld(const void* p, int64_t i) {
  if (KVDT == UVMI_I8) return (float)((const int8_t*)p)[i];
  if (KVDT == UVMI_F16) return half_bits_to_float(((const uint16_t*)p)[i]);
  if (KVDT == UVMI_F32) return ((const float*)p)[i];
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
  const RowPlan rp = plan_row(P, b);
  if (sid >= rp.nsplit) return;
  struct { int s0, s1; } c;
  c.s0 = rp.a0 + sid * rp.chunk;
  c.s1 = min(c.s0 + rp.chunk, rp.p + 1);
  const int lo_eff = max(rp.lo, c.s0);
  const bool direct = rp.nsplit == 1;
  constexpr int MAXG = 16, MAXD = 4;  // hd <= 256
  float mrun[MAXG], lrun[MAXG], acc[MAXG][MAXD];
#pragma unroll
  for (int gi = 0; gi < MAXG; gi++) {
    mrun[gi] = -INFINITY;
    lrun[gi] = 0.f;
#pragma unroll
    for (int j = 0; j < MAXD; j++) acc[gi][j] = 0.f;
  }
  int64_t cb = P.rows ? load_index(P.rows, P.idx64, b) : (int64_t)b;
  if (cb < 0) cb = 0;
  const int64_t kb0 = cb * P.skb + (int64_t)h * P.skh, vb0 = cb * P.svb + (int64_t)h * P.svh;
  const int64_t ks0 = cb * P.ssb + (int64_t)h * P.ssh, vs0 = cb * P.stb + (int64_t)h * P.sth;
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
          if (direct) {
            const float v = lrun[gi] > 0.f ? acc[gi][dj] / lrun[gi] : 0.f;
            elem<ODT>::st(P.out, (int64_t)b * P.sob + (int64_t)(h * G + gi) * P.soh + d, v);
          } else {
            P.ws_o[(item * G + gi) * hd + d] = acc[gi][dj];
          }
        }
      }
      if (!direct && lane == 0) {
        P.ws_m[item * G + gi] = mrun[gi];
        P.ws_l[item * G + gi] = lrun[gi];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------- combine
// One wave per (row, kv head), all G query heads: out = sum_s w_s o_s / sum_s w_s l_s, w_s = 2^(m_s - max m); empty
// splits (m = -inf) get weight 0 (decode_attn.py:96-115 of the reference).  Rows that fit one chunk were written by
// the attention kernel and are skipped.
template <int ODT>
__global__ __launch_bounds__(256) void attn_combine(AttnParams P) {
  const int lane = threadIdx.x & 63;
  const int64_t bk = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (bk >= (int64_t)P.B * P.KH) return;
  const int b = (int)(bk / P.KH), h = (int)(bk % P.KH);
  const RowPlan rp = plan_row(P, b);
  if (rp.nsplit <= 1) return;
  for (int gi = 0; gi < P.G; gi++) {
    float mx = -INFINITY;
    for (int s = 0; s < rp.nsplit; s++) mx = fmaxf(mx, P.ws_m[(bk * P.splits + s) * P.G + gi]);
    const float ms = mx == -INFINITY ? 0.f : mx;
    float den = 0.f;
    float num[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < rp.nsplit; s++) {
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
}

// ---------------------------------------------------------------------------------------------------- host side
static int check_common(const uvmi_attn_args* a) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_decode_attn: null args");
  UVMI_REQUIRE(a->q && a->k_cache && a->v_cache && a->pos && a->starts && a->out, UVMI_EINVAL, "uvmi_decode_attn: null pointer");
  UVMI_REQUIRE(a->B >= 0 && a->H > 0 && a->KH > 0 && a->S > 0 && a->hd > 0, UVMI_EINVAL, "uvmi_decode_attn: bad sizes");
  UVMI_REQUIRE(a->H % a->KH == 0, UVMI_EINVAL, "uvmi_decode_attn: H=%d is not a multiple of KH=%d", a->H, a->KH);
  UVMI_REQUIRE(a->q_dtype == UVMI_F16 || a->q_dtype == UVMI_BF16 || a->q_dtype == UVMI_F32, UVMI_EUNSUPPORTED,
               "uvmi_decode_attn: q must be F16, BF16 or F32");
  UVMI_REQUIRE(a->out_dtype == UVMI_F16 || a->out_dtype == UVMI_BF16 || a->out_dtype == UVMI_F32, UVMI_EUNSUPPORTED,
               "uvmi_decode_attn: out must be F16, BF16 or F32");
  UVMI_REQUIRE(a->kv_dtype == UVMI_I8 || a->kv_dtype == UVMI_F16 || a->kv_dtype == UVMI_BF16 || a->kv_dtype == UVMI_F32, UVMI_EUNSUPPORTED,
               "uvmi_decode_attn: cache must be I8, F16, BF16 or F32");
  UVMI_REQUIRE(a->kv_dtype != UVMI_I8 || (a->k_scale && a->v_scale), UVMI_EINVAL, "uvmi_decode_attn: int8 cache needs k_scale and v_scale");
  UVMI_REQUIRE(a->idx_dtype == UVMI_I64 || a->idx_dtype == UVMI_I32, UVMI_EINVAL, "uvmi_decode_attn: pos/starts must be I32 or I64");
  UVMI_REQUIRE(a->num_splits >= 1 && a->num_splits <= 1024, UVMI_EINVAL, "uvmi_decode_attn: num_splits=%d out of range", a->num_splits);
  UVMI_REQUIRE(a->window >= 0 && a->chunk_keys >= 0, UVMI_EINVAL, "uvmi_decode_attn: negative window or chunk_keys");
  UVMI_REQUIRE(a->hd <= 256 && a->H / a->KH <= 16, UVMI_EUNSUPPORTED, "uvmi_decode_attn: head_dim %d / group %d beyond 256 / 16", a->hd,
               a->H / a->KH);
  return UVMI_OK;
}

static bool mfma_ok(const uvmi_attn_args* a) {
  const int G = a->H / a->KH;
  if (a->hd != 64 || a->kv_dtype != UVMI_I8 || G > 8) return false;
  if (a->q_dtype == UVMI_F32) return false;  // fp32 queries keep every product and probability in fp32: the generic kernel
  if (!(a->scale > 0.f)) return false;  // the running maximum is tracked before the (positive) softmax scale
  if (a->ring && (a->S % 32 != 0)) return false;
  if (a->sks > (1 << 20) || a->svs > (1 << 20) || a->sks < 0 || a->svs < 0) return false;  // 32-bit tile offsets
  if (a->S % 4 != 0 || a->S < 32) return false;  // 8-byte scale loads; a whole 32-key tile at slot 0 must exist
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

// The MFMA kernel on a cache that holds K / V unquantized in the q dtype.
static bool mfma16_ok(const uvmi_attn_args* a) {
  const int G = a->H / a->KH;
  if (a->hd != 64 || G > 8 || a->kv_dtype != a->q_dtype || (a->q_dtype != UVMI_F16 && a->q_dtype != UVMI_BF16)) return false;
  if (!(a->scale > 0.f)) return false;
  if (a->ring && (a->S % 32 != 0)) return false;
  if (a->S < 32) return false;  // a whole 32-key tile at slot 0 must exist
  if (a->sks > (1 << 19) || a->svs > (1 << 19) || a->sks < 0 || a->svs < 0) return false;  // 32-bit tile offsets in bytes
  auto al = [](const void* p, int n) { return ((uintptr_t)p % n) == 0; };
  if (!al(a->q, 16) || a->sqb % 8 || a->sqh % 8) return false;
  if (!al(a->k_cache, 16) || a->skb % 8 || a->skh % 8 || a->sks % 8) return false;   // 16-byte K loads
  if (!al(a->v_cache, 8) || a->svb % 4 || a->svh % 4 || a->svs % 4) return false;    // 8-byte V loads
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
  // One workgroup (4 waves streaming interleaved tiles) per (row, kv head, split).  A row is only cut when there are
  // fewer rows than compute units, and never into chunks shorter than 256 keys: the combine pass costs more than the
  // imbalance it removes once every CU has a workgroup.
  const int64_t want = (n_cus + n_bk - 1) / n_bk;
  int64_t cap = ctx / 256;
  if (cap < 1) cap = 1;
  int64_t s = want < cap ? want : cap;
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

extern "C" int uvmi_decode_attn_path(const uvmi_attn_args* a) {
  int rc = check_common(a);
  if (rc) return rc;
  return mfma_ok(a) || mfma16_ok(a) ? 1 : 0;
}

// The launch sequence of uvmi_decode_attn with the split partials in `ws` (ws_bytes of device memory; unused when
// num_splits == 1): the caller's workspace, or this library's own scratch array.
static int decode_attn_launch(const uvmi_attn_args* a, void* ws, size_t ws_bytes, const char* who, void* stream, int probe = 0) {
  int rc = check_common(a);
  if (rc) return rc;
  if (a->B == 0) return UVMI_OK;
  hipStream_t st = (hipStream_t)stream;
  AttnParams P;
  P.q = a->q; P.kc = a->k_cache; P.vc = a->v_cache; P.ks = a->k_scale; P.vs = a->v_scale;
  P.pos = a->pos; P.starts = a->starts; P.rows = a->rows; P.out = a->out;
  P.sqb = a->sqb; P.sqh = a->sqh; P.skb = a->skb; P.skh = a->skh; P.sks = a->sks; P.svb = a->svb; P.svh = a->svh; P.svs = a->svs;
  P.ssb = a->ssb; P.ssh = a->ssh; P.stb = a->stb; P.sth = a->sth; P.sob = a->sob; P.soh = a->soh;
  P.B = a->B; P.H = a->H; P.KH = a->KH; P.G = a->H / a->KH; P.S = a->S; P.hd = a->hd;
  P.window = a->window; P.ring = a->ring ? 1 : 0; P.splits = a->num_splits; P.idx64 = a->idx_dtype == UVMI_I64;
  P.chunk_keys = a->chunk_keys > 0 ? ((a->chunk_keys + 31) & ~31) : 0;
  P.gran = 32;
  P.n_items = (int64_t)a->B * a->KH * a->num_splits;
  P.scale_log2 = a->scale * LOG2E;
  P.ws_o = P.ws_m = P.ws_l = nullptr;
  P.post_vhat = a->post_vhat; P.post_gate = a->post_gate; P.post_xsa = a->post_xsa; P.post_dt = a->post_round_dtype;
  P.f_qkv = nullptr; P.f_rope_tab = nullptr; P.f_rope_n = 1; P.f_rope = 0;
  if (const uvmi_attn_qkv_fuse* f = a->fuse) {
    UVMI_REQUIRE((mfma_ok(a) || mfma16_ok(a)) && a->num_splits == 1, UVMI_EUNSUPPORTED,
                 "uvmi_decode_attn: fused QKV post-processing needs the MFMA kernel (head_dim 64, int8 cache or one of the q dtype, aligned rows) and num_splits == 1");
    UVMI_REQUIRE(a->out_dtype == a->q_dtype, UVMI_EUNSUPPORTED, "uvmi_decode_attn: fused QKV post-processing writes the q dtype");
    UVMI_REQUIRE(f->qkv && ((uintptr_t)f->qkv % 16) == 0 && f->row_stride % 8 == 0 && f->ext_col >= (a->H + 2 * a->KH) * 64 &&
                     f->row_stride >= f->ext_col + a->H + a->KH, UVMI_EINVAL, "uvmi_decode_attn: bad fused qkv layout");
    UVMI_REQUIRE(!f->rope || (f->n_pairs == 16 && f->rope_table && f->rope_positions > 0 && ((uintptr_t)f->rope_table % 128) == 0), UVMI_EUNSUPPORTED,
                 "uvmi_decode_attn: fused rotation needs n_pairs == 16 and a 128-byte aligned rope_table");
    UVMI_REQUIRE(!f->has_ve || (f->ve_table && f->tok && f->vocab > 0 && ((uintptr_t)f->ve_table % 16) == 0), UVMI_EINVAL,
                 "uvmi_decode_attn: fused value embedding needs ve_table, tok and vocab");
    P.f_qkv = f->qkv; P.f_sqkv = f->row_stride; P.f_ext = f->ext_col; P.f_has_gate = f->has_gate ? 1 : 0;
    P.f_tok = f->tok; P.f_ve = f->ve_table; P.f_vocab = f->vocab; P.f_has_ve = f->has_ve ? 1 : 0;
    P.f_rope_tab = f->rope_table; P.f_rope_n = f->rope ? f->rope_positions : 1; P.f_rope = f->rope ? 1 : 0; P.f_eps = f->eps; P.f_xsa_eps = f->xsa_eps;
    P.post_vhat = nullptr; P.post_gate = nullptr;
  }
  if (a->post_vhat && !a->fuse) {
    UVMI_REQUIRE((mfma_ok(a) || mfma16_ok(a)) && a->num_splits == 1, UVMI_EUNSUPPORTED,
                 "uvmi_decode_attn: the fused post epilogue needs the MFMA kernel (head_dim 64, int8 cache or one of the q dtype) and num_splits == 1");
    UVMI_REQUIRE(is_float_dtype(a->post_round_dtype) && ((uintptr_t)a->post_vhat % 16) == 0, UVMI_EINVAL, "uvmi_decode_attn: bad post arguments");
  }
  if (a->num_splits > 1) {
    const size_t need = uvmi_decode_attn_workspace_bytes(a->B, a->H, a->KH, a->hd, a->num_splits);
    UVMI_REQUIRE(ws && ws_bytes >= need, UVMI_EWORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need, ws_bytes);
    UVMI_REQUIRE(((uintptr_t)ws % 16) == 0, UVMI_EWORKSPACE, "%s: workspace must be 16-byte aligned", who);
    const size_t rows = (size_t)a->B * a->H * a->num_splits;
    P.ws_o = (float*)ws;
    P.ws_m = P.ws_o + rows * a->hd;
    P.ws_l = P.ws_m + rows;
  }
  UVMI_REQUIRE(P.n_items < (1LL << 31), UVMI_EUNSUPPORTED, "uvmi_decode_attn: too many work items");
  const bool kv16 = !mfma_ok(a) && mfma16_ok(a);
  if (mfma_ok(a) || kv16) {
    // Waves per work item.  Long rows are streamed by all 4 waves of a workgroup, short ones by 2 or 1; and when 4 waves
    // per item would need more wave slots than the device has at this kernel's occupancy (4 per SIMD), 2 per item keep
    // the whole launch resident in one round instead of two (measured: 2000 rows x ~230 keys, 15.6 us against 18.9 us).
    // Already from 4/5 of the slots on, 2 waves per item are the faster form (measured inside a 2048-sequence rollout, whose
    // contexts are 800 - 1100 keys by then: steps of 832 - 1024 rows 0.589 - 0.607 ms against 0.609 - 0.621).
    const int ctx = a->window > 0 && a->window < a->S ? a->window : a->S;
    int wpr = ctx >= 256 ? 4 : (ctx >= 128 ? 2 : 1);
    {
      int cus = uvmi_device_cus();
      if (cus <= 0) cus = 256;
      const int64_t slots = (int64_t)cus * 16;
      while (wpr > 1 && P.n_items * wpr > slots && P.n_items * (wpr / 2) <= slots) wpr /= 2;
      if (wpr == 4 && P.n_items * 5 > slots) wpr = 2;
      // Rows of a known, short length - a window or ring of at most 512 keys, 16 tiles - are a chain of latencies rather than
      // a stream: they run fastest with about one wave per SIMD (measured on 256-key rings: 4 waves per row up to ~300 rows,
      // 2 up to ~650, 1 beyond; 500 rows 6.1 us with 2 against 6.9 with 4, 1000 rows 9.5 us with 1 against 9.8 with 2).  With
      // the fused QKV post-processing two waves keep sharing the row's own key and value up to the full device (1000 rows
      // 11.9 us with 2 against 12.5 with 1).
      if ((a->ring || (a->window > 0 && a->window < a->S)) && ctx <= 512) {
        if (wpr == 4 && P.n_items * 4 > (int64_t)cus * 5) wpr = 2;
        if (wpr == 2 && !a->fuse && P.n_items * 2 > (int64_t)cus * 5) wpr = 1;
      }
    }
    P.gran = 32 * wpr;
    if (P.chunk_keys) P.chunk_keys = (P.chunk_keys + P.gran - 1) / P.gran * P.gran;
    const int ipb = 4 / wpr;
    const dim3 grid((unsigned)((P.n_items + ipb - 1) / ipb)), blk(256);
#define UVMI_LEAD P.pos, P.starts, P.rows, (a->fuse ? P.f_qkv : P.q), P.n_items, P.idx64, P.splits, P.KH
#define UVMI_L(QD, OD)                                                                                \
  do {                                                                                                \
    if (wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD, 4, false>), grid, blk, 0, st, UVMI_LEAD, P);      \
    else if (wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD, 2, false>), grid, blk, 0, st, UVMI_LEAD, P); \
    else hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD, 1, false>), grid, blk, 0, st, UVMI_LEAD, P);               \
  } while (0)
#define UVMI_LF(QD)                                                                                   \
  do {                                                                                                \
    if (fast && wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 4, true, false, true>), grid, blk, 0, st, UVMI_LEAD, P);       \
    else if (fast && wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 2, true, false, true>), grid, blk, 0, st, UVMI_LEAD, P);  \
    else if (fast) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 1, true, false, true>), grid, blk, 0, st, UVMI_LEAD, P);              \
    else if (wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 4, true>), grid, blk, 0, st, UVMI_LEAD, P);  \
    else if (wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 2, true>), grid, blk, 0, st, UVMI_LEAD, P);  \
    else hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 1, true>), grid, blk, 0, st, UVMI_LEAD, P);                \
  } while (0)
#define UVMI_LFAST(QD)                                                                                \
  do {                                                                                                \
    if (wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 4, false, false, true>), grid, blk, 0, st, UVMI_LEAD, P);      \
    else if (wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 2, false, false, true>), grid, blk, 0, st, UVMI_LEAD, P); \
    else hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 1, false, false, true>), grid, blk, 0, st, UVMI_LEAD, P);               \
  } while (0)
#define UVMI_L16(QD, OD)                                                                              \
  do {                                                                                                \
    if (wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD, 4, false, true>), grid, blk, 0, st, UVMI_LEAD, P);      \
    else if (wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD, 2, false, true>), grid, blk, 0, st, UVMI_LEAD, P); \
    else hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, OD, 1, false, true>), grid, blk, 0, st, UVMI_LEAD, P);               \
  } while (0)
#define UVMI_LF16(QD)                                                                                 \
  do {                                                                                                \
    if (wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 4, true, true>), grid, blk, 0, st, UVMI_LEAD, P);      \
    else if (wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 2, true, true>), grid, blk, 0, st, UVMI_LEAD, P); \
    else hipLaunchKernelGGL((attn_mfma_i8_hd64<QD, QD, 1, true, true>), grid, blk, 0, st, UVMI_LEAD, P);               \
  } while (0)
    const int od = a->out_dtype;  // rows that fit one chunk are written directly even when num_splits > 1
    // the engine's decode-step shape has an instantiation of its own (see FAST)
    const bool fast = !kv16 && a->num_splits == 1 && a->KH == 1 && a->H == 8 && a->idx_dtype == UVMI_I64;
    if (probe) {
      UVMI_REQUIRE(fast && !a->fuse && od == a->q_dtype && a->q_dtype == UVMI_BF16, UVMI_EUNSUPPORTED,
                   "uvmi_decode_attn_probe: only the engine's decode shape (int8 cache, bf16 q and output, 8 heads on 1 kv head, 64-bit indices, one split, no fused QKV)");
#define UVMI_LP(PR)                                                                                                                   \
  do {                                                                                                                                \
    if (wpr == 4) hipLaunchKernelGGL((attn_mfma_i8_hd64<UVMI_BF16, UVMI_BF16, 4, false, false, true, PR>), grid, blk, 0, st, UVMI_LEAD, P);      \
    else if (wpr == 2) hipLaunchKernelGGL((attn_mfma_i8_hd64<UVMI_BF16, UVMI_BF16, 2, false, false, true, PR>), grid, blk, 0, st, UVMI_LEAD, P); \
    else hipLaunchKernelGGL((attn_mfma_i8_hd64<UVMI_BF16, UVMI_BF16, 1, false, false, true, PR>), grid, blk, 0, st, UVMI_LEAD, P);               \
  } while (0)
      if (probe == 1) UVMI_LP(1); else UVMI_LP(2);
#undef UVMI_LP
    } else if (kv16 && a->fuse) {
      if (a->q_dtype == UVMI_F16) UVMI_LF16(UVMI_F16); else UVMI_LF16(UVMI_BF16);
    } else if (kv16) {
      if (a->q_dtype == UVMI_F16) {
        if (od == UVMI_F16) UVMI_L16(UVMI_F16, UVMI_F16); else if (od == UVMI_BF16) UVMI_L16(UVMI_F16, UVMI_BF16); else UVMI_L16(UVMI_F16, UVMI_F32);
      } else {
        if (od == UVMI_F16) UVMI_L16(UVMI_BF16, UVMI_F16); else if (od == UVMI_BF16) UVMI_L16(UVMI_BF16, UVMI_BF16); else UVMI_L16(UVMI_BF16, UVMI_F32);
      }
    } else if (a->fuse) {
      if (a->q_dtype == UVMI_F16) UVMI_LF(UVMI_F16); else UVMI_LF(UVMI_BF16);
    } else if (fast && od == a->q_dtype) {
      if (a->q_dtype == UVMI_F16) UVMI_LFAST(UVMI_F16); else UVMI_LFAST(UVMI_BF16);
    } else if (a->q_dtype == UVMI_F16) {
      if (od == UVMI_F16) UVMI_L(UVMI_F16, UVMI_F16); else if (od == UVMI_BF16) UVMI_L(UVMI_F16, UVMI_BF16); else UVMI_L(UVMI_F16, UVMI_F32);
    } else {
      if (od == UVMI_F16) UVMI_L(UVMI_BF16, UVMI_F16); else if (od == UVMI_BF16) UVMI_L(UVMI_BF16, UVMI_BF16); else UVMI_L(UVMI_BF16, UVMI_F32);
    }
#undef UVMI_L
#undef UVMI_LF
#undef UVMI_LFAST
#undef UVMI_L16
#undef UVMI_LF16
#undef UVMI_LEAD
  } else {
    const dim3 grid((unsigned)P.n_items), blk(64);
    const size_t sh = ((size_t)P.G * a->hd + (size_t)P.G * 64) * 4;
    const int od = a->out_dtype;
#define UVMI_L(QD, KD, OD) hipLaunchKernelGGL((attn_generic<QD, KD, OD>), grid, blk, sh, st, P)
#define UVMI_LO(QD, KD) do { if (od == UVMI_F16) UVMI_L(QD, KD, UVMI_F16); else if (od == UVMI_BF16) UVMI_L(QD, KD, UVMI_BF16); else UVMI_L(QD, KD, UVMI_F32); } while (0)
#define UVMI_LK(QD) do { if (a->kv_dtype == UVMI_I8) UVMI_LO(QD, UVMI_I8); else if (a->kv_dtype == UVMI_F16) UVMI_LO(QD, UVMI_F16); else if (a->kv_dtype == UVMI_F32) UVMI_LO(QD, UVMI_F32); else UVMI_LO(QD, UVMI_BF16); } while (0)
    if (a->q_dtype == UVMI_F16) UVMI_LK(UVMI_F16); else if (a->q_dtype == UVMI_F32) UVMI_LK(UVMI_F32); else UVMI_LK(UVMI_BF16);
#undef UVMI_LK
#undef UVMI_LO
#undef UVMI_L
  }
  UVMI_CHECK_LAUNCH("uvmi_decode_attn");
  if (a->num_splits > 1) {
    const int64_t rows = (int64_t)a->B * a->KH;
    const dim3 grid((unsigned)((rows + 3) / 4)), blk(256);
    if (a->out_dtype == UVMI_F16) hipLaunchKernelGGL((attn_combine<UVMI_F16>), grid, blk, 0, st, P);
    else if (a->out_dtype == UVMI_BF16) hipLaunchKernelGGL((attn_combine<UVMI_BF16>), grid, blk, 0, st, P);
    else hipLaunchKernelGGL((attn_combine<UVMI_F32>), grid, blk, 0, st, P);
    UVMI_CHECK_LAUNCH("uvmi_decode_attn(combine)");
  }
  return UVMI_OK;
}

extern "C" int uvmi_decode_attn(const uvmi_attn_args* a, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_decode_attn: null args");
  return decode_attn_launch(a, a->workspace, a->workspace_bytes, "uvmi_decode_attn", stream);
}

extern "C" int uvmi_decode_attn_probe(const uvmi_attn_args* a, int mode, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_decode_attn_probe: null args");
  UVMI_REQUIRE(mode == 1 || mode == 2, UVMI_EINVAL, "uvmi_decode_attn_probe: mode %d (1: memory stream only, 2: arithmetic only)", mode);
  return decode_attn_launch(a, a->workspace, a->workspace_bytes, "uvmi_decode_attn_probe", stream, mode);
}

// ------------------------------------------------------------------------------------ the entry point that allocates nothing
// Split partials of uvmi_decode_attn_noalloc live in this array instead of a caller's workspace.  It is part of the
// library's code object: every GPU the library runs on holds its own copy, at its own address, until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress - never a device address.
static __device__ __align__(256) unsigned char scratch[UVMI_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device ordinal, resolved on the first call there
}  // namespace

extern "C" int uvmi_decode_attn_noalloc(const uvmi_attn_args* a, void* stream) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_decode_attn_noalloc: null args");
  void* ws = nullptr;
  if (a->num_splits > 1) {
    const size_t need = uvmi_decode_attn_workspace_bytes(a->B, a->H, a->KH, a->hd, a->num_splits);
    UVMI_REQUIRE(need <= (size_t)UVMI_NOALLOC_SCRATCH_BYTES, UVMI_EWORKSPACE,
                 "uvmi_decode_attn_noalloc: B=%d H=%d num_splits=%d needs %zu bytes of split partials, the built-in scratch holds %zu; "
                 "use fewer splits or uvmi_decode_attn with a workspace", a->B, a->H, a->num_splits, need, (size_t)UVMI_NOALLOC_SCRATCH_BYTES);
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    UVMI_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, UVMI_EHIP, "uvmi_decode_attn_noalloc: hipGetDevice: %s (device %d)",
                 hipGetErrorString(e), dev);
    {
      std::lock_guard<std::mutex> lock(g_scratch_mu);
      if (!g_scratch_ptr[dev]) {  // once per device, with that device current
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        UVMI_REQUIRE(e == hipSuccess && p, UVMI_EHIP, "uvmi_decode_attn_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
      }
      ws = g_scratch_ptr[dev];
    }
  }
  return decode_attn_launch(a, ws, ws ? (size_t)UVMI_NOALLOC_SCRATCH_BYTES : 0, "uvmi_decode_attn_noalloc", stream);
}
