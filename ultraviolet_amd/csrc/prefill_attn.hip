// Packed causal self-attention with an optional sliding window over unquantized K/V: the attention of a packed prefill.
//
// Contract (ultraviolet/kernels/varlen_attn.py:87-115 of the reference): q (N, H, hd), k / v (N, KH, hd) hold the
// tokens of several sequences back to back, cu_seqlens their boundaries; query i sees keys j of its own sequence with
// i - window < j <= i.
//
// prefill_attn_mfma_hd64 (head_dim 64, 16-bit q/k/v of one dtype, up to 8 query heads per kv head):
//   * a wave owns 16 consecutive packed tokens x 4 query heads of one kv head, and walks the keys in 32-key
//     super-tiles.  Query blocks are aligned to the packed index, not to the sequences: a block that straddles a
//     boundary walks the union of its rows' key ranges and masks per (row, key), so the grid is ceil(N / 16) blocks
//     with no search for "which sequence is block i in";
//   * S^T = K . Q^T with v_mfma_f32_16x16x32 (A = 16 keys x 32 dims, B = 32 dims x 16 rows): a lane of the accumulator
//     holds 4 consecutive keys of one query row, for two 16-key tiles A and B.  Exactly these 8 values, rounded to
//     the 16-bit input type, are the lane's slice of the B operand of O^T = V^T . P^T when contraction slot 8g+j is
//     key 4g+j of tile A (j < 4) or of tile B (j >= 4): probabilities never move between lanes;
//   * V^T operands come from 8-byte loads (lane = dims 4m..4m+3 of 8 keys) regrouped with v_perm_b32 into four
//     operands whose row m is head dim 4m + t; they are built once per super-tile and shared by the wave's 4 heads,
//     as are the K operands (16-byte reads, lane = key m, dims 8g..8g+7 of each half);
//   * the 4 waves of a workgroup are 2 consecutive query blocks x 2 head groups (4 blocks x 1 group for up to 4 query
//     heads per kv head) of one kv head and walk the same keys, so a super-tile of K and V is fetched once per workgroup:
//     each thread requests 16 bytes of K and of V two tiles ahead into registers, parks them in one of two LDS halves
//     (K rows chunk-swizzled, so the 16-byte operand reads are conflict-free) and the waves take their operands from
//     there, one barrier per tile; a wave skips the tiles outside its own block's key range;
//   * online softmax per (row, head) in the exp2 domain; tiles that every row of the block sees completely skip the
//     mask arithmetic (one branch per tile, so the four heads of a tile form one block the scheduler interleaves);
//   * workgroup ids are remapped so that each XCD (one L2 each) owns a contiguous range of query blocks and therefore
//     whole sequences.
//
// Everything else (fp32 K/V, other head dims) goes token by token through the decode kernel's generic path with the
// packed K/V as a batch-stride-0 "cache".
#include "common.h"
#include "attn_mfma_util.h"

#include <climits>
#include <type_traits>

namespace uvmi {

struct PrefillParams {
  const void* q; const void* k; const void* v; void* out;
  const int32_t* seg_start;  // (N,) packed index of the first token of each token's sequence
  int64_t sqn, sqh, skn, skh, svn, svh, son, soh;
  int N, H, KH, G, window, n_hg;   // n_hg: head groups of 4 query heads per kv head, 1 or 2
  int n_wg;                        // workgroups with work: ceil(query blocks / (4 / n_hg)) * KH
  float scale_log2;
  const float* post_vhat; const float* post_gate; const float* post_xsa;  // fused Attention.post epilogue when post_vhat != null
  float* lse_out; int64_t lse_stride;  // optional (H, lse_stride) fp32: log2 of each row's sum of exp2(scale_log2 s) (the backward's statistics)
};

// seg_start[i] = cu[s] for the last s with cu[s] <= i (empty sequences are skipped); pidx[i] = i.
__global__ __launch_bounds__(256) void prefill_segments(const void* cu, int idx64, int n_seg, int N, int32_t* seg_start, int32_t* pidx) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  int lo = 0, hi = n_seg;  // invariant: cu[lo] <= i, and hi == n_seg or cu[hi] > i
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (load_index(cu, idx64, mid) <= i) lo = mid; else hi = mid;
  }
  seg_start[i] = (int32_t)load_index(cu, idx64, lo);
  pidx[i] = i;
}

struct PTile {   // one 32-key super-tile as loaded (32 dwords per lane)
  pu4 k[4];      // [tile A dims 0..31, tile A dims 32..63, tile B dims 0..31, tile B dims 32..63]: key m, dims 8g..8g+7
  pu2 v[8];      // keys 4g+j of tile A (j < 4) / tile B (j >= 4), dims 4m..4m+3
};

constexpr int HPW = 4;  // query heads per wave

constexpr int RING = 2;  // super-tiles requested ahead of the one being parked in LDS

template <int DT, int ODT>
__global__ __launch_bounds__(256) void prefill_attn_mfma_hd64(PrefillParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[2][2][4096];  // [half][K, V][32 keys x 128 B]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // gridDim.x is a multiple of 8; ids congruent mod 8 run on one XCD and get a contiguous range of work
  const int per = gridDim.x >> 3;
  const int bid = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (bid >= P.n_wg) return;   // (the whole workgroup: no barrier is left waiting)
  const int kvh = bid % P.KH;
  const int qg = bid / P.KH;               // group of 4 / n_hg consecutive query blocks
  const int hsh = P.n_hg - 1;              // n_hg is 1 or 2
  const int qbw = 4 >> hsh;
  const int hg = wave & hsh;
  const int qb = qg * qbw + (wave >> hsh);
  const int m = lane & 15, g = lane >> 4;
  const int G = P.G;
  const float c = P.scale_log2;

  // ---- this lane's query row (accumulator column m) and its key range; a wave whose block starts past the last token
  // (the tail of the last group) has an empty range and only helps with the loads
  const int r0 = qb * 16;
  const bool wave_ok = r0 < P.N;
  const int row = r0 + m;
  const bool row_ok = row < P.N;
  const int rowc = row_ok ? row : P.N - 1;
  int lo_n = P.seg_start[rowc];
  if (P.window > 0 && row - P.window + 1 > lo_n) lo_n = row - P.window + 1;
  if (!row_ok) lo_n = INT_MAX;
  const int rl = min(r0 + 15, P.N - 1);                                       // last real row of the block
  const int lo_first = __builtin_amdgcn_readfirstlane(lo_n);                  // lo is non-decreasing in the row
  const int lo_last = __builtin_amdgcn_readfirstlane(__shfl(lo_n, wave_ok ? rl - r0 : 0, 64));
  const int kbeg = wave_ok ? lo_first & ~31 : 0, kend = wave_ok ? rl + 1 : 0;
  // ---- the workgroup's key range: from the first row's lower bound (the smallest of the group) to its last row
  const int row0 = qg * qbw * 16;          // < N
  int lo0 = P.seg_start[row0];
  if (P.window > 0 && row0 - P.window + 1 > lo0) lo0 = row0 - P.window + 1;
  const int kbeg_wg = __builtin_amdgcn_readfirstlane(lo0) & ~31;
  const int kend_wg = min(row0 + qbw * 16, P.N);
  const int nk = (kend_wg - kbeg_wg + 31) >> 5;   // >= 1

  // ---- Q^T operands: lane (row m, group g) holds q[row][head][32 s + 8 g .. + 8] for s = 0, 1
  pu4 Q[HPW][2];
#pragma unroll
  for (int hh = 0; hh < HPW; hh++) {
    const int hq = hg * HPW + hh;
    Q[hh][0] = Q[hh][1] = pu4{0u, 0u, 0u, 0u};
    if (hq < G) {
      const uint16_t* qp = (const uint16_t*)P.q + (int64_t)rowc * P.sqn + (int64_t)(kvh * G + hq) * P.sqh + 8 * g;
      Q[hh][0] = *(const pu4*)qp;
      Q[hh][1] = *(const pu4*)(qp + 32);
    }
  }

  pf4 O[HPW][4];
  float mrun[HPW], lrun[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; hh++) {
#pragma unroll
    for (int t = 0; t < 4; t++) O[hh][t] = pf4{0.f, 0.f, 0.f, 0.f};
    mrun[hh] = -INFINITY;
    lrun[hh] = 0.f;
  }

  // ---- addressing: one descriptor per stream, per-lane byte offsets
  const uint16_t* kbase = (const uint16_t*)P.k + (int64_t)kvh * P.skh;
  const uint16_t* vbase = (const uint16_t*)P.v + (int64_t)kvh * P.svh;
  const uint32_t skn2 = (uint32_t)P.skn * 2, svn2 = (uint32_t)P.svn * 2;  // row strides in bytes
  const __amdgpu_buffer_rsrc_t rK = __builtin_amdgcn_make_buffer_rsrc((void*)kbase, 0, (int)((uint32_t)(P.N - 1) * skn2 + 128), 0x00020000);
  const __amdgpu_buffer_rsrc_t rV = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, (int)((uint32_t)(P.N - 1) * svn2 + 128), 0x00020000);

  // ---- K / V super-tiles go global -> registers (RING tiles ahead) -> LDS (two halves) -> MFMA operands.  Thread t moves
  // 16 bytes of K and of V per tile: key t / 8, chunk t % 8 of the 128-byte row.  Rows are clamped to N - 1 (the keys of a
  // clamped row are masked); tiles past the group's last are re-reads of the last one.  K rows are stored with their
  // 16-byte chunks XOR-swizzled by (key / 2) % 8, which makes both the stores and the operand reads (lane = key m, chunk
  // 4 s + g) free of bank conflicts; V rows are stored as they are (an operand read takes whole 128-byte rows).
  pu4 rk[RING], rv[RING];
  const int lkey = tid >> 3, lch = tid & 7;
  const uint32_t kst = (uint32_t)lkey * 128 + (uint32_t)((lch ^ ((lkey >> 1) & 7)) << 4), vst = (uint32_t)lkey * 128 + (uint32_t)lch * 16;
  auto fetch = [&](int k, int slot) {
    const int tb = kbeg_wg + 32 * min(k, nk - 1);
    const uint32_t r = (uint32_t)min(tb + lkey, P.N - 1);
    rk[slot] = __builtin_amdgcn_raw_buffer_load_b128(rK, r * skn2 + 16 * lch, 0, 0);
    rv[slot] = __builtin_amdgcn_raw_buffer_load_b128(rV, r * svn2 + 16 * lch, 0, 0);
  };
  auto park = [&](int slot, int half) {
    *(pu4*)(&smem[half][0][kst]) = rk[slot];
    *(pu4*)(&smem[half][1][vst]) = rv[slot];
  };
  const uint32_t kld0 = (uint32_t)m * 128 + (uint32_t)((g ^ ((m >> 1) & 7)) << 4), kld1 = (uint32_t)m * 128 + (uint32_t)(((4 + g) ^ ((m >> 1) & 7)) << 4);
  const uint32_t vld = (uint32_t)(4 * g) * 128 + 8 * m;
  auto read_tile = [&](int half, PTile& T) {
    const unsigned char* sk = smem[half][0];
    const unsigned char* sv = smem[half][1];
    T.k[0] = *(const pu4*)(sk + kld0);
    T.k[1] = *(const pu4*)(sk + kld1);
    T.k[2] = *(const pu4*)(sk + 2048 + kld0);
    T.k[3] = *(const pu4*)(sk + 2048 + kld1);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      T.v[j] = *(const pu2*)(sv + vld + 128 * j);
      T.v[4 + j] = *(const pu2*)(sv + 2048 + vld + 128 * j);
    }
  };

  auto step_t = [&](const PTile& T, int tb, auto EDGE) {
    constexpr bool edge = decltype(EDGE)::value;
    // V^T operands: operand t, row m is head dim 4m + t; dword p of an operand holds contraction slots 2p, 2p+1
    pu4 VA[4];
    {
      constexpr uint32_t LO = 0x05040100u, HI = 0x07060302u;
#pragma unroll
      for (int p = 0; p < 4; p++) {
        VA[0][p] = __builtin_amdgcn_perm(T.v[2 * p + 1].x, T.v[2 * p].x, LO);
        VA[1][p] = __builtin_amdgcn_perm(T.v[2 * p + 1].x, T.v[2 * p].x, HI);
        VA[2][p] = __builtin_amdgcn_perm(T.v[2 * p + 1].y, T.v[2 * p].y, LO);
        VA[3][p] = __builtin_amdgcn_perm(T.v[2 * p + 1].y, T.v[2 * p].y, HI);
      }
    }
    const int kA = tb + 4 * g, kB = kA + 16;  // first of this lane's 4 keys in tile A / B
#pragma unroll
    for (int hh = 0; hh < HPW; hh++) {
      pf4 sA = pf4{0.f, 0.f, 0.f, 0.f}, sB = pf4{0.f, 0.f, 0.f, 0.f};
      sA = mfma16<DT>(T.k[0], Q[hh][0], sA);
      sB = mfma16<DT>(T.k[2], Q[hh][0], sB);
      sA = mfma16<DT>(T.k[1], Q[hh][1], sA);
      sB = mfma16<DT>(T.k[3], Q[hh][1], sB);
      float t[8] = {sA[0], sA[1], sA[2], sA[3], sB[0], sB[1], sB[2], sB[3]};
      if (edge) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          if (kA + i < lo_n || kA + i > row) t[i] = -INFINITY;
          if (kB + i < lo_n || kB + i > row) t[4 + i] = -INFINITY;
        }
      }
      float mx = fmaxf(fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3])), fmaxf(fmaxf(t[4], t[5]), fmaxf(t[6], t[7])));
      mx = pmax32(pmax16(mx));
      {  // rescale by alpha = exp2((m_old - m_new) c), 1 where the row's maximum did not grow.  Unconditional: a branch
         // here would split the four heads into separate blocks and stop the scheduler from overlapping one head's
         // softmax arithmetic with the next head's MFMAs
        const float mnew = fmaxf(mrun[hh], mx);
        const float alpha = mnew == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f((mrun[hh] - mnew) * c);
#pragma unroll
        for (int tt = 0; tt < 4; tt++) O[hh][tt] *= alpha;
        lrun[hh] *= alpha;
        mrun[hh] = mnew;
      }
      const float mc = mrun[hh] == -INFINITY ? 0.f : mrun[hh] * c;
      float p[8];
#pragma unroll
      for (int i = 0; i < 8; i++) p[i] = __builtin_amdgcn_exp2f(fmaf(t[i], c, -mc));
      lrun[hh] += ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
      const pu4 PB = pu4{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7])};
#pragma unroll
      for (int tt = 0; tt < 4; tt++) O[hh][tt] = mfma16<DT>(VA[tt], PB, O[hh][tt]);
    }
  };

  // the mask test is hoisted out of the head loop (one branch per tile, two straight-line bodies), so that the four
  // heads of a tile form one block the scheduler can interleave
  auto step = [&](const PTile& T, int tb, bool edge) {
    if (edge) step_t(T, tb, std::true_type{}); else step_t(T, tb, std::false_type{});
  };

  {
    // a tile needs no mask when every row of the block sees all of it: it starts at or after the last row's lower
    // bound and ends at or before the first row
    auto edge_of = [&](int tb) { return !(tb >= lo_last && tb + 31 <= r0); };
    // iteration k: this wave's operands of tile k come out of LDS half k % 2 (when the tile lies in the wave's own range),
    // tile k + 1 is parked in the other half, tile k + 1 + RING is requested into the ring slot that frees, then the
    // arithmetic of tile k runs; the barrier lets the next iteration overwrite the half just read
    auto iteration = [&](int k, int d) {
      const int tb = kbeg_wg + 32 * k;
      const bool act = tb >= kbeg && tb < kend;   // wave-uniform
      PTile T;
      if (act) read_tile(k & 1, T);
      park((d + 1) % RING, (k + 1) & 1);
      fetch(k + 1 + RING, (d + 1) % RING);
      if (act) step(T, tb, edge_of(tb));
      __syncthreads();
    };
#pragma unroll
    for (int d = 0; d < RING; d++) fetch(d, d);
    park(0, 0);
    fetch(RING, 0);
    __syncthreads();
    int k = 0;
    for (; k + RING <= nk; k += RING) {
#pragma unroll
      for (int d = 0; d < RING; d++) iteration(k + d, d);
    }
#pragma unroll
    for (int d = 0; d < RING - 1; d++)
      if (k + d < nk) iteration(k + d, d);   // workgroup-uniform
  }

  // ---- normalise and store: lane (row m, group g) holds head dims 16g .. 16g+15 (O[t][i] is dim 16g + 4i + t)
  // Optional epilogue, as in the decode kernel: z (rounded to the activation type, as the attention output tensor would be)
  // -> XSA with the token's normalised v -> per-head gate; the 4 lane groups of a row reduce z . v_hat between them.
  const bool has_post = P.post_vhat != nullptr;
  float vv[16];
  if (has_post) {
    const float* vp = P.post_vhat + ((int64_t)rowc * P.KH + kvh) * 64 + 16 * g;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float4 x = *(const float4*)(vp + 4 * i);
      vv[4 * i] = x.x; vv[4 * i + 1] = x.y; vv[4 * i + 2] = x.z; vv[4 * i + 3] = x.w;
    }
  }
  auto rnd = [&](float x) -> float { return DT == UVMI_BF16 ? bf16_to_float(float_to_bf16(x)) : (float)(half_t)x; };
#pragma unroll
  for (int hh = 0; hh < HPW; hh++) {
    const int hq = hg * HPW + hh;
    const float l = psum32(psum16(lrun[hh]));
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (P.lse_out && g == 0 && hq < G && row_ok)   // (+inf for a row without keys: its probabilities come out as 0)
      P.lse_out[(int64_t)(kvh * G + hq) * P.lse_stride + row] = l > 0.f ? mrun[hh] * c + __builtin_amdgcn_logf(l) : INFINITY;
    if (P.out == nullptr) continue;   // statistics only
    float o[16];
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int i = 0; i < 4; i++) o[4 * i + t] = O[hh][t][i] * inv;
    if (has_post) {  // (every lane takes part in the reduction; lanes of absent heads / rows compute on clamped operands)
      const int head = kvh * G + (hq < G ? hq : G - 1);
      float proj = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        o[i] = rnd(o[i]);
        proj += o[i] * vv[i];
      }
      if (P.post_xsa) {
        proj = psum32(psum16(proj));
        const float ah = P.post_xsa[head] * proj;
#pragma unroll
        for (int i = 0; i < 16; i++) o[i] = rnd(o[i] - ah * vv[i]);
      }
      const float gate = P.post_gate ? P.post_gate[(int64_t)rowc * P.H + head] : 1.0f;
#pragma unroll
      for (int i = 0; i < 16; i++) o[i] *= gate;
    }
    if (hq >= G || !row_ok) continue;
    const int64_t off = (int64_t)row * P.son + (int64_t)(kvh * G + hq) * P.soh + 16 * g;
    if (ODT == UVMI_F32) {
      float* op = (float*)P.out + off;
#pragma unroll
      for (int i = 0; i < 4; i++) *(float4*)(op + 4 * i) = float4{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    } else {
      uint32_t w[8];
#pragma unroll
      for (int i = 0; i < 8; i++) w[i] = ODT == UVMI_BF16 ? pack2<UVMI_BF16>(o[2 * i], o[2 * i + 1]) : pack2<UVMI_F16>(o[2 * i], o[2 * i + 1]);
      uint16_t* op = (uint16_t*)P.out + off;
      *(uint4*)op = uint4{w[0], w[1], w[2], w[3]};
      *(uint4*)(op + 8) = uint4{w[4], w[5], w[6], w[7]};
    }
  }
}

// ---------------------------------------------------------------------------------------------------- host side
static int check_prefill(const uvmi_prefill_attn_args* a) {
  UVMI_REQUIRE(a, UVMI_EINVAL, "uvmi_prefill_attn: null args");
  UVMI_REQUIRE(a->N >= 0 && a->H > 0 && a->KH > 0 && a->hd > 0 && a->n_seg >= 0, UVMI_EINVAL, "uvmi_prefill_attn: bad sizes");
  if (a->N == 0) return UVMI_OK;
  UVMI_REQUIRE(a->q && a->k && a->v && a->cu_seqlens && a->out, UVMI_EINVAL, "uvmi_prefill_attn: null pointer");
  UVMI_REQUIRE(a->n_seg >= 1, UVMI_EINVAL, "uvmi_prefill_attn: N > 0 needs at least one sequence");
  UVMI_REQUIRE(a->H % a->KH == 0, UVMI_EINVAL, "uvmi_prefill_attn: H=%d is not a multiple of KH=%d", a->H, a->KH);
  UVMI_REQUIRE(a->q_dtype == UVMI_F16 || a->q_dtype == UVMI_BF16 || a->q_dtype == UVMI_F32, UVMI_EUNSUPPORTED,
               "uvmi_prefill_attn: q must be F16, BF16 or F32");
  UVMI_REQUIRE(is_float_dtype(a->kv_dtype), UVMI_EUNSUPPORTED, "uvmi_prefill_attn: k/v must be F16, BF16 or F32");
  UVMI_REQUIRE(is_float_dtype(a->out_dtype), UVMI_EUNSUPPORTED, "uvmi_prefill_attn: out must be F16, BF16 or F32");
  UVMI_REQUIRE(a->idx_dtype == UVMI_I64 || a->idx_dtype == UVMI_I32, UVMI_EINVAL, "uvmi_prefill_attn: cu_seqlens must be I32 or I64");
  UVMI_REQUIRE(a->window >= 0, UVMI_EINVAL, "uvmi_prefill_attn: negative window");
  UVMI_REQUIRE(a->hd <= 256 && a->H / a->KH <= 16, UVMI_EUNSUPPORTED, "uvmi_prefill_attn: head_dim %d / group %d beyond 256 / 16", a->hd,
               a->H / a->KH);
  const size_t need = uvmi_prefill_attn_workspace_bytes(a->N);
  UVMI_REQUIRE(a->workspace && a->workspace_bytes >= need, UVMI_EWORKSPACE, "uvmi_prefill_attn: workspace of %zu bytes needed, %zu given",
               need, a->workspace_bytes);
  UVMI_REQUIRE(((uintptr_t)a->workspace % 16) == 0, UVMI_EWORKSPACE, "uvmi_prefill_attn: workspace must be 16-byte aligned");
  return UVMI_OK;
}

static bool prefill_mfma_ok_stats(const uvmi_prefill_attn_args* a) {   // (as below, without an output tensor)
  if (a->hd != 64 || a->H / a->KH > 8 || a->kv_dtype != a->q_dtype || a->q_dtype == UVMI_F32) return false;   // 16-bit operands
  if (!(a->scale > 0.f)) return false;
  auto al = [](const void* p, int n) { return ((uintptr_t)p % n) == 0; };
  if (!al(a->q, 16) || a->sqn % 8 || a->sqh % 8) return false;
  if (!al(a->k, 16) || a->skn % 8 || a->skh % 8 || !al(a->v, 16) || a->svn % 8 || a->svh % 8) return false;
  if (a->skn <= 0 || a->svn <= 0) return false;
  if ((int64_t)a->N * a->skn * 2 >= (1LL << 31) || (int64_t)a->N * a->svn * 2 >= (1LL << 31)) return false;
  return true;
}

static bool prefill_mfma_ok(const uvmi_prefill_attn_args* a) {
  if (a->hd != 64 || a->H / a->KH > 8 || a->kv_dtype != a->q_dtype || a->q_dtype == UVMI_F32) return false;   // 16-bit operands
  if (!(a->scale > 0.f)) return false;  // the running maximum is tracked before the (positive) softmax scale
  auto al = [](const void* p, int n) { return ((uintptr_t)p % n) == 0; };
  if (!al(a->q, 16) || a->sqn % 8 || a->sqh % 8) return false;
  if (!al(a->k, 16) || a->skn % 8 || a->skh % 8 || !al(a->v, 16) || a->svn % 8 || a->svh % 8) return false;
  if (a->skn <= 0 || a->svn <= 0) return false;
  if ((int64_t)a->N * a->skn * 2 >= (1LL << 31) || (int64_t)a->N * a->svn * 2 >= (1LL << 31)) return false;  // 32-bit buffer offsets
  const int ob = a->out_dtype == UVMI_F32 ? 4 : 2;
  if (!al(a->out, 16) || (a->son * ob) % 16 || (a->soh * ob) % 16) return false;
  return true;
}

static int launch_mfma(const uvmi_prefill_attn_args* a, const int32_t* seg_start, float* lse_out, int64_t lse_stride, hipStream_t st) {
  PrefillParams P;
  P.q = a->q; P.k = a->k; P.v = a->v; P.out = a->out; P.seg_start = seg_start;
  P.sqn = a->sqn; P.sqh = a->sqh; P.skn = a->skn; P.skh = a->skh; P.svn = a->svn; P.svh = a->svh; P.son = a->son; P.soh = a->soh;
  P.N = a->N; P.H = a->H; P.KH = a->KH; P.G = a->H / a->KH; P.window = a->window;
  P.n_hg = (P.G + HPW - 1) / HPW;   // 1 or 2 (G <= 8)
  const int64_t n_qb = (a->N + 15) / 16, qbw = 4 / P.n_hg;
  const int64_t n_wg = (n_qb + qbw - 1) / qbw * a->KH;
  P.scale_log2 = a->scale * 1.4426950408889634f;
  P.post_vhat = a->post_vhat; P.post_gate = a->post_gate; P.post_xsa = a->post_xsa;
  P.lse_out = lse_out; P.lse_stride = lse_stride;
  UVMI_REQUIRE(n_wg < (1LL << 30), UVMI_EUNSUPPORTED, "uvmi_prefill_attn: too many work items");
  P.n_wg = (int)n_wg;
  const unsigned nblk = (unsigned)((n_wg + 7) / 8 * 8);
  const dim3 grid(nblk), blk(256);
  const int od = a->out_dtype;
#define UVMI_L(QD)                                                                                                \
  do {                                                                                                            \
    if (od == UVMI_F16) hipLaunchKernelGGL((prefill_attn_mfma_hd64<QD, UVMI_F16>), grid, blk, 0, st, P);          \
    else if (od == UVMI_BF16) hipLaunchKernelGGL((prefill_attn_mfma_hd64<QD, UVMI_BF16>), grid, blk, 0, st, P);   \
    else hipLaunchKernelGGL((prefill_attn_mfma_hd64<QD, UVMI_F32>), grid, blk, 0, st, P);                         \
  } while (0)
  if (a->q_dtype == UVMI_F16) UVMI_L(UVMI_F16); else UVMI_L(UVMI_BF16);
#undef UVMI_L
  UVMI_CHECK_LAUNCH("uvmi_prefill_attn");
  return UVMI_OK;
}

// For the backward (prefill_attn_bwd.hip): the segment table of cu_seqlens into seg_start (N ints; pidx: N ints of scratch) and
// the rows' softmax statistics into lse (H, lse_stride), from one forward pass that stores no output.  a->out may be null.
int prefill_attn_stats(const uvmi_prefill_attn_args* a, int32_t* seg_start, int32_t* pidx, float* lse, int64_t lse_stride, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(prefill_segments, dim3((unsigned)((a->N + 255) / 256)), dim3(256), 0, st, a->cu_seqlens, a->idx_dtype == UVMI_I64 ? 1 : 0,
                     a->n_seg, a->N, seg_start, pidx);
  UVMI_CHECK_LAUNCH("uvmi_prefill_attn_bwd(segments)");
  uvmi_prefill_attn_args b = *a;
  b.out = nullptr; b.out_dtype = a->q_dtype; b.son = (int64_t)a->H * 64; b.soh = 64;
  b.post_vhat = nullptr; b.post_gate = nullptr; b.post_xsa = nullptr;
  UVMI_REQUIRE(prefill_mfma_ok_stats(&b), UVMI_EUNSUPPORTED, "uvmi_prefill_attn_bwd: q / k / v layout not served by the MFMA kernels");
  return launch_mfma(&b, seg_start, lse, lse_stride, st);
}

}  // namespace uvmi

using namespace uvmi;

extern "C" size_t uvmi_prefill_attn_workspace_bytes(int N) {
  if (N <= 0) return 0;
  return (((size_t)N * 4 + 255) / 256 * 256) * 2;
}

extern "C" int uvmi_prefill_attn_path(const uvmi_prefill_attn_args* a) {
  int rc = check_prefill(a);
  if (rc) return rc;
  return prefill_mfma_ok(a) ? 1 : 0;
}

extern "C" int uvmi_prefill_attn(const uvmi_prefill_attn_args* a, void* stream) {
  int rc = check_prefill(a);
  if (rc) return rc;
  if (a->N == 0) return UVMI_OK;
  hipStream_t st = (hipStream_t)stream;
  int32_t* seg_start = (int32_t*)a->workspace;
  int32_t* pidx = (int32_t*)((char*)a->workspace + ((size_t)a->N * 4 + 255) / 256 * 256);
  if (!a->segments_ready) {
    hipLaunchKernelGGL(prefill_segments, dim3((unsigned)((a->N + 255) / 256)), dim3(256), 0, st, a->cu_seqlens, a->idx_dtype == UVMI_I64 ? 1 : 0,
                       a->n_seg, a->N, seg_start, pidx);
    UVMI_CHECK_LAUNCH("uvmi_prefill_attn(segments)");
  }
  if (a->post_vhat) {
    UVMI_REQUIRE(prefill_mfma_ok(a), UVMI_EUNSUPPORTED, "uvmi_prefill_attn: the fused post epilogue needs the MFMA kernel (head_dim 64, 16-bit q / k / v)");
    UVMI_REQUIRE(((uintptr_t)a->post_vhat % 16) == 0, UVMI_EINVAL, "uvmi_prefill_attn: post_vhat must be 16-byte aligned");
  }
  if (!prefill_mfma_ok(a)) {
    // every packed token is a decode row whose "cache" is the packed K / V of the call (batch stride 0)
    uvmi_attn_args d = {};
    d.q = a->q; d.q_dtype = a->q_dtype; d.sqb = a->sqn; d.sqh = a->sqh;
    d.k_cache = a->k; d.v_cache = a->v; d.kv_dtype = a->kv_dtype;
    d.skb = 0; d.skh = a->skh; d.sks = a->skn; d.svb = 0; d.svh = a->svh; d.svs = a->svn;
    d.pos = pidx; d.starts = seg_start; d.idx_dtype = UVMI_I32;
    d.out = a->out; d.out_dtype = a->out_dtype; d.sob = a->son; d.soh = a->soh;
    d.B = a->N; d.H = a->H; d.KH = a->KH; d.S = a->N; d.hd = a->hd;
    d.scale = a->scale; d.window = a->window; d.ring = 0; d.num_splits = 1;
    return uvmi_decode_attn(&d, stream);
  }
  return launch_mfma(a, seg_start, nullptr, 0, st);
}

