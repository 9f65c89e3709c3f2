// Skinny 16-bit GEMM for the projections of a small decode step: C[M, N] = A[M, K] . W[N, K]^T, fp32 accumulation, M of
// a few hundred rows at most.  These are the F.linear calls of the reference's fused inference path
// (ultraviolet/model.py:302-335 attention projections, 388-391 MLP).  At this size a projection is a weight-streaming
// problem - 0.7 to 4.3 MB of weights that the previous layer has pushed out of the L2, against a few hundred KB of
// activations - and a launch lasts as long as its longest chain of dependent memory round trips.  The kernel has one:
//
//   * a workgroup of 4 waves owns 64 rows x BN columns (BN = 16 or 32); wave w owns rows 16w..16w+15;
//   * at kernel start every thread requests its share of the workgroup's whole weight strip (BN rows x K, 8 consecutive
//     lanes on one 128-byte segment) and the first 16 K-steps of its wave's activation rows, all in one burst; nothing
//     that follows depends on another global load;
//   * the weight strip is parked in LDS (row pitch K * 2 + 16 bytes, which spreads the 16 rows of an operand read over
//     all banks) behind the only barrier of the kernel; the activation operand never touches LDS: lane (r, g) reads its
//     16 bytes of row r, k = 32 s + 8 g.., straight from global memory in MFMA operand order, through a ring of 16
//     registers-quads that is refilled as it is consumed (exact wait counts: the main loop's body has no branches);
//   * the MFMA's A input is the weight slab and its B input the activation slab, so the accumulator holds C^T: a lane
//     has 4 consecutive columns n of one row m and stores them as one 8-byte write;
//   * rows past M, weight rows past N and K-steps past K are cut off by the buffer bounds (offset pushed out of range:
//     zero, no traffic), so no branch surrounds a load;
//   * tiles are dealt to the XCDs in contiguous runs with the row block fastest, so all row blocks of a weight strip run
//     on one XCD and the strip leaves HBM once;
//   * epilogue SWIGLU: W holds w_gate and w_up interleaved in slabs of 16 rows, so with BN = 32 accumulator 0 is gate and
//     accumulator 1 is up of the same 16 output columns, and act = silu(g) * u is formed in registers with the roundings
//     of the separate SwiGLU pass (g, u and silu(g) rounded to the activation type): the (M, 2f) intermediate never exists;
//   * epilogue RESID: C = ca * R + cb * (A W^T) with a residual input R (M, N), the block's residual update
//     (ultraviolet/model.py:567-571) in the arithmetic of the separate residual-add kernel (the product rounded to the
//     activation type first, then the sum rounded);
//   * NORM: the activation rows are RMS-normalised on the fly.  RMSNorm has no weight here, so norm(a) W^T = rsqrt(mean(a^2)
//     + eps) * (a W^T): the kernel sums a^2 of its rows as their K-steps pass through the ring and scales the accumulator
//     once at the end - the normalised activations are never written (nor rounded to the activation type: the result is
//     the exact row scale of the un-normalised product, a rounding step closer to exact than the two-pass path).
#include "common.h"
#include "gemm_util.h"

namespace uvmi {

struct SkinnyParams {
  const void* a; const void* w; void* c;
  uint32_t lda2, ldw2;  // row pitches in bytes
  int64_t ldc;          // elements
  int M, N, K;
  int tiles_m, tiles_n;
};

constexpr int SK_BM = 64;       // rows per workgroup
constexpr int SK_RING = 16;     // activation K-steps (of 32) in flight per wave
// problems of at most this many 16-row x BN tiles split K over the waves of 16-row workgroups (measured on 640 / 1664-deep
// projections: faster up to ~500 workgroups, two per compute unit; beyond, the weight strips are re-read too often)
constexpr int SK_KSPLIT_TILES = 512;
constexpr int SK_WPASS = 16;    // most passes of the weight-strip load (32 (row, 128-byte segment) units per pass)

__device__ __forceinline__ float gxsum16(float v) {  // v + the value of lane l ^ 16
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float gxsum32(float v) {  // v + the value of lane l ^ 32
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// EPI 0: C = A W^T (M, N).  EPI 1 (BN = 32): W rows are [gate 16 | up 16] slabs; C = silu(gate) * up, (M, N / 2).
// EPI 2: C = ca * R + cb * (A W^T).  NORM: A stands for its RMS-normalised rows.
// (individual scalar arguments rather than a parameter block: they are preloaded into SGPRs with the wave, so the first
// loads need not wait for a load of the kernel arguments)
template <int DT, int BN, int EPI, bool NORM>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const void* a_a, const void* a_w, void* a_c, uint32_t a_lda2, uint32_t a_ldw2,
                                                          int a_M, int a_N, int a_K, int a_tiles_m, int a_tiles_n, int64_t a_ldc,
                                                          float a_eps, const void* a_res, int64_t a_ldr, float a_ca, float a_cb) {
  SkinnyParams P;
  P.a = a_a; P.w = a_w; P.c = a_c; P.lda2 = a_lda2; P.ldw2 = a_ldw2; P.ldc = a_ldc; P.M = a_M; P.N = a_N; P.K = a_K;
  P.tiles_m = a_tiles_m; P.tiles_n = a_tiles_n;
  extern __shared__ __attribute__((aligned(16))) unsigned char wlds[];  // BN rows of K * 2 + 16 bytes
  constexpr int TN = BN / 16;
  constexpr uint32_t OOB = 0x40000000u;  // added to an offset that must read as zero (every valid offset is below 2^30)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int T = P.tiles_m * P.tiles_n;
  const int per = (T + 7) / 8;
  const int L = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
  if (L >= T) return;
  const int bn = L / P.tiles_m, bm = L % P.tiles_m;
  const int m0 = bm * SK_BM, n0 = bn * BN;
  const int r = lane & 15, g = lane >> 4;
  const int ns = P.K / 32;                    // K-steps of one MFMA
  const int segs = P.K / 64;                  // 128-byte segments per weight row
  const uint32_t pitch = (uint32_t)P.K * 2 + 16;

  const uint32_t boundA = (uint32_t)(P.M - 1) * P.lda2 + (uint32_t)P.K * 2;
  const uint32_t boundW = (uint32_t)(P.N - 1) * P.ldw2 + (uint32_t)P.K * 2;
  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc((void*)P.a, 0, (int)boundA, 0x00020000);
  const __amdgpu_buffer_rsrc_t rW = __builtin_amdgcn_make_buffer_rsrc((void*)P.w, 0, (int)boundW, 0x00020000);

  // ---- weight strip: unit u = tid / 8 of a pass is (row u % BN, segment u / BN + (32 / BN) pass); lane tid % 8 takes
  // 16 bytes of the segment
  constexpr int SPP = 32 / BN;                // segments per pass
  const int wrow = (tid >> 3) % BN, wseg0 = (tid >> 3) / BN, wch = tid & 7;
  const int passes = (segs + SPP - 1) / SPP;
  const uint32_t wbase = (n0 + wrow < P.N ? 0u : OOB) + (uint32_t)(n0 + wrow) * P.ldw2 + 16 * wch;
  gu4 wst[SK_WPASS];
#pragma unroll
  for (int p = 0; p < SK_WPASS; p++) {
    const int seg = wseg0 + SPP * p;
    wst[p] = __builtin_amdgcn_raw_buffer_load_b128(rW, wbase + (seg < segs ? (uint32_t)seg * 128 : OOB), 0, 0);
  }
  // ---- activation operand ring: lane (r, g) holds A[m0 + 16 wave + r][32 s + 8 g .. + 8] of K-step s
  const int arow = m0 + 16 * wave + r;
  const uint32_t abase = (arow < P.M ? 0u : OOB) + (uint32_t)arow * P.lda2 + 16 * g;
  gu4 ring[SK_RING];
  auto request = [&](int s) -> gu4 {
    return __builtin_amdgcn_raw_buffer_load_b128(rA, abase + (s < ns ? (uint32_t)s * 64 : OOB), 0, 0);
  };
#pragma unroll
  for (int d = 0; d < SK_RING; d++) ring[d] = request(d);

  // ---- park the strip in LDS (waits for the strip only: it was requested first, and loads complete in order)
#pragma unroll
  for (int p = 0; p < SK_WPASS; p++) {
    const int seg = wseg0 + SPP * p;
    if (p < passes && seg < segs) *(gu4*)(wlds + wrow * pitch + seg * 128 + 16 * wch) = wst[p];
  }
  __syncthreads();

  gf4 acc[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) acc[j] = gf4{0.f, 0.f, 0.f, 0.f};
  const unsigned char* wop = wlds + r * pitch + 16 * g;  // operand read: row r of a 16-row slab, 16 bytes at k = 8 g
  float ss = 0.f;  // NORM: sum of squares of this lane's quarter of row r
  auto step = [&](int s, gu4& slot) {
    gu4 w[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) w[j] = *(const gu4*)(wop + 16 * j * pitch + s * 64);
#pragma unroll
    for (int j = 0; j < TN; j++) acc[j] = gmfma<DT>(w[j], slot, acc[j]);
    if (NORM) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float lo, hi;
        if (DT == UVMI_BF16) { lo = __uint_as_float(slot[i] << 16); hi = __uint_as_float(slot[i] & 0xffff0000u); }
        else { lo = half_bits_to_float((uint16_t)(slot[i] & 0xffff)); hi = half_bits_to_float((uint16_t)(slot[i] >> 16)); }
        ss = fmaf(lo, lo, ss);
        ss = fmaf(hi, hi, ss);
      }
    }
    slot = request(s + SK_RING);
  };
  // whole turns of the ring run in a loop whose body has no branches, which keeps the wait before a step at "all but the
  // later steps' loads"; the last ns % SK_RING steps follow outside the loop
  int s = 0;
  for (; s + SK_RING <= ns; s += SK_RING) {
#pragma unroll
    for (int d = 0; d < SK_RING; d++) step(s + d, ring[d]);
  }
#pragma unroll
  for (int d = 0; d < SK_RING - 1; d++)
    if (s + d < ns) step(s + d, ring[d]);  // workgroup-uniform

  // accumulator j: lane (r, g) holds C[m0 + 16 wave + r][n0 + 16 j + 4 g + t], t = 0..3: the same row r whose quarter the
  // lane summed, so the row scale needs the 4 lane groups' sums and nothing else
  if (NORM) {
    ss = gxsum32(gxsum16(ss));
    const float rn = rsqrtf(ss / (float)P.K + a_eps);
#pragma unroll
    for (int j = 0; j < TN; j++) acc[j] *= rn;
  }
  if (arow >= P.M) return;
  if (EPI == 2) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int n = n0 + 16 * j;
      if (n >= P.N) continue;
      const gf4 v = acc[j];
      const uint2 rw = *(const uint2*)((const uint16_t*)a_res + (int64_t)arow * a_ldr + n + 4 * g);
      float x[4], o[4];
      if (DT == UVMI_BF16) {
        x[0] = __uint_as_float(rw.x << 16); x[1] = __uint_as_float(rw.x & 0xffff0000u);
        x[2] = __uint_as_float(rw.y << 16); x[3] = __uint_as_float(rw.y & 0xffff0000u);
      } else {
        x[0] = half_bits_to_float((uint16_t)(rw.x & 0xffff)); x[1] = half_bits_to_float((uint16_t)(rw.x >> 16));
        x[2] = half_bits_to_float((uint16_t)(rw.y & 0xffff)); x[3] = half_bits_to_float((uint16_t)(rw.y >> 16));
      }
#pragma unroll
      for (int t = 0; t < 4; t++) o[t] = a_ca * x[t] + a_cb * ground<DT>(v[t]);
      uint16_t* cp = (uint16_t*)P.c + (int64_t)arow * P.ldc + n + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
    }
  } else if (EPI == 0) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int n = n0 + 16 * j;
      if (n >= P.N) continue;
      const gf4 v = acc[j];
      uint16_t* cp = (uint16_t*)P.c + (int64_t)arow * P.ldc + n + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(v[0], v[1]), gpack<DT>(v[2], v[3])};
    }
  } else {
    static_assert(EPI != 1 || BN == 32, "the SwiGLU epilogue pairs two 16-row slabs");
    if (n0 < P.N) {
      const gf4 gt = acc[0], up = acc[TN - 1];
      float o[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const float gv = ground<DT>(gt[t]), uv = ground<DT>(up[t]);
        o[t] = silu_round<DT>(gv) * uv;
      }
      uint16_t* cp = (uint16_t*)P.c + (int64_t)arow * P.ldc + (n0 >> 1) + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
    }
  }
}


// The same product for the smallest steps, where a 64-row workgroup would leave most compute units idle and every wave
// would walk all of K: a workgroup owns 16 rows x BN columns and its 4 waves split K in quarters.  Each wave requests its
// quarter of the weight strip (4 consecutive lanes on 64 bytes of a weight row) and of the 16 activation rows in one
// burst, parks its own strip quarter in its own LDS region (no workgroup barrier before the loop), multiplies, and the four
// partial accumulators (and, with NORM, partial sums of squares) meet in LDS, where the first wave adds them and runs the
// epilogue.  K % 128 == 0, K / 4 <= 512.
template <int DT, int BN, int EPI, bool NORM>
__global__ __launch_bounds__(256) void gemm_skinny_ksplit_kernel(const void* a_a, const void* a_w, void* a_c, uint32_t a_lda2, uint32_t a_ldw2,
                                                                 int a_M, int a_N, int a_K, int a_tiles_m, int a_tiles_n, int64_t a_ldc,
                                                                 float a_eps, const void* a_res, int64_t a_ldr, float a_ca, float a_cb) {
  extern __shared__ __attribute__((aligned(16))) unsigned char wlds[];  // 4 x [BN rows of K / 2 + 16 bytes], then the partials
  constexpr int TN = BN / 16;
  constexpr int RP = BN / 16;                 // row passes of the strip load (16 rows per pass)
  constexpr int MAXCP = 16 / RP;              // most chunk passes (4 chunks of 16 bytes per pass)
  constexpr int MAXS = 16;                    // most K-steps per wave
  constexpr uint32_t OOB = 0x40000000u;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int T = a_tiles_m * a_tiles_n;
  const int per = (T + 7) / 8;
  const int L = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
  if (L >= T) return;
  const int bn = L / a_tiles_m, bm = L % a_tiles_m;
  const int m0 = bm * 16, n0 = bn * BN;
  const int r = lane & 15, g = lane >> 4;
  const int nsw = a_K / 128;                  // K-steps (of 32) per wave
  const int kq2 = a_K / 2;                    // bytes of a row's K quarter
  const uint32_t pitch = (uint32_t)kq2 + 16;
  const int cps = kq2 / 64;                   // chunk passes: 64 bytes (4 lanes) of a weight row per pass
  const uint32_t kbase = (uint32_t)wave * (uint32_t)kq2;  // byte offset of this wave's quarter inside a row

  const uint32_t boundA = (uint32_t)(a_M - 1) * a_lda2 + (uint32_t)a_K * 2;
  const uint32_t boundW = (uint32_t)(a_N - 1) * a_ldw2 + (uint32_t)a_K * 2;
  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc((void*)a_a, 0, (int)boundA, 0x00020000);
  const __amdgpu_buffer_rsrc_t rW = __builtin_amdgcn_make_buffer_rsrc((void*)a_w, 0, (int)boundW, 0x00020000);

  // ---- this wave's quarter of the weight strip: lane -> row (lane / 4) + 16 j, bytes 16 (lane % 4) + 64 i of the quarter
  const int wr = lane >> 2, wc = lane & 3;
  gu4 wst[RP][MAXCP];
#pragma unroll
  for (int j = 0; j < RP; j++) {
    const int row = n0 + wr + 16 * j;
    const uint32_t base = (row < a_N ? 0u : OOB) + (uint32_t)row * a_ldw2 + kbase + 16 * wc;
#pragma unroll
    for (int i = 0; i < MAXCP; i++) wst[j][i] = __builtin_amdgcn_raw_buffer_load_b128(rW, base + (i < cps ? (uint32_t)i * 64 : OOB), 0, 0);
  }
  // ---- this wave's quarter of the 16 activation rows, in MFMA operand order: lane (r, g) = row r, k = 32 s + 8 g ..
  const int arow = m0 + r;
  const uint32_t abase = (arow < a_M ? 0u : OOB) + (uint32_t)arow * a_lda2 + kbase + 16 * g;
  gu4 av[MAXS];
#pragma unroll
  for (int s = 0; s < MAXS; s++) av[s] = __builtin_amdgcn_raw_buffer_load_b128(rA, abase + (s < nsw ? (uint32_t)s * 64 : OOB), 0, 0);

  unsigned char* mine = wlds + (size_t)wave * BN * pitch;
#pragma unroll
  for (int j = 0; j < RP; j++)
#pragma unroll
    for (int i = 0; i < MAXCP; i++)
      if (i < cps) *(gu4*)(mine + (wr + 16 * j) * pitch + 64 * i + 16 * wc) = wst[j][i];
  __builtin_amdgcn_wave_barrier();  // the region is this wave's own: its LDS operations complete in order

  gf4 acc[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) acc[j] = gf4{0.f, 0.f, 0.f, 0.f};
  float ss = 0.f;
  const unsigned char* wop = mine + r * pitch + 16 * g;
#pragma unroll
  for (int s = 0; s < MAXS; s++) {
    if (s < nsw) {  // workgroup-uniform
      gu4 w[TN];
#pragma unroll
      for (int j = 0; j < TN; j++) w[j] = *(const gu4*)(wop + 16 * j * pitch + s * 64);
#pragma unroll
      for (int j = 0; j < TN; j++) acc[j] = gmfma<DT>(w[j], av[s], acc[j]);
      if (NORM) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float lo, hi;
          if (DT == UVMI_BF16) { lo = __uint_as_float(av[s][i] << 16); hi = __uint_as_float(av[s][i] & 0xffff0000u); }
          else { lo = half_bits_to_float((uint16_t)(av[s][i] & 0xffff)); hi = half_bits_to_float((uint16_t)(av[s][i] >> 16)); }
          ss = fmaf(lo, lo, ss);
          ss = fmaf(hi, hi, ss);
        }
      }
    }
  }
  // ---- the four partial results meet in LDS; the first wave adds them (in wave order) and finishes
  float* red = (float*)(wlds + (size_t)4 * BN * pitch);   // [4 waves][TN * 4 + 1][64 lanes]
  constexpr int RW = TN * 4 + 1;
#pragma unroll
  for (int j = 0; j < TN; j++)
#pragma unroll
    for (int t = 0; t < 4; t++) red[(wave * RW + j * 4 + t) * 64 + lane] = acc[j][t];
  if (NORM) red[(wave * RW + TN * 4) * 64 + lane] = ss;
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < 4; w++) {
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int t = 0; t < 4; t++) acc[j][t] += red[(w * RW + j * 4 + t) * 64 + lane];
    if (NORM) ss += red[(w * RW + TN * 4) * 64 + lane];
  }
  if (NORM) {
    ss = gxsum32(gxsum16(ss));
    const float rn = rsqrtf(ss / (float)a_K + a_eps);
#pragma unroll
    for (int j = 0; j < TN; j++) acc[j] *= rn;
  }
  if (arow >= a_M) return;
  if (EPI == 2) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int n = n0 + 16 * j;
      if (n >= a_N) continue;
      const gf4 v = acc[j];
      const uint2 rw = *(const uint2*)((const uint16_t*)a_res + (int64_t)arow * a_ldr + n + 4 * g);
      float x[4], o[4];
      if (DT == UVMI_BF16) {
        x[0] = __uint_as_float(rw.x << 16); x[1] = __uint_as_float(rw.x & 0xffff0000u);
        x[2] = __uint_as_float(rw.y << 16); x[3] = __uint_as_float(rw.y & 0xffff0000u);
      } else {
        x[0] = half_bits_to_float((uint16_t)(rw.x & 0xffff)); x[1] = half_bits_to_float((uint16_t)(rw.x >> 16));
        x[2] = half_bits_to_float((uint16_t)(rw.y & 0xffff)); x[3] = half_bits_to_float((uint16_t)(rw.y >> 16));
      }
#pragma unroll
      for (int t = 0; t < 4; t++) o[t] = a_ca * x[t] + a_cb * ground<DT>(v[t]);
      uint16_t* cp = (uint16_t*)a_c + (int64_t)arow * a_ldc + n + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
    }
  } else if (EPI == 0) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int n = n0 + 16 * j;
      if (n >= a_N) continue;
      const gf4 v = acc[j];
      uint16_t* cp = (uint16_t*)a_c + (int64_t)arow * a_ldc + n + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(v[0], v[1]), gpack<DT>(v[2], v[3])};
    }
  } else {
    static_assert(EPI != 1 || BN == 32, "the SwiGLU epilogue pairs two 16-row slabs");
    if (n0 < a_N) {
      const gf4 gt = acc[0], up = acc[TN - 1];
      float o[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const float gv = ground<DT>(gt[t]), uv = ground<DT>(up[t]);
        o[t] = silu_round<DT>(gv) * uv;
      }
      uint16_t* cp = (uint16_t*)a_c + (int64_t)arow * a_ldc + (n0 >> 1) + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
    }
  }
}

}  // namespace uvmi

using namespace uvmi;

namespace uvmi {
void gemm_tile_launch(const uvmi_gemm_args* a, bool big, hipStream_t st);  // gemm_tile.hip
void gemm_big_launch(const uvmi_gemm_args* a, int tile, hipStream_t st);   // gemm_big.hip
}

// Rows from which the tiled kernel takes over from the skinny forms when config == 0 (measured on UV-50M's projections):
// 448 for the narrow projections (N ~ 640: fewer rows give the 64 x 64 grid too few tiles); the wide gate-up projection with
// its SwiGLU epilogue already from 128 rows (2 x 52 tiles: 6.8 us at 128 - 256 rows and 9.0 us at 384, where the 64-row
// skinny form takes 7.6 - 10.5 and 15.4 us).
constexpr int64_t TILE_MIN_ROWS = 448, TILE_MIN_ROWS_SWIGLU = 128;
// Rows from which the 256 x 256 tile of gemm_big.hip takes over (one workgroup per compute unit: it needs several rounds of
// tiles to pay; measured on UV-50M's projections at 2 k - 33 k rows: from ~12 k rows it is the fastest form for every
// projection, for the wide gate-up projection with its SwiGLU epilogue already from 4 k).
constexpr int64_t BIG_MIN_ROWS = 12288, BIG_MIN_ROWS_SWIGLU = 4096;

// what the 256 x 256 kernel assumes beyond uvmi_gemm_tn_supported: two slabs at least, 16-byte stores and residual loads
static bool big_ok(const uvmi_gemm_args* a) {
  if (a->K < 128 || ((uintptr_t)a->c % 16) != 0 || a->ldc % 8 != 0) return false;
  if (a->epilogue == UVMI_GEMM_RESID && (((uintptr_t)a->resid % 16) != 0 || a->ldr % 8 != 0)) return false;
  return true;
}

static int skinny_bn(int K, int epilogue) {  // widest strip that fits 64 KB of LDS: 32 rows up to K = 960, else 16
  if (epilogue == UVMI_GEMM_SWIGLU) return K <= 960 ? 32 : 0;
  if (K <= 960) return 32;
  return K <= 1984 ? 16 : 0;
}

extern "C" int uvmi_gemm_tn_supported(int dtype, int64_t M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int epilogue) {
  if (dtype != UVMI_F16 && dtype != UVMI_BF16) return 0;
  if (epilogue != UVMI_GEMM_STORE && epilogue != UVMI_GEMM_SWIGLU && epilogue != UVMI_GEMM_RESID) return 0;
  if (M < 0 || M > (1 << 16) || N <= 0 || K <= 0 || K % 64 != 0 || K > 8192) return 0;  // (the skinny forms add K <= 1984 / 960)
  if (N % (epilogue == UVMI_GEMM_SWIGLU ? 32 : 16) != 0) return 0;
  if (lda < K || ldw < K || lda % 8 != 0 || ldw % 8 != 0 || ldc % 4 != 0) return 0;
  if (ldc < (epilogue == UVMI_GEMM_SWIGLU ? N / 2 : N)) return 0;
  if ((M + 64) * lda * 2 >= (1LL << 30) || ((int64_t)N + 64) * ldw * 2 >= (1LL << 30)) return 0;  // 32-bit offsets with room for the out-of-range mark
  return 1;
}

template <int DT, int BN>
static void launch_skinny(const uvmi_gemm_args* a, const SkinnyParams& P, dim3 grid, size_t lds, hipStream_t st, bool ksplit) {
  const dim3 blk(256);
#define UVMI_GO(EPI, NORM)                                                                                                             \
  do {                                                                                                                                 \
    if (ksplit)                                                                                                                        \
      hipLaunchKernelGGL((gemm_skinny_ksplit_kernel<DT, BN, EPI, NORM>), grid, blk, lds, st, P.a, P.w, P.c, P.lda2, P.ldw2, P.M, P.N,  \
                         P.K, P.tiles_m, P.tiles_n, P.ldc, a->eps, a->resid, a->ldr, a->ca, a->cb);                                    \
    else                                                                                                                               \
      hipLaunchKernelGGL((gemm_skinny_kernel<DT, BN, EPI, NORM>), grid, blk, lds, st, P.a, P.w, P.c, P.lda2, P.ldw2, P.M, P.N, P.K,    \
                         P.tiles_m, P.tiles_n, P.ldc, a->eps, a->resid, a->ldr, a->ca, a->cb);                                         \
  } while (0)
  const bool norm = a->norm_a != 0;
  if (a->epilogue == UVMI_GEMM_RESID) { if (norm) UVMI_GO(2, true); else UVMI_GO(2, false); }
  else if (a->epilogue == UVMI_GEMM_SWIGLU) {
    if constexpr (BN == 32) { if (norm) UVMI_GO(1, true); else UVMI_GO(1, false); }
  } else { if (norm) UVMI_GO(0, true); else UVMI_GO(0, false); }
#undef UVMI_GO
}

extern "C" int uvmi_gemm_tn_ex(const uvmi_gemm_args* a, void* stream) {
  UVMI_REQUIRE(a && a->a && a->w && a->c, UVMI_EINVAL, "uvmi_gemm_tn: null pointer");
  UVMI_REQUIRE(uvmi_gemm_tn_supported(a->dtype, a->M, a->N, a->K, a->lda, a->ldw, a->ldc, a->epilogue), UVMI_EUNSUPPORTED,
               "uvmi_gemm_tn: unsupported problem (dtype %d, M %lld, N %d, K %d, lda %lld, ldw %lld, ldc %lld, epilogue %d): needs F16 / BF16, "
               "K %% 64 == 0, N %% 16 == 0 (32 with SWIGLU), lda, ldw %% 8 == 0, ldc %% 4 == 0",
               a->dtype, (long long)a->M, a->N, a->K, (long long)a->lda, (long long)a->ldw, (long long)a->ldc, a->epilogue);
  UVMI_REQUIRE(((uintptr_t)a->a % 16) == 0 && ((uintptr_t)a->w % 16) == 0 && ((uintptr_t)a->c % 8) == 0, UVMI_EINVAL, "uvmi_gemm_tn: misaligned pointer");
  if (a->epilogue == UVMI_GEMM_RESID)
    UVMI_REQUIRE(a->resid && ((uintptr_t)a->resid % 8) == 0 && a->ldr % 4 == 0 && a->ldr >= a->N, UVMI_EINVAL,
                 "uvmi_gemm_tn: the RESID epilogue needs an 8-byte aligned residual with a pitch that is a multiple of 4 and >= N");
  UVMI_REQUIRE(!a->norm_a || a->eps >= 0.f, UVMI_EINVAL, "uvmi_gemm_tn: negative eps");
  UVMI_REQUIRE(a->config >= 0 && a->config <= 6, UVMI_EINVAL, "uvmi_gemm_tn: config %d", a->config);
  if (a->M == 0) return UVMI_OK;
  const int BN = skinny_bn(a->K, a->epilogue);
  UVMI_REQUIRE(BN != 0 || a->config == 0 || a->config >= 3, UVMI_EUNSUPPORTED, "uvmi_gemm_tn: K = %d is beyond the skinny forms (config 1, 2)", a->K);
  // (also a product of fewer rows whose 256 x 256 tiles still come to two rounds of the device or more - the tied head,
  // 2048 x 32768: 104 us against 129 us on 128 x 128 tiles)
  int cus_big = uvmi_device_cus();
  if (cus_big <= 0) cus_big = 256;
  const bool many_big_tiles = a->M >= 1024 && ((a->M + 255) / 256) * (((int64_t)a->N + 255) / 256) >= 2 * (int64_t)cus_big;
  if (a->config == 5 || (a->config == 0 && (many_big_tiles || a->M >= (a->epilogue == UVMI_GEMM_SWIGLU ? BIG_MIN_ROWS_SWIGLU : BIG_MIN_ROWS)) && big_ok(a))) {
    UVMI_REQUIRE(big_ok(a), UVMI_EUNSUPPORTED,
                 "uvmi_gemm_tn: config 5 (256 x 256 tiles) needs K >= 128, C (and the residual) 16-byte aligned, ldc (ldr) %% 8 == 0");
    // An output whose width fills 128-wide tiles much better than 256-wide ones (N = 640: 5 tiles of 128 against 3 of 256, a
    // sixth of which would be computed for nothing) runs on the 128 x 128 form of the same kernel (measured at 33 216 rows:
    // the output projection 37.5 us against 40.8, the down projection 79.8 against 84.8).
    const int64_t pad128 = ((int64_t)a->N + 127) / 128 * 128, pad256 = ((int64_t)a->N + 255) / 256 * 256;
    const int tile = a->config == 0 && pad128 * 10 < pad256 * 9 ? 128 : 256;
    gemm_big_launch(a, tile, (hipStream_t)stream);
    UVMI_CHECK_LAUNCH("uvmi_gemm_tn(direct to LDS)");
    return UVMI_OK;
  }
  if (a->config == 6) {
    UVMI_REQUIRE(big_ok(a), UVMI_EUNSUPPORTED,
                 "uvmi_gemm_tn: config %d (tiles loaded straight into LDS) needs K >= 128, C (and the residual) 16-byte aligned, ldc (ldr) %% 8 == 0", a->config);
    gemm_big_launch(a, 128, (hipStream_t)stream);
    UVMI_CHECK_LAUNCH("uvmi_gemm_tn(128 x 128, direct)");
    return UVMI_OK;
  }
  const int64_t tile_min_rows = a->epilogue == UVMI_GEMM_SWIGLU && a->N >= 2048 ? TILE_MIN_ROWS_SWIGLU : TILE_MIN_ROWS;
  if (a->config >= 3 || (a->config == 0 && (BN == 0 || a->M >= tile_min_rows))) {
    // tiled kernel: 128 x 128 tiles when there are enough of them for 3/5 of the compute units, else 64 x 64
    int cus = uvmi_device_cus();
    if (cus <= 0) cus = 256;
    const int64_t t128 = ((a->M + 127) / 128) * ((a->N + 127) / 128);
    const bool big = a->config == 3 || (a->config == 0 && 5 * t128 >= 3 * cus);   // (measured crossover: gate-up at ~640 rows)
    if (big && a->config == 0 && big_ok(a)) {   // the 128 x 128 tile in its direct-to-LDS form (gemm_big.hip): faster wherever it applies
      gemm_big_launch(a, 128, (hipStream_t)stream);
      UVMI_CHECK_LAUNCH("uvmi_gemm_tn(128 x 128, direct)");
      return UVMI_OK;
    }
    gemm_tile_launch(a, big, (hipStream_t)stream);
    UVMI_CHECK_LAUNCH("uvmi_gemm_tn(tiled)");
    return UVMI_OK;
  }
  // the smallest problems split K over the waves of a 16-row workgroup (more, shorter workgroups); config forces a form
  const bool can_split = a->K % 128 == 0;
  const int64_t t_split = ((a->M + 15) / 16) * ((a->N + BN - 1) / BN);
  const bool ksplit = a->config == 2 ? can_split : (a->config == 1 ? false : (can_split && t_split <= SK_KSPLIT_TILES));
  SkinnyParams P;
  P.a = a->a; P.w = a->w; P.c = a->c; P.lda2 = (uint32_t)a->lda * 2; P.ldw2 = (uint32_t)a->ldw * 2; P.ldc = a->ldc;
  P.M = (int)a->M; P.N = a->N; P.K = a->K;
  const int bm = ksplit ? 16 : SK_BM;
  P.tiles_m = (int)((a->M + bm - 1) / bm);
  P.tiles_n = (a->N + BN - 1) / BN;
  const int T = P.tiles_m * P.tiles_n;
  const dim3 grid((unsigned)(((T + 7) / 8) * 8));
  // one strip: at most 32 * 1936 = 62 KB, 16 * 3984 = 64 KB; split: the strip in four regions with their own padding + 9 KB
  const size_t lds = ksplit ? (size_t)4 * BN * ((size_t)a->K / 2 + 16) + (size_t)4 * (BN / 16 * 4 + 1) * 256
                            : (size_t)BN * ((size_t)a->K * 2 + 16);
  hipStream_t st = (hipStream_t)stream;
  if (a->dtype == UVMI_F16) { if (BN == 32) launch_skinny<UVMI_F16, 32>(a, P, grid, lds, st, ksplit); else launch_skinny<UVMI_F16, 16>(a, P, grid, lds, st, ksplit); }
  else { if (BN == 32) launch_skinny<UVMI_BF16, 32>(a, P, grid, lds, st, ksplit); else launch_skinny<UVMI_BF16, 16>(a, P, grid, lds, st, ksplit); }
  UVMI_CHECK_LAUNCH("uvmi_gemm_tn");
  return UVMI_OK;
}

extern "C" int uvmi_gemm_tn(const void* a, const void* w, void* c, int dtype, int64_t M, int N, int K, int64_t lda, int64_t ldw,
                            int64_t ldc, int epilogue, void* stream) {
  uvmi_gemm_args g = {};
  g.a = a; g.w = w; g.c = c; g.dtype = dtype; g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldw = ldw; g.ldc = ldc; g.epilogue = epilogue;
  UVMI_REQUIRE(epilogue != UVMI_GEMM_RESID, UVMI_EINVAL, "uvmi_gemm_tn: the RESID epilogue takes its residual through uvmi_gemm_tn_ex");
  return uvmi_gemm_tn_ex(&g, stream);
}
