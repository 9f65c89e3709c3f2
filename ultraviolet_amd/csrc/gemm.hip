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
//     of the separate SwiGLU pass (g, u and silu(g) rounded to the activation type): the (M, 2f) intermediate never exists.
#include "common.h"

namespace uvmi {

typedef _Float16 gh8 __attribute__((ext_vector_type(8)));
typedef __bf16 gb8 __attribute__((ext_vector_type(8)));
typedef float gf4 __attribute__((ext_vector_type(4)));
typedef unsigned int gu4 __attribute__((ext_vector_type(4)));

struct SkinnyParams {
  const void* a; const void* w; void* c;
  uint32_t lda2, ldw2;  // row pitches in bytes
  int64_t ldc;          // elements
  int M, N, K;
  int tiles_m, tiles_n;
};

template <int DT>
__device__ __forceinline__ gf4 gmfma(gu4 a, gu4 b, gf4 c) {
  if constexpr (DT == UVMI_F16) {
    gh8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, c, 0, 0, 0);
  } else {
    gb8 x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, c, 0, 0, 0);
  }
}

template <int DT> __device__ __forceinline__ float ground(float v) {
  if constexpr (DT == UVMI_F16) return (float)(half_t)v;
  else return bf16_to_float(float_to_bf16(v));
}
template <int DT> __device__ __forceinline__ uint32_t gpack(float a, float b) {
  const uint32_t lo = DT == UVMI_BF16 ? float_to_bf16(a) : float_to_half_bits(a);
  const uint32_t hi = DT == UVMI_BF16 ? float_to_bf16(b) : float_to_half_bits(b);
  return lo | (hi << 16);
}

constexpr int SK_BM = 64;       // rows per workgroup
constexpr int SK_RING = 16;     // activation K-steps (of 32) in flight per wave
constexpr int SK_WPASS = 16;    // most passes of the weight-strip load (32 (row, 128-byte segment) units per pass)

// EPI 0: C = A W^T (M, N).  EPI 1 (BN = 32): W rows are [gate 16 | up 16] slabs; C = silu(gate) * up, (M, N / 2).
// (individual scalar arguments rather than a parameter block: they are preloaded into SGPRs with the wave, so the first
// loads need not wait for a load of the kernel arguments)
template <int DT, int BN, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const void* a_a, const void* a_w, void* a_c, uint32_t a_lda2, uint32_t a_ldw2,
                                                          int a_M, int a_N, int a_K, int a_tiles_m, int a_tiles_n, int64_t a_ldc) {
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
  auto step = [&](int s, gu4& slot) {
    gu4 w[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) w[j] = *(const gu4*)(wop + 16 * j * pitch + s * 64);
#pragma unroll
    for (int j = 0; j < TN; j++) acc[j] = gmfma<DT>(w[j], slot, acc[j]);
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

  // accumulator j: lane (r, g) holds C[m0 + 16 wave + r][n0 + 16 j + 4 g + t], t = 0..3
  if (arow >= P.M) return;
  if (EPI == 0) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int n = n0 + 16 * j;
      if (n >= P.N) continue;
      const gf4 v = acc[j];
      uint16_t* cp = (uint16_t*)P.c + (int64_t)arow * P.ldc + n + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(v[0], v[1]), gpack<DT>(v[2], v[3])};
    }
  } else {
    static_assert(EPI == 0 || BN == 32, "the SwiGLU epilogue pairs two 16-row slabs");
    if (n0 < P.N) {
      const gf4 gt = acc[0], up = acc[TN - 1];
      float o[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const float gv = ground<DT>(gt[t]), uv = ground<DT>(up[t]);
        o[t] = ground<DT>(gv / (1.0f + __expf(-gv))) * uv;
      }
      uint16_t* cp = (uint16_t*)P.c + (int64_t)arow * P.ldc + (n0 >> 1) + 4 * g;
      *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
    }
  }
}

}  // namespace uvmi

using namespace uvmi;

static int skinny_bn(int K, int epilogue) {  // widest strip that fits 64 KB of LDS: 32 rows up to K = 960, else 16
  if (epilogue == UVMI_GEMM_SWIGLU) return K <= 960 ? 32 : 0;
  if (K <= 960) return 32;
  return K <= 1984 ? 16 : 0;
}

extern "C" int uvmi_gemm_tn_supported(int dtype, int64_t M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int epilogue) {
  if (dtype != UVMI_F16 && dtype != UVMI_BF16) return 0;
  if (epilogue != UVMI_GEMM_STORE && epilogue != UVMI_GEMM_SWIGLU) return 0;
  if (M < 0 || M > (1 << 16) || N <= 0 || K <= 0 || K % 64 != 0 || skinny_bn(K, epilogue) == 0) return 0;
  if (N % (epilogue == UVMI_GEMM_SWIGLU ? 32 : 16) != 0) return 0;
  if (lda < K || ldw < K || lda % 8 != 0 || ldw % 8 != 0 || ldc % 4 != 0) return 0;
  if (ldc < (epilogue == UVMI_GEMM_SWIGLU ? N / 2 : N)) return 0;
  if ((M + 64) * lda * 2 >= (1LL << 30) || ((int64_t)N + 64) * ldw * 2 >= (1LL << 30)) return 0;  // 32-bit offsets with room for the out-of-range mark
  return 1;
}

extern "C" int uvmi_gemm_tn(const void* a, const void* w, void* c, int dtype, int64_t M, int N, int K, int64_t lda, int64_t ldw,
                            int64_t ldc, int epilogue, void* stream) {
  UVMI_REQUIRE(a && w && c, UVMI_EINVAL, "uvmi_gemm_tn: null pointer");
  UVMI_REQUIRE(uvmi_gemm_tn_supported(dtype, M, N, K, lda, ldw, ldc, epilogue), UVMI_EUNSUPPORTED,
               "uvmi_gemm_tn: unsupported problem (dtype %d, M %lld, N %d, K %d, lda %lld, ldw %lld, ldc %lld, epilogue %d): needs F16 / BF16, "
               "K %% 64 == 0, K <= 1984 (960 with SWIGLU), N %% 16 == 0 (32 with SWIGLU), lda, ldw %% 8 == 0, ldc %% 4 == 0",
               dtype, (long long)M, N, K, (long long)lda, (long long)ldw, (long long)ldc, epilogue);
  UVMI_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)c % 8) == 0, UVMI_EINVAL, "uvmi_gemm_tn: misaligned pointer");
  if (M == 0) return UVMI_OK;
  const int BN = skinny_bn(K, epilogue);
  SkinnyParams P;
  P.a = a; P.w = w; P.c = c; P.lda2 = (uint32_t)lda * 2; P.ldw2 = (uint32_t)ldw * 2; P.ldc = ldc; P.M = (int)M; P.N = N; P.K = K;
  P.tiles_m = (int)((M + SK_BM - 1) / SK_BM);
  P.tiles_n = (N + BN - 1) / BN;
  const int T = P.tiles_m * P.tiles_n;
  const dim3 grid((unsigned)(((T + 7) / 8) * 8)), blk(256);
  const size_t lds = (size_t)BN * ((size_t)K * 2 + 16);  // at most 32 * 1936 = 62 KB, 16 * 3984 = 64 KB
  hipStream_t st = (hipStream_t)stream;
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, grid, blk, lds, st, P.a, P.w, P.c, P.lda2, P.ldw2, P.M, P.N, P.K, P.tiles_m, P.tiles_n, P.ldc);
  };
  if (dtype == UVMI_F16) {
    if (epilogue == UVMI_GEMM_SWIGLU) go(gemm_skinny_kernel<UVMI_F16, 32, 1>);
    else if (BN == 32) go(gemm_skinny_kernel<UVMI_F16, 32, 0>);
    else go(gemm_skinny_kernel<UVMI_F16, 16, 0>);
  } else {
    if (epilogue == UVMI_GEMM_SWIGLU) go(gemm_skinny_kernel<UVMI_BF16, 32, 1>);
    else if (BN == 32) go(gemm_skinny_kernel<UVMI_BF16, 32, 0>);
    else go(gemm_skinny_kernel<UVMI_BF16, 16, 0>);
  }
  UVMI_CHECK_LAUNCH("uvmi_gemm_tn");
  return UVMI_OK;
}
