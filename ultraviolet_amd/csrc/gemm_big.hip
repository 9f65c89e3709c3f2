// 16-bit GEMM for passes of many thousand rows (a packed prefill, a mixed prefill + decode pass): the same product and
// epilogues as the tiled kernel of gemm_tile.hip - C[M, N] = A[M, K] . W[N, K]^T with fp32 accumulation, SwiGLU on
// interleaved gate / up slabs, the block's residual update, the RMS pre-norm as a row scale (the F.linear calls of the
// reference's fused inference path, ultraviolet/model.py:302-335, 388-391, with what surrounds them, :566-571) - on a
// 256 x 256 tile.
//
// What bounds a GEMM of this size on gfx950 is not the matrix cores but what feeds them.  Measured on the part: a compute
// unit takes ~52 bytes per clock from the L2 when every request is a whole 128-byte line and half of that when requests
// are 64-byte row segments, and its LDS delivers ~128 bytes per clock.  Hence:
//   * a workgroup of 8 waves (2 x 4) owns a 256 x 256 tile, a wave 128 x 64 of it: per K-step of 32 a wave reads 12 operand
//     fragments from LDS for 32 MFMAs (the 64 x 64 wave tile of the smaller kernels reads 8 for 16), and the tile takes
//     half the L2 bytes per flop of a 128 x 128 tile;
//   * K is walked in slabs of 64: a row's share of a slab is one whole 128-byte line;
//   * slabs go from global memory straight into LDS (global_load_lds, 16 bytes per lane): no staging registers, no LDS
//     store instructions.  A wave-load lands as 1 KB of consecutive LDS - 8 rows of 128 bytes - so the xor swizzle that
//     keeps the operand reads conflict-free (16-byte chunk index ^ (row / 2) % 8) is applied on the global side: lane l
//     of a load fetches the chunk that belongs at physical position l % 8 of its row;
//   * two LDS stages of 64 KB (A and W slab each 256 rows x 128 B).  An iteration multiplies slab k out of one stage while
//     slab k + 1 lands in the other; its operand reads run one MFMA group (8 MFMAs) ahead of their use, and before its
//     last group it waits for slab k + 1, refills its own stage with slab k + 2 and requests slab k + 1's first operands:
//     one barrier per slab, no bubble between slabs;
//   * the accumulator holds C^T fragments (a lane has 4 consecutive columns of one row); the epilogue converts, transposes
//     4 x 4 across the lane groups with permlane swaps, and each lane stores 16 consecutive columns - whole 128-byte lines
//     per row instead of 8-byte pieces;
//   * tiles are dealt to the XCDs in contiguous runs, as in the tiled kernel.
// One workgroup per compute unit (128 KB of LDS, 2 waves per SIMD).  K >= 128; C and the residual 16-byte aligned with
// pitches that are multiples of 8 elements (the caller checks).
#include "common.h"
#include "gemm_util.h"

namespace uvmi {

struct BigParams {
  const void* a; const void* w; void* c; const void* r;
  uint32_t lda2, ldw2;  // row pitches in bytes
  int64_t ldc, ldr;     // elements
  int M, N, K, tiles_m, tiles_n;
  int rowsplit;
  float eps, ca, cb;
};

#define UVMI_LDSP(p) ((__attribute__((address_space(3))) void*)(p))
#define UVMI_GLBP(p) ((const __attribute__((address_space(1))) void*)(p))

// 4 x 4 transpose of one dword per (register j, lane group g = lane / 16): afterwards register j of group g holds what
// register g of group j held.  (permlane32_swap exchanges the upper 32 lanes of its first operand with the lower 32 of its
// second, permlane16_swap does the same inside each half.)
__device__ __forceinline__ void xpose4(uint32_t (&x)[4]) {
  auto s0 = __builtin_amdgcn_permlane32_swap(x[0], x[2], false, false);
  auto s1 = __builtin_amdgcn_permlane32_swap(x[1], x[3], false, false);
  x[0] = s0[0]; x[2] = s0[1]; x[1] = s1[0]; x[3] = s1[1];
  auto t0 = __builtin_amdgcn_permlane16_swap(x[0], x[1], false, false);
  auto t1 = __builtin_amdgcn_permlane16_swap(x[2], x[3], false, false);
  x[0] = t0[0]; x[1] = t0[1]; x[2] = t1[0]; x[3] = t1[1];
}
// 2 x 2 transpose between (register j, lane / 16 % 2)
__device__ __forceinline__ void xpose2(uint32_t& x0, uint32_t& x1) {
  auto t = __builtin_amdgcn_permlane16_swap(x0, x1, false, false);
  x0 = t[0]; x1 = t[1];
}
template <int DT> __device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi) {
  if (DT == UVMI_BF16) { lo = __uint_as_float(w << 16); hi = __uint_as_float(w & 0xffff0000u); }
  else { lo = half_bits_to_float((uint16_t)(w & 0xffff)); hi = half_bits_to_float((uint16_t)(w >> 16)); }
}

// EPI 0: C = A W^T (M, N).  EPI 1: W rows are [gate 16 | up 16] slabs; C = silu(gate) * up, (M, N / 2).
// EPI 2: C = ca * R + cb * (A W^T).  NORM: A stands for its RMS-normalised rows.
// FI: 16-row fragments per wave along M: 8 - the 256 x 256 tile on 8 waves (2 x 4); 4 - a 128 x 128 tile on 4 waves (2 x 2,
// 64 x 64 per wave, two workgroups per compute unit) for passes whose 256 x 256 tiles would not fill the device.  (A
// 64 x 64 tile on 2 waves was measured too: no faster than the tiled kernel's 64 x 64 form at 2 k rows.)
template <int DT, int EPI, bool NORM, int FI>
__global__ __launch_bounds__(64 * FI) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_big_kernel(BigParams P) {
  constexpr int WN = FI / 2;                   // waves along N (2 along M)
  constexpr int BM = 32 * FI, BN = 64 * WN;
  // one array per stage and operand: the compiler can then tell that the operand reads of one stage do not touch the
  // stage a load in flight is writing, and does not wait for that load
  __shared__ __attribute__((aligned(1024))) unsigned char sA0[BM * 128];
  __shared__ __attribute__((aligned(1024))) unsigned char sA1[BM * 128];
  __shared__ __attribute__((aligned(1024))) unsigned char sB0[BN * 128];
  __shared__ __attribute__((aligned(1024))) unsigned char sB1[BN * 128];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int T = P.tiles_m * P.tiles_n;
  const int per = (T + 7) / 8;
  const int L = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
  if (L >= T) return;
  const int bn = P.rowsplit ? L % P.tiles_n : L / P.tiles_m, bm = P.rowsplit ? L / P.tiles_n : L % P.tiles_m;
  const int m0 = bm * BM, n0 = bn * BN;
  const int nk = P.K / 64;

  // ---- loader: wave w fills blocks 4 w .. 4 w + 3 (8 rows each) of A and of W (BM = BN = 32 x the number of waves).  Rows
  // past M / N repeat the last row: what they produce is never stored.
  uint32_t offA[4], offB[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int rl = 8 * (4 * wave + i) + (lane >> 3);   // row inside the tile
    const int ch = (lane & 7) ^ ((rl >> 1) & 7);
    int row = m0 + rl;
    row = row < P.M ? row : P.M - 1;
    offA[i] = (uint32_t)row * P.lda2 + 16 * ch;
    row = n0 + rl;
    row = row < P.N ? row : P.N - 1;
    offB[i] = (uint32_t)row * P.ldw2 + 16 * ch;
  }
  const unsigned char* ga = (const unsigned char*)P.a;
  const unsigned char* gw = (const unsigned char*)P.w;
  auto issue = [&](unsigned char* sa, unsigned char* sb, int kt) {   // (past the last slab: the last slab again, into a stage nobody reads)
    const uint32_t ko = (uint32_t)(kt < nk ? kt : nk - 1) * 128;
#pragma unroll
    for (int i = 0; i < 4; i++)
      __builtin_amdgcn_global_load_lds(UVMI_GLBP(ga + offA[i] + ko), UVMI_LDSP(sa + (4 * wave + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++)
      __builtin_amdgcn_global_load_lds(UVMI_GLBP(gw + offB[i] + ko), UVMI_LDSP(sb + (4 * wave + i) * 1024), 16, 0, 0);
  };

  // ---- reader: wave (wm, wn) owns rows 16 FI wm .., columns 64 wn ..; lane (r, g) reads chunk (4 s + g) ^ ((r / 2) % 8) of
  // row r of a 16-row fragment for K-step s
  const int wm = wave / WN, wn = wave % WN;
  const int r = lane & 15, g = lane >> 4;
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int s = 0; s < 2; s++) {
    const uint32_t lo = (uint32_t)r * 128 + (uint32_t)((((4 * s + g) ^ ((r >> 1) & 7))) << 4);
    a_off[s] = (uint32_t)wm * (16 * FI * 128) + lo;
    b_off[s] = (uint32_t)wn * 8192 + lo;
  }
  gf4 acc[FI][4];
#pragma unroll
  for (int i = 0; i < FI; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = gf4{0.f, 0.f, 0.f, 0.f};

  gu4 w0[4], w1[4], f0[2], f1[2], f2[2];
  auto read_b = [&](const unsigned char* sb, int s, gu4* w) {
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = *(const gu4*)(sb + b_off[s] + j * 2048);
  };
  auto read_a = [&](const unsigned char* sa, int s, int i, gu4* f) {
    f[0] = *(const gu4*)(sa + a_off[s] + i * 2048);
    f[1] = *(const gu4*)(sa + a_off[s] + (i + 1) * 2048);
  };
  // (the MFMA's A input is the weight fragment, its B input the activation fragment: the accumulator holds C^T)
  auto mm1 = [&](int i, const gu4* f, const gu4* w) { acc[i][0] = gmfma<DT>(w[0], f[0], acc[i][0]); };
  auto mm7 = [&](int i, const gu4* f, const gu4* w) {
#pragma unroll
    for (int j = 1; j < 4; j++) acc[i][j] = gmfma<DT>(w[j], f[0], acc[i][j]);
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i + 1][j] = gmfma<DT>(w[j], f[1], acc[i + 1][j]);
  };
  // NORM: the squares of the rows are summed from the operand fragments as they pass: wave (wm, wn) takes row pair wn of
  // each K-step (rows 16 FI wm + 32 wn + 16 u + r, u = 0, 1; lane (r, g) sees 8 of a row's 32 values)
  float ss[2] = {0.f, 0.f};
  auto sumsq = [&](int pair, const gu4* f) {
    if (NORM && wn == pair) {
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float lo, hi;
          unpack2<DT>(f[u][e], lo, hi);
          ss[u] = fmaf(lo, lo, ss[u]);
          ss[u] = fmaf(hi, hi, ss[u]);
        }
    }
  };
#define UVMI_SB() __builtin_amdgcn_sched_barrier(0)

  issue(sA0, sB0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
  asm volatile("s_barrier" ::: "memory");
  issue(sA1, sB1, 1);
  read_b(sB0, 0, w0);
  read_a(sA0, 0, 0, f0);
  // Iteration k multiplies slab k out of stage S: 8 groups of 8 MFMAs (K-step s, row pair p); the operands of a group are
  // requested behind the first MFMA of the group before it, so a wait for them comes seven MFMAs after their request.
  // Before the last group: slab k + 1 has landed in the other stage (own loads: the wait; the other waves': the barrier)
  // and every read of stage S is complete, so S is refilled with slab k + 2 and the first operands of slab k + 1 are
  // requested.
#define UVMI_ITER(SA, SB_, SAN, SBN, k)                                                                                  \
  do {                                                                                                                   \
    mm1(0, f0, w0); UVMI_SB(); read_a(SA, 0, 2, f1); UVMI_SB(); mm7(0, f0, w0); sumsq(0, f0); UVMI_SB();                 \
    mm1(2, f1, w0); UVMI_SB(); read_a(SA, 0, 4, f2); UVMI_SB(); mm7(2, f1, w0); sumsq(1, f1); UVMI_SB();                 \
    mm1(4, f2, w0); UVMI_SB(); read_a(SA, 0, 6, f0); UVMI_SB(); mm7(4, f2, w0); sumsq(2, f2); UVMI_SB();                 \
    mm1(6, f0, w0); UVMI_SB(); read_b(SB_, 1, w1); read_a(SA, 1, 0, f1); UVMI_SB(); mm7(6, f0, w0); sumsq(3, f0); UVMI_SB(); \
    mm1(0, f1, w1); UVMI_SB(); read_a(SA, 1, 2, f2); UVMI_SB(); mm7(0, f1, w1); sumsq(0, f1); UVMI_SB();                 \
    mm1(2, f2, w1); UVMI_SB(); read_a(SA, 1, 4, f0); UVMI_SB(); mm7(2, f2, w1); sumsq(1, f2); UVMI_SB();                 \
    mm1(4, f0, w1); UVMI_SB(); read_a(SA, 1, 6, f1); UVMI_SB(); mm7(4, f0, w1); sumsq(2, f0); UVMI_SB();                 \
    __builtin_amdgcn_s_waitcnt(0x0f70);                                                                                  \
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");                                                      \
    issue(SA, SB_, (k) + 2);                                                                                             \
    read_b(SBN, 0, w0); read_a(SAN, 0, 0, f0); UVMI_SB();                                                                \
    mm1(6, f1, w1); mm7(6, f1, w1); sumsq(3, f1); UVMI_SB();                                                             \
  } while (0)
  // FI = 4: 4 groups per slab; the first operands of the next slab arrive in the buffer the iteration's second group used,
  // so two iterations alternate the roles of f0 and f1
#define UVMI_ITER4(SA, SB_, SAN, SBN, k, X, Y)                                                                           \
  do {                                                                                                                   \
    mm1(0, X, w0); UVMI_SB(); read_a(SA, 0, 2, Y); UVMI_SB(); mm7(0, X, w0); sumsq(0, X); UVMI_SB();                     \
    mm1(2, Y, w0); UVMI_SB(); read_b(SB_, 1, w1); read_a(SA, 1, 0, f2); UVMI_SB(); mm7(2, Y, w0); sumsq(1, Y); UVMI_SB(); \
    mm1(0, f2, w1); UVMI_SB(); read_a(SA, 1, 2, X); UVMI_SB(); mm7(0, f2, w1); sumsq(0, f2); UVMI_SB();                  \
    __builtin_amdgcn_s_waitcnt(0x0f70);                                                                                  \
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");                                                      \
    issue(SA, SB_, (k) + 2);                                                                                             \
    read_b(SBN, 0, w0); read_a(SAN, 0, 0, Y); UVMI_SB();                                                                 \
    mm1(2, X, w1); mm7(2, X, w1); sumsq(1, X); UVMI_SB();                                                                \
  } while (0)
  int k = 0;
  if constexpr (FI == 8) {
    for (; k + 2 <= nk; k += 2) {
      UVMI_ITER(sA0, sB0, sA1, sB1, k);
      UVMI_ITER(sA1, sB1, sA0, sB0, k + 1);
    }
    if (k < nk) UVMI_ITER(sA0, sB0, sA1, sB1, k);
  } else {
    for (; k + 2 <= nk; k += 2) {
      UVMI_ITER4(sA0, sB0, sA1, sB1, k, f0, f1);
      UVMI_ITER4(sA1, sB1, sA0, sB0, k + 1, f1, f0);
    }
    if (k < nk) UVMI_ITER4(sA0, sB0, sA1, sB1, k, f0, f1);
  }
#undef UVMI_ITER4
#undef UVMI_ITER
#undef UVMI_SB
  __builtin_amdgcn_s_waitcnt(0x0f70);   // the loads past the last slab have landed before LDS is reused or the wave ends

  // ---- row scales of the pre-norm: the 4 lane groups of a row add their sums; LDS carries the scales to every wave
  float rn[FI];
#pragma unroll
  for (int i = 0; i < FI; i++) rn[i] = 1.0f;
  if (NORM) {
    float* sRS = (float*)sA0;
    __syncthreads();   // every wave's loads have landed and its operand reads are done
#pragma unroll
    for (int u = 0; u < 2; u++) {
      float v = ss[u];
      v += lane_xor16(v);
      v = xsum32(v);
      if (g == 0) sRS[16 * FI * wm + 32 * wn + 16 * u + r] = rsqrtf(v / (float)P.K + P.eps);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < FI; i++) rn[i] = sRS[16 * FI * wm + 16 * i + r];
  }

  // ---- epilogue: accumulator (i, j): lane (r, g) holds C[m0 + 16 FI wm + 16 i + r][n0 + 64 wn + 16 j + 4 g + t], t = 0..3
#pragma unroll
  for (int i = 0; i < FI; i++) {
    const int row = m0 + 16 * FI * wm + 16 * i + r;
    if (EPI == 1) {
      // gate slab j, up slab j + 1 -> 4 outputs per slab pair; after the 2 x 2 transpose lane (r, g) holds the 8 consecutive
      // output columns 16 (g % 2) + 8 (g / 2) .. of the wave's 32
      uint32_t x0[2], x1[2];
#pragma unroll
      for (int jp = 0; jp < 2; jp++) {
        float o[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
          const float gv = ground<DT>(acc[i][2 * jp][t] * rn[i]), uv = ground<DT>(acc[i][2 * jp + 1][t] * rn[i]);
          o[t] = silu_round<DT>(gv) * uv;
        }
        (jp == 0 ? x0 : x1)[0] = gpack<DT>(o[0], o[1]);
        (jp == 0 ? x0 : x1)[1] = gpack<DT>(o[2], o[3]);
      }
      xpose2(x0[0], x1[0]);
      xpose2(x0[1], x1[1]);
      const int n = (n0 >> 1) + 32 * wn + 16 * (g & 1) + 8 * (g >> 1);   // output column
      if (row < P.M && 2 * n < P.N) {
        uint16_t* cp = (uint16_t*)P.c + (int64_t)row * P.ldc + n;
        *(uint4*)cp = uint4{x0[0], x0[1], x1[0], x1[1]};
      }
    } else {
      uint32_t lo[4], hi[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        lo[j] = gpack<DT>(acc[i][j][0] * rn[i], acc[i][j][1] * rn[i]);
        hi[j] = gpack<DT>(acc[i][j][2] * rn[i], acc[i][j][3] * rn[i]);
      }
      xpose4(lo);
      xpose4(hi);
      // lane (r, g) now holds columns 16 g .. 16 g + 15 of the wave's 64: words lo[0] hi[0] lo[1] hi[1] ...
      const int n = n0 + 64 * wn + 16 * g;
      if (row < P.M && n < P.N) {
        uint32_t wds[8] = {lo[0], hi[0], lo[1], hi[1], lo[2], hi[2], lo[3], hi[3]};
        if (EPI == 2) {
          const uint16_t* rp = (const uint16_t*)P.r + (int64_t)row * P.ldr + n;
          const uint4 q0 = *(const uint4*)rp, q1 = *(const uint4*)(rp + 8);
          const uint32_t rw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
          for (int e = 0; e < 8; e++) {
            float p0, p1, x0, x1;
            unpack2<DT>(wds[e], p0, p1);   // the product, already rounded to the activation type
            unpack2<DT>(rw[e], x0, x1);
            wds[e] = gpack<DT>(P.ca * x0 + P.cb * p0, P.ca * x1 + P.cb * p1);
          }
        }
        uint16_t* cp = (uint16_t*)P.c + (int64_t)row * P.ldc + n;
        *(uint4*)cp = uint4{wds[0], wds[1], wds[2], wds[3]};
        *(uint4*)(cp + 8) = uint4{wds[4], wds[5], wds[6], wds[7]};
      }
    }
  }
}

template <int DT, int FI>
static void launch_big(const uvmi_gemm_args* a, const BigParams& P, hipStream_t st) {
  const int T = P.tiles_m * P.tiles_n;
  const dim3 grid((unsigned)(((T + 7) / 8) * 8)), blk(64 * FI);
#define UVMI_GO(EPI, NORM) hipLaunchKernelGGL((gemm_big_kernel<DT, EPI, NORM, FI>), grid, blk, 0, st, P)
  const bool norm = a->norm_a != 0;
  if (a->epilogue == UVMI_GEMM_RESID) { if (norm) UVMI_GO(2, true); else UVMI_GO(2, false); }
  else if (a->epilogue == UVMI_GEMM_SWIGLU) { if (norm) UVMI_GO(1, true); else UVMI_GO(1, false); }
  else { if (norm) UVMI_GO(0, true); else UVMI_GO(0, false); }
#undef UVMI_GO
}

// Arguments are validated by the caller (uvmi_gemm_tn_ex), which also checks K >= 128.  tile: 256 or 128.
void gemm_big_launch(const uvmi_gemm_args* a, int tile, hipStream_t st) {
  BigParams P;
  P.a = a->a; P.w = a->w; P.c = a->c; P.r = a->resid;
  P.lda2 = (uint32_t)a->lda * 2; P.ldw2 = (uint32_t)a->ldw * 2; P.ldc = a->ldc; P.ldr = a->ldr;
  P.M = (int)a->M; P.N = a->N; P.K = a->K;
  P.tiles_m = (int)((a->M + tile - 1) / tile);
  P.tiles_n = (a->N + tile - 1) / tile;
  P.eps = a->eps; P.ca = a->ca; P.cb = a->cb;
  const double bytes_a = (double)a->M * a->K, bytes_w = (double)a->N * a->K;
  P.rowsplit = bytes_a / 8 + bytes_w < bytes_a + bytes_w / 8;
  if (a->dtype == UVMI_F16) { if (tile == 256) launch_big<UVMI_F16, 8>(a, P, st); else launch_big<UVMI_F16, 4>(a, P, st); }
  else { if (tile == 256) launch_big<UVMI_BF16, 8>(a, P, st); else launch_big<UVMI_BF16, 4>(a, P, st); }
}

}  // namespace uvmi
