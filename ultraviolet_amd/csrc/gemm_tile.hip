// Tiled 16-bit GEMM for the projections of a large decode step (several hundred to a few thousand rows):
// C[M, N] = A[M, K] . W[N, K]^T with fp32 accumulation and the epilogues of the skinny kernel (gemm.hip) - SwiGLU on
// interleaved gate / up slabs, the block's residual update, the RMS pre-norm as a row scale.  These are the F.linear calls
// of the reference's fused inference path (ultraviolet/model.py:302-335, 388-391) with what surrounds them (:566-571).
//
// At this size a projection is a contraction of 1 - 9 GFLOP whose operands (a few MB) live in the L2 / last-level cache:
// the kernel is bound by how fast a compute unit can feed its matrix cores from LDS.
//   * a workgroup of 4 waves (2 x 2) owns a BM x BN tile (128 x 128, or 64 x 64 when the larger tile would leave compute
//     units idle); K is walked in slabs of 64;
//   * a slab of A and of W is fetched by 16-byte buffer loads (8 consecutive lanes on one 128-byte row segment) into
//     registers while the previous slab is multiplied, then parked in the other half of a double-buffered LDS tile: one
//     barrier per slab;
//   * LDS rows are 128 bytes (one slab) with the 16-byte chunk index xor-ed with (row / 2) % 8, which makes both the
//     row-wise writes and the 16-row operand reads (lane (r, g) reads chunk 4 s + g of row r) touch every bank once;
//   * the MFMA's A input is the weight fragment and its B input the activation fragment, so an accumulator holds C^T: a
//     lane has 4 consecutive columns of one row and stores them as one 8-byte write;
//   * rows past M, weight rows past N and slabs past K read as zero through the buffer bounds (offset pushed out of range),
//     so the loop body has no branches;
//   * tiles are dealt to the XCDs in contiguous runs, by row blocks or by weight strips, whichever leaves the smaller
//     working set per XCD (an eighth of A plus all of W, or all of A plus an eighth of W): it must fit that XCD's 4 MB L2,
//     or every strip streams the other operand from beyond it again;
//   * NORM: the threads that fetch A sum the squares of what they fetch; the row scale rsqrt(mean + eps) meets the
//     accumulators in the epilogue.
#include "common.h"
#include "gemm_util.h"

namespace uvmi {

struct TileParams {
  const void* a; const void* w; void* c; const void* r;
  uint32_t lda2, ldw2;  // row pitches in bytes
  int64_t ldc, ldr;     // elements
  int M, N, K, tiles_m, tiles_n;
  int rowsplit;         // an XCD's run of tiles walks the column tiles of its row blocks (else the row blocks of its column tiles)
  float eps, ca, cb;
};

// EPI 0: C = A W^T (M, N).  EPI 1: W rows are [gate 16 | up 16] slabs; C = silu(gate) * up, (M, N / 2).
// EPI 2: C = ca * R + cb * (A W^T).  NORM: A stands for its RMS-normalised rows.
template <int DT, int BM, int BN, int D, int EPI, bool NORM>
__global__ __launch_bounds__(256) void gemm_tile_kernel(TileParams P) {
  constexpr int PA = BM / 32, PB = BN / 32;  // load passes: 32 rows x 8 chunks of 16 bytes per pass of a group
  constexpr int FM = BM / 32, FN = BN / 32;  // 16-row fragments per wave in each direction (2 x 2 waves)
  constexpr uint32_t OOB = 0x40000000u;      // added to an offset that must read as zero (every valid offset is below 2^30)
  __shared__ __attribute__((aligned(16))) unsigned char sA_[2][BM * 128];
  __shared__ __attribute__((aligned(16))) unsigned char sB_[2][BN * 128];
  auto sA = [&](int buf) { return sA_[buf]; };
  auto sB = [&](int buf) { return sB_[buf]; };
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

  const uint32_t boundA = (uint32_t)(P.M - 1) * P.lda2 + (uint32_t)P.K * 2;
  const uint32_t boundW = (uint32_t)(P.N - 1) * P.ldw2 + (uint32_t)P.K * 2;
  const __amdgpu_buffer_rsrc_t rA = __builtin_amdgcn_make_buffer_rsrc((void*)P.a, 0, (int)boundA, 0x00020000);
  const __amdgpu_buffer_rsrc_t rW = __builtin_amdgcn_make_buffer_rsrc((void*)P.w, 0, (int)boundW, 0x00020000);

  // ---- fetch: thread (lr = tid / 8, ch = tid % 8) takes chunk ch of rows lr + 32 p
  const int lr = tid >> 3, ch = tid & 7;
  uint32_t goA[PA], goB[PB];
#pragma unroll
  for (int p = 0; p < PA; p++) {
    const int row = m0 + 32 * p + lr;
    goA[p] = (row < P.M ? 0u : OOB) + (uint32_t)row * P.lda2 + 16 * ch;
  }
#pragma unroll
  for (int p = 0; p < PB; p++) {
    const int row = n0 + 32 * p + lr;
    goB[p] = (row < P.N ? 0u : OOB) + (uint32_t)row * P.ldw2 + 16 * ch;
  }
  const uint32_t st_off = (uint32_t)lr * 128 + (uint32_t)((ch ^ ((lr >> 1) & 7)) << 4);  // + 32 p rows
  // a ring of D slabs in registers: slab j waits in slot j % D from its request until it is parked in LDS, D - 1 slabs
  // of multiplying later, so a slab's trip from the L2 is hidden behind the slabs ahead of it
  gu4 ra[D][PA], rb[D][PB];
  float ss[PA];
#pragma unroll
  for (int p = 0; p < PA; p++) ss[p] = 0.f;
  auto fetch = [&](int kt, int slot) {
    const uint32_t ko = kt < nk ? (uint32_t)kt * 128 : OOB;
#pragma unroll
    for (int p = 0; p < PA; p++) ra[slot][p] = __builtin_amdgcn_raw_buffer_load_b128(rA, goA[p] + ko, 0, 0);
#pragma unroll
    for (int p = 0; p < PB; p++) rb[slot][p] = __builtin_amdgcn_raw_buffer_load_b128(rW, goB[p] + ko, 0, 0);
  };
  auto park = [&](int slot, int buf) {
#pragma unroll
    for (int p = 0; p < PA; p++) {
      *(gu4*)(sA(buf) + 32 * p * 128 + st_off) = ra[slot][p];
      if (NORM) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const uint32_t w = ra[slot][p][i];
          float lo, hi;
          if (DT == UVMI_BF16) { lo = __uint_as_float(w << 16); hi = __uint_as_float(w & 0xffff0000u); }
          else { lo = half_bits_to_float((uint16_t)(w & 0xffff)); hi = half_bits_to_float((uint16_t)(w >> 16)); }
          ss[p] = fmaf(lo, lo, ss[p]);
          ss[p] = fmaf(hi, hi, ss[p]);
        }
      }
    }
#pragma unroll
    for (int p = 0; p < PB; p++) *(gu4*)(sB(buf) + 32 * p * 128 + st_off) = rb[slot][p];
  };

  // ---- multiply: wave (wm, wn) owns rows wm BM/2.., columns wn BN/2..; lane (r, g) reads chunk 4 s + g of row r
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 15, g = lane >> 4;
  uint32_t ld_off[2];
#pragma unroll
  for (int s = 0; s < 2; s++) ld_off[s] = (uint32_t)r * 128 + (uint32_t)((((4 * s + g) ^ ((r >> 1) & 7))) << 4);
  const uint32_t a_base = (uint32_t)(wm * (BM / 2)) * 128, b_base = (uint32_t)(wn * (BN / 2)) * 128;
  gf4 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++) acc[i][j] = gf4{0.f, 0.f, 0.f, 0.f};
  gu4 wf[2][FN], af[2][FM];
  auto read_operands = [&](int buf) {
#pragma unroll
    for (int s = 0; s < 2; s++) {
#pragma unroll
      for (int j = 0; j < FN; j++) wf[s][j] = *(const gu4*)(sB(buf) + b_base + 16 * j * 128 + ld_off[s]);
#pragma unroll
      for (int i = 0; i < FM; i++) af[s][i] = *(const gu4*)(sA(buf) + a_base + 16 * i * 128 + ld_off[s]);
    }
  };
  auto multiply = [&]() {
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++) acc[i][j] = gmfma<DT>(wf[s][j], af[s][i], acc[i][j]);
  };

#pragma unroll
  for (int d = 0; d < D; d++) fetch(d, d);   // (past the last slab: zeros, no traffic)
  park(0, 0);
  fetch(D, 0);
  __syncthreads();
  // iteration k multiplies slab k out of LDS half k % 2, parks slab k + 1 in the other half and requests slab k + 1 + D into
  // the slot that frees; whole turns of the ring run without branches, the last nk % D iterations follow outside the loop
  // (order inside an iteration: all operand reads of the slab, then the next slab's LDS writes and the request that
  // refills the ring, then the MFMAs - which run while those writes and requests drain and other waves read)
  auto iteration = [&](int k, int d) {
    read_operands(k & 1);
    __builtin_amdgcn_sched_barrier(0);
    park((d + 1) % D, (k + 1) & 1);          // (the slab past the end lands in the half nobody reads again)
    fetch(k + 1 + D, (d + 1) % D);
    __builtin_amdgcn_sched_barrier(0);
    multiply();
    __syncthreads();
  };
  int kt = 0;
  for (; kt + D <= nk; kt += D) {
#pragma unroll
    for (int d = 0; d < D; d++) iteration(kt + d, d);
  }
#pragma unroll
  for (int d = 0; d < D - 1; d++)
    if (kt + d < nk) iteration(kt + d, d);   // workgroup-uniform

  // ---- row scales of the pre-norm: the 8 lanes of a row add their sums; LDS (free now) carries them to the epilogue
  float* sRS = (float*)sA(0);
  if (NORM) {
#pragma unroll
    for (int p = 0; p < PA; p++) {
      float v = ss[p];
      v += __shfl_xor(v, 1, 64);
      v += __shfl_xor(v, 2, 64);
      v += __shfl_xor(v, 4, 64);
      if (ch == 0) sRS[32 * p + lr] = rsqrtf(v / (float)P.K + P.eps);
    }
    __syncthreads();
  }

  // ---- epilogue: accumulator (i, j): lane (r, g) holds C[m0 + wm BM/2 + 16 i + r][n0 + wn BN/2 + 16 j + 4 g + t], t = 0..3
#pragma unroll
  for (int i = 0; i < FM; i++) {
    const int rl = wm * (BM / 2) + 16 * i + r;
    const int row = m0 + rl;
    if (row >= P.M) continue;
    const float rn = NORM ? sRS[rl] : 1.0f;
    if (EPI == 1) {
#pragma unroll
      for (int j = 0; j < FN; j += 2) {
        const int n = n0 + wn * (BN / 2) + 16 * j;  // gate slab at W rows n.., up slab at n + 16..
        if (n >= P.N) continue;
        float o[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
          const float gv = ground<DT>(acc[i][j][t] * rn), uv = ground<DT>(acc[i][j + 1][t] * rn);
          o[t] = silu_round<DT>(gv) * uv;
        }
        uint16_t* cp = (uint16_t*)P.c + (int64_t)row * P.ldc + (n >> 1) + 4 * g;
        *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
      }
    } else {
#pragma unroll
      for (int j = 0; j < FN; j++) {
        const int n = n0 + wn * (BN / 2) + 16 * j;
        if (n >= P.N) continue;
        float o[4];
#pragma unroll
        for (int t = 0; t < 4; t++) o[t] = acc[i][j][t] * rn;
        if (EPI == 2) {
          const uint2 rw = *(const uint2*)((const uint16_t*)P.r + (int64_t)row * P.ldr + n + 4 * g);
          float x[4];
          if (DT == UVMI_BF16) {
            x[0] = __uint_as_float(rw.x << 16); x[1] = __uint_as_float(rw.x & 0xffff0000u);
            x[2] = __uint_as_float(rw.y << 16); x[3] = __uint_as_float(rw.y & 0xffff0000u);
          } else {
            x[0] = half_bits_to_float((uint16_t)(rw.x & 0xffff)); x[1] = half_bits_to_float((uint16_t)(rw.x >> 16));
            x[2] = half_bits_to_float((uint16_t)(rw.y & 0xffff)); x[3] = half_bits_to_float((uint16_t)(rw.y >> 16));
          }
#pragma unroll
          for (int t = 0; t < 4; t++) o[t] = P.ca * x[t] + P.cb * ground<DT>(o[t]);
        }
        uint16_t* cp = (uint16_t*)P.c + (int64_t)row * P.ldc + n + 4 * g;
        *(uint2*)cp = uint2{gpack<DT>(o[0], o[1]), gpack<DT>(o[2], o[3])};
      }
    }
  }
}

template <int DT, int BM, int BN, int D>
static void launch_tile(const uvmi_gemm_args* a, const TileParams& P, hipStream_t st) {
  const int T = P.tiles_m * P.tiles_n;
  const dim3 grid((unsigned)(((T + 7) / 8) * 8)), blk(256);
#define UVMI_GO(EPI, NORM) hipLaunchKernelGGL((gemm_tile_kernel<DT, BM, BN, D, EPI, NORM>), grid, blk, 0, st, P)
  const bool norm = a->norm_a != 0;
  if (a->epilogue == UVMI_GEMM_RESID) { if (norm) UVMI_GO(2, true); else UVMI_GO(2, false); }
  else if (a->epilogue == UVMI_GEMM_SWIGLU) { if (norm) UVMI_GO(1, true); else UVMI_GO(1, false); }
  else { if (norm) UVMI_GO(0, true); else UVMI_GO(0, false); }
#undef UVMI_GO
}

// Arguments are validated by the caller (uvmi_gemm_tn_ex).  big: 128 x 128 tiles with two slabs in flight, else 64 x 64 with four.
void gemm_tile_launch(const uvmi_gemm_args* a, bool big, hipStream_t st) {
  TileParams P;
  P.a = a->a; P.w = a->w; P.c = a->c; P.r = a->resid;
  P.lda2 = (uint32_t)a->lda * 2; P.ldw2 = (uint32_t)a->ldw * 2; P.ldc = a->ldc; P.ldr = a->ldr;
  P.M = (int)a->M; P.N = a->N; P.K = a->K;
  const int bm = big ? 128 : 64;
  P.tiles_m = (int)((a->M + bm - 1) / bm);
  P.tiles_n = (a->N + bm - 1) / bm;
  P.eps = a->eps; P.ca = a->ca; P.cb = a->cb;
  const double bytes_a = (double)a->M * a->K, bytes_w = (double)a->N * a->K;
  P.rowsplit = bytes_a / 8 + bytes_w < bytes_a + bytes_w / 8;
  if (a->dtype == UVMI_F16) { if (big) launch_tile<UVMI_F16, 128, 128, 2>(a, P, st); else launch_tile<UVMI_F16, 64, 64, 4>(a, P, st); }
  else { if (big) launch_tile<UVMI_BF16, 128, 128, 2>(a, P, st); else launch_tile<UVMI_BF16, 64, 64, 4>(a, P, st); }
}

}  // namespace uvmi
