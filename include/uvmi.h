/*
 * uvmi.h - C ABI of the MI355X (gfx950) decode engine kernels for UV-50M.
 *
 * Every entry point takes raw device pointers, explicit sizes and strides (in ELEMENTS unless a name says
 * bytes) and a HIP stream handle (hipStream_t passed as void*; NULL = the default stream).  No entry point
 * allocates device memory, synchronises the device or throws: the return value is 0 on success or a negative
 * UVMI_E* code, and uvmi_last_error() returns a thread-local message for the last failure on this thread.
 * All launches go to the device that is current on the calling thread, so callers running a second Python
 * thread under another device (reference: scripts/rl_grpo.py:519-521) are served.  The library keeps no state
 * between calls, with two stated exceptions: a per-thread cached compute-unit count, and uvmi_decode_attn_noalloc,
 * which keeps a process-wide table of one device address per GPU (filled under a mutex on the first call on each
 * device) and a scratch array in device memory that all its calls on one GPU share (see its declaration).
 *
 * uvmi_version() is the revision of this header's argument structs: it moves whenever a struct gains a field, so a
 * caller built against an older header can tell that the layout it passes is no longer the one the library reads.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the reference checkout).
 */
#ifndef UVMI_H
#define UVMI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define UVMI_OK 0
#define UVMI_EINVAL (-1)      /* malformed argument (null pointer, negative size, bad enum) */
#define UVMI_EUNSUPPORTED (-2) /* shape / dtype / alignment the kernels do not cover */
#define UVMI_EWORKSPACE (-3)  /* workspace pointer missing or too small */
#define UVMI_EHIP (-4)        /* a HIP runtime call failed (message holds hipGetErrorString) */

/* element types */
#define UVMI_F16 0
#define UVMI_BF16 1
#define UVMI_F32 2
#define UVMI_I8 3
#define UVMI_I32 4
#define UVMI_I64 5

/* Revision of the argument structs below (uvmi_version() returns the value the library was built with). */
#define UVMI_ABI_VERSION 4
int uvmi_version(void);
const char* uvmi_last_error(void);
/* Number of compute units of the current device (used by the split heuristics); <0 on error. */
int uvmi_device_cus(void);

/* ------------------------------------------------------------------------------------------------------------
 * int8 KV quantizer and cache writes.  Replaces ultraviolet/kernels/kv_quant.py.
 * ---------------------------------------------------------------------------------------------------------- */

/* quantize_kv (kv_quant.py:12-19): n_rows rows of hd elements (x_row_stride elements apart, unit inner stride)
 * -> q int8 (n_rows, hd) contiguous, scale fp16 (n_rows,) contiguous.  s16 = fp16(absmax/127); the row is divided
 * by max(float(s16), 1e-30) with IEEE fp32 division, rounded half-to-even and clamped to +-127.  Bit-exact. */
int uvmi_quantize_rows(const void* x, int x_dtype, int64_t n_rows, int hd, int64_t x_row_stride,
                       int8_t* q, uint16_t* scale, void* stream);

/* dequantize_kv (kv_quant.py:22-23): out[r, :] = q[r, :] * float(scale[r]) cast to out_dtype. */
int uvmi_dequantize_rows(const int8_t* q, const uint16_t* scale, int64_t n_rows, int hd, void* out, int out_dtype,
                         void* stream);

/* kv_write (kv_quant.py:26-36): quantize row r of x and store it at row flat_idx[r] of the contiguous
 * (cache_rows, hd) int8 view of the cache and at element flat_idx[r] of the flat fp16 scale view.
 * flat_idx is int64 (idx_dtype UVMI_I64) or int32; rows whose index falls outside [0, cache_rows) are skipped.
 * If scale is NULL the cache holds cache_dtype (F16/BF16) values and rows are copied with a cast. */
int uvmi_kv_write(void* cache, int cache_dtype, uint16_t* scale, int64_t cache_rows, const void* flat_idx,
                  int idx_dtype, const void* x, int x_dtype, int64_t n_rows, int hd, int64_t x_row_stride,
                  void* stream);

/* Fused decode-time append of K and V of one layer (fast_decode.py:291-294, 315-317): for every row b and kv
 * head h, quantize k[b, h, :] and v[b, h, :] and store them at slot pos[b] (linear cache) or pos[b] % S (ring)
 * of k_cache / v_cache (B, KH, S, hd; batch/head/slot strides given) with their fp16 scales (B, KH, S).
 * One launch for both tensors.  Rows with pos[b] < 0, or pos[b] >= S on a linear cache, are skipped. */
typedef struct uvmi_kv_append_args {
  const void* k; const void* v; int x_dtype;            /* (B, KH, hd) new keys / values */
  int64_t sxb, sxh;                                     /* strides of k and v (shared) */
  int8_t* k_cache; int8_t* v_cache;                     /* (B, KH, S, hd) */
  int64_t scb, sch, scs;                                /* cache strides (shared by K and V) */
  uint16_t* k_scale; uint16_t* v_scale;                 /* (B, KH, S) fp16 */
  int64_t ssb, ssh;                                     /* scale strides (slot stride 1) */
  const void* pos; int idx_dtype;                       /* (B,) position being written */
  const void* rows;                                     /* optional (B,) cache row of each input row (same
                                                           idx_dtype); NULL = identity */
  int B, KH, S, hd, ring;
} uvmi_kv_append_args;
int uvmi_kv_append(const uvmi_kv_append_args* a, void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * Ragged single-query decode attention.  Replaces decode_attention / mathk::decode_attn
 * (ultraviolet/kernels/decode_attn.py:174-230, kernels/decode_attn_cuda.py:273-309).
 * ---------------------------------------------------------------------------------------------------------- */
struct uvmi_attn_qkv_fuse;
typedef struct uvmi_attn_args {
  const void* q; int q_dtype;              /* (B, H, hd) F16 / BF16 (the MFMA kernel multiplies in 16 bits) or F32 (the generic
                                              kernel: every product and probability stays fp32), inner stride 1 */
  int64_t sqb, sqh;
  const void* k_cache; const void* v_cache; int kv_dtype; /* (B, KH, S, hd) I8, F16, BF16 or F32, inner stride 1 */
  int64_t skb, skh, sks, svb, svh, svs;
  const void* k_scale; const void* v_scale; /* (B, KH, S) fp16 when kv_dtype == I8, else NULL */
  int64_t ssb, ssh, stb, sth;
  const void* pos; const void* starts; int idx_dtype; /* (B,) I64 or I32: position of the current key (already
                                                         written) and first valid position of each row */
  const void* rows;                        /* optional (B,) cache row of each query row (same idx_dtype): lets a compacted
                                              batch of active slots address a larger cache; rows[b] < 0 marks a padding
                                              row (no keys, zero output); NULL = identity */
  void* out; int out_dtype;                /* (B, H, hd) F16 / BF16 / F32, inner stride 1 */
  int64_t sob, soh;
  int B, H, KH, S, hd;
  float scale;                             /* softmax scale applied to q.k */
  int window;                              /* 0 = unlimited; else keys pos-window+1..pos */
  int ring;                                /* slot of position t is t % S (else t) */
  int num_splits;                          /* >= 1: upper bound on the chunks a row's key range is cut into */
  int chunk_keys;                          /* 0: every row is cut into num_splits equal chunks (the reference's rule,
                                              decode_attn.py:42-44); > 0: chunks of at least this many keys, so short
                                              rows use fewer work items and a row that fits one chunk skips the combine */
  void* workspace; size_t workspace_bytes; /* >= uvmi_decode_attn_workspace_bytes(...) when num_splits > 1 */
  /* Optional fused epilogue, used when post_vhat != NULL (needs the MFMA kernel - head_dim 64, an int8 cache or one in
   * the q dtype - and num_splits == 1): Attention.post
   * before the output projection (ultraviolet/model.py:321-333): XSA z -= xsa[h] (z . v_hat) v_hat with the unquantized
   * current v, then z *= 2 sigmoid(gate_w[h] . xn[:gate_ch]); out then holds that result in out_dtype. */
  const float* post_vhat;                  /* (B, KH, hd) fp32 normalized current v (uvmi_qkv_post vhat_out); enables the epilogue */
  const float* post_gate;                  /* (B, H) fp32 gate values (uvmi_qkv_post gate_out), or NULL */
  const float* post_xsa;                   /* (H,) tanh(alpha) fp32, or NULL */
  int post_round_dtype;                    /* activation dtype whose rounding the epilogue follows (F16 / BF16 / F32) */
  const struct uvmi_attn_qkv_fuse* fuse;   /* optional: take q and the row's own key from the projection output (below) */
} uvmi_attn_args;

/* Fused QKV post-processing for decode rows (uvmi_attn_args.fuse).  The attention kernel then does what uvmi_qkv_post
 * does for the row's own token (QK-norm, partial rotation, value embedding, append at pos[b]: int8 codes and fp16 scales,
 * or k and v themselves on a cache held in the q dtype - the reference's Attention.qkv + fast_decode.py:291-294, 315-317) and attends the cached range lo..pos-1 plus that key from registers,
 * so the step needs no separate post-processing launch.  `qkv` is the output of the projection GEMM, (B, row_stride)
 * in the q dtype: H*64 q values, KH*64 k, KH*64 v, then at column ext_col the H gate logits (W_gate[h] . xn[:gate_ch],
 * formed by appending the gate rows to the projection weight) and the KH value-embedding gate logits.  q / sqb / sqh of
 * the attention arguments are ignored; k_cache, v_cache and the scales are written at the rows' positions.  The XSA /
 * gate epilogue is always applied (post_vhat and post_gate are ignored: the kernel forms them; post_xsa may be NULL).
 * Needs the MFMA path (head_dim 64, an int8 cache or one in the q dtype), num_splits == 1, q dtype = activation dtype,
 * n_pairs 16 when rope. */
typedef struct uvmi_attn_qkv_fuse {
  const void* qkv; int64_t row_stride;     /* elements */
  int ext_col;                             /* first gate-logit column */
  int has_gate;                            /* gate logits present (else gate = 1) */
  const void* tok;                         /* (B,) token ids (idx_dtype of the attention arguments), for the value embedding */
  const void* ve_table; int64_t vocab;     /* (vocab, KH, 64) value embedding in the q dtype, or NULL (has_ve = 0) */
  int has_ve;
  const float* rope_table; int rope_positions; /* uvmi_rope_table output for n_pairs = 16 (128-byte aligned) and its row count:
                                                 every pos[b] must be below it */
  int n_pairs; int rope;
  float eps, xsa_eps;
} uvmi_attn_qkv_fuse;
/* The rotation table of the fused path: out (n_positions, 2 * n_pairs) fp32, row p = cos(p * inv_freq[j]) for j <
 * n_pairs, then sin, each rounded to round_dtype - the values uvmi_qkv_post forms per token (the reference keeps the same
 * table as a buffer of the model, ultraviolet/model.py:198-226). */
int uvmi_rope_table(const float* inv_freq, int n_pairs, int64_t n_positions, int round_dtype, float* out, void* stream);

/* Keys attended by row b: absolute positions max(starts[b], pos[b]-window+1, 0) .. pos[b]; a row with no valid
 * key yields zeros.  fp32 accumulation; int8 caches are dequantised in registers (K scale on the score column,
 * V scale on the probability).  Deterministic for a given num_splits. */
int uvmi_decode_attn(const uvmi_attn_args* a, void* stream);
size_t uvmi_decode_attn_workspace_bytes(int B, int H, int KH, int hd, int num_splits);
/* default_splits (decode_attn.py:121-129) re-derived for 256 CUs x wave64: enough (row, kv head, split) work
 * items to fill the device, each chunk >= min_chunk keys, at most 64.  n_cus <= 0: query the current device. */
int uvmi_default_splits(int64_t n_bk, int ctx, int n_cus);
/* 1 if uvmi_decode_attn runs the MFMA kernel for these arguments (head_dim 64, up to 8 query heads per kv head, an
 * int8 cache with fp16 scales or a cache held unquantized in the q dtype, aligned rows), 0 if the generic kernel (any
 * hd <= 256, G <= 16), negative if unsupported.  Mirrors decode_attn_cuda.supported (decode_attn_cuda.py:265-270). */
int uvmi_decode_attn_path(const uvmi_attn_args* a);

/* Measurement aid, no counterpart in the reference: the launch uvmi_decode_attn would make for these arguments with one
 * half of the kernel's work taken out - mode 1 keeps the memory stream (every K / V / scale tile is loaded as in the real
 * kernel and folded into the state with a few xors; no products, no exponentials), mode 2 keeps the arithmetic (tiles are
 * made up in registers; the cache is not read).  `out` is written with meaningless values.  Timed beside the real launch
 * the two say which of the kernel's resources bounds it.  Only the engine's decode shape: int8 cache, bf16 q and out, 8
 * query heads on one kv head, I64 indices, num_splits 1, no fuse; anything else returns UVMI_EUNSUPPORTED. */
int uvmi_decode_attn_probe(const uvmi_attn_args* a, int mode, void* stream);

/* uvmi_decode_attn for callers that cannot allocate device memory - code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference (its op allocates its split partials per call,
 * ultraviolet/kernels/decode_attn.py:157-159).  Same arguments, kernels and results as uvmi_decode_attn, except that
 * workspace / workspace_bytes are ignored: when num_splits > 1 the split partials go to an array of
 * UVMI_NOALLOC_SCRATCH_BYTES that is part of the library's device code (each GPU the library runs on holds it until the
 * process ends).  A call whose partials (uvmi_decode_attn_workspace_bytes) exceed it returns UVMI_EWORKSPACE.  The call
 * makes no hipMalloc / hipFree and no allocating library call; its first use on a device looks the array's address up
 * once (make that first call outside a graph capture).  Nothing in the array has to start at zero - every partial a
 * call reads it has written itself - but all calls on one GPU share it: calls that overlap on one GPU (two streams,
 * two threads) race; serialise them or use uvmi_decode_attn with separate workspaces. */
#define UVMI_NOALLOC_SCRATCH_BYTES (8u << 20)
int uvmi_decode_attn_noalloc(const uvmi_attn_args* a, void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * 16-bit GEMM of a decode step's projections: C (M, N) = A (M, K) . W (N, K)^T, fp32 accumulation, A, W, C in `dtype`
 * (F16 / BF16), rows contiguous with pitches lda, ldw, ldc (elements).  Replaces the F.linear calls of the reference's
 * fused inference path (ultraviolet/model.py:302-335 attention projections, 388-391 MLP).  K % 64 == 0, K <= 8192;
 * N % 16 == 0.  Three kernel families behind one entry point:
 *   - skinny forms for steps of up to a few hundred rows, where the weights are the traffic: a workgroup requests its
 *     whole weight strip and its activation rows in one burst (K <= 1984; 960 with SWIGLU);
 *   - a tiled form (128 x 128 or 64 x 64 tiles, operand slabs double-buffered in LDS behind a ring of slabs in flight)
 *     for steps of several hundred to a few thousand rows, where the product is bound by feeding the matrix cores;
 *   - a form whose slabs go from global memory straight into LDS, with operand reads pipelined ahead of the MFMAs and
 *     whole-line stores: 256 x 256 tiles (128 x 64 per wave) for the passes of many thousand rows - a packed prefill, a
 *     mixed prefill + decode pass - where L2 and LDS bandwidth per flop decide, and 128 x 128 tiles in place of the
 *     tiled form's wherever C is 16-byte aligned.
 * epilogue UVMI_GEMM_SWIGLU (N % 32 == 0): W holds w_gate and w_up interleaved in slabs of 16 rows ([gate 0..15 |
 * up 0..15 | gate 16..31 | ...], N = 2 f rows) and C (M, f) = silu(A w_gate^T) * (A w_up^T) with the roundings of the
 * separate SwiGLU pass (model.py:388-391).
 * ---------------------------------------------------------------------------------------------------------- */
#define UVMI_GEMM_STORE 0
#define UVMI_GEMM_SWIGLU 1
#define UVMI_GEMM_RESID 2
int uvmi_gemm_tn_supported(int dtype, int64_t M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int epilogue);
int uvmi_gemm_tn(const void* a, const void* w, void* c, int dtype, int64_t M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc,
                 int epilogue, void* stream);
/* The same GEMM with the two fusions that remove the residual-add + norm launch between a block's projections
 * (ultraviolet/model.py:567-571):
 *   epilogue UVMI_GEMM_RESID: C = ca * resid + cb * (A W^T), resid (M, N) in `dtype` with pitch ldr - the product is rounded
 *     to `dtype` first and the sum rounded again, as a GEMM followed by the residual-add kernel would;
 *   norm_a != 0: A stands for rmsnorm(A) (no weight, epsilon eps): the kernel sums the squares of its rows while they stream
 *     and scales the product by rsqrt(mean + eps); the normalised rows are neither written nor rounded to `dtype`.
 * Any epilogue combines with norm_a. */
typedef struct uvmi_gemm_args {
  const void* a; const void* w; void* c; int dtype;
  int64_t M; int N, K;
  int64_t lda, ldw, ldc;
  int epilogue;
  int norm_a; float eps;
  const void* resid; int64_t ldr; float ca, cb;
  int config;                              /* 0: built-in choice of the kernel form by size; 1: skinny, 64-row workgroups; 2: skinny,
                                              16-row workgroups whose waves split K (needs K % 128 == 0, else form 1); 3: tiled,
                                              128 x 128; 4: tiled, 64 x 64; 5: 256 x 256 tiles, 6: 128 x 128 tiles, both with slabs
                                              loaded straight into LDS (need K >= 128, C and resid 16-byte aligned, ldc,
                                              ldr % 8 == 0) - for tuning and tests */
} uvmi_gemm_args;
int uvmi_gemm_tn_ex(const uvmi_gemm_args* a, void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * Packed (cu_seqlens) causal self-attention with an optional sliding window over unquantized K/V: the attention of
 * a packed prefill.  Replaces varlen_attention (ultraviolet/kernels/varlen_attn.py:87-93, forward only) as called
 * by the packed prefill (ultraviolet/kernels/fast_decode.py:117-163, 210-269).
 * Query i of a segment sees keys j of the same segment with i - window < j <= i (window 0: every j <= i).
 * ---------------------------------------------------------------------------------------------------------- */
typedef struct uvmi_prefill_attn_args {
  const void* q; int q_dtype;              /* (N, H, hd) F16 / BF16, or F32 (generic kernel), inner stride 1 */
  int64_t sqn, sqh;                        /* strides in elements */
  const void* k; const void* v; int kv_dtype; /* (N, KH, hd) F16 / BF16 / F32, inner stride 1 */
  int64_t skn, skh, svn, svh;
  const void* cu_seqlens; int idx_dtype;   /* (n_seg + 1,) I32 / I64, non-decreasing, cu[0] = 0, cu[n_seg] = N */
  int n_seg;
  void* out; int out_dtype;                /* (N, H, hd) F16 / BF16 / F32, inner stride 1 */
  int64_t son, soh;
  int N, H, KH, hd;
  float scale;
  int window;
  void* workspace; size_t workspace_bytes; /* >= uvmi_prefill_attn_workspace_bytes(N): per-token segment table */
  int segments_ready;                      /* non-zero: the workspace already holds the table of these cu_seqlens (an earlier
                                              call with the same workspace, e.g. the previous layer's): skip building it */
  /* Optional fused epilogue, used when post_vhat != NULL (MFMA kernel only): Attention.post before the output projection
   * (ultraviolet/model.py:321-333), as in uvmi_attn_args: XSA z -= xsa[h] (z . v_hat) v_hat, then z *= gate[token][h]. */
  const float* post_vhat;                  /* (N, KH, hd) fp32 normalized v of every token (uvmi_qkv_post vhat_out) */
  const float* post_gate;                  /* (N, H) fp32 gate values (uvmi_qkv_post gate_out), or NULL */
  const float* post_xsa;                   /* (H,) tanh(alpha) fp32, or NULL */
} uvmi_prefill_attn_args;
/* The MFMA kernel runs when hd == 64, H / KH <= 8, q and k/v share a 16-bit dtype and rows are 16-byte aligned
 * (probabilities are rounded to that dtype for P.V, accumulation is fp32); anything else that uvmi_decode_attn's
 * generic kernel accepts runs there, token by token.  Two launches: the segment table (unless segments_ready), then the
 * attention. */
int uvmi_prefill_attn(const uvmi_prefill_attn_args* a, void* stream);
size_t uvmi_prefill_attn_workspace_bytes(int N);
/* 1 = MFMA kernel, 0 = generic kernel, negative = unsupported */
int uvmi_prefill_attn_path(const uvmi_prefill_attn_args* a);

/* Backward of uvmi_prefill_attn: replaces mathk::varlen_attn_bwd (ultraviolet/kernels/varlen_attn.py:56-66, the
 * aten._efficient_attention_backward call with K / V expanded to the query heads and their gradients summed back over the
 * group).  All tensors contiguous: q, o, go, dq (N, H, hd); k, v, dk, dv (N, KH, hd), one 16-bit dtype, head_dim 64;
 * cu_seqlens (n_seg + 1,) as in the forward.  The row log-sum-exp is recomputed (the forward does not return it).  fp32
 * arithmetic on the vector units (a first, plain form: no matrix cores).  workspace: (2 N H) fp32 (lse and go . o). */
typedef struct uvmi_prefill_attn_bwd_args {
  const void* q; const void* k; const void* v; const void* o; const void* go; int dtype;
  void* dq; void* dk; void* dv;
  const void* cu_seqlens; int idx_dtype; int n_seg;
  int N, H, KH, hd;
  float scale;
  int window;                              /* 0 = none */
  void* workspace; size_t workspace_bytes; /* >= uvmi_prefill_attn_bwd_workspace_bytes(N, H) */
} uvmi_prefill_attn_bwd_args;
int uvmi_prefill_attn_bwd(const uvmi_prefill_attn_bwd_args* a, void* stream);
size_t uvmi_prefill_attn_bwd_workspace_bytes(int N, int H);

/* ------------------------------------------------------------------------------------------------------------
 * Fused softcap + categorical draw + behaviour log-prob.  Replaces fused_sample
 * (ultraviolet/kernels/fused_sample.py:68-77) and the torch.rand call feeding it (ultraviolet/perf.py:595).
 * ---------------------------------------------------------------------------------------------------------- */
struct uvmi_sample_commit;
typedef struct uvmi_sample_args {
  const void* x; int x_dtype;      /* (B, V) raw head output before the softcap; F16 / BF16 / F32 */
  int64_t stride;                  /* row stride of x */
  const float* u;                  /* (B,) uniforms in [0, 1), or NULL to draw them from Philox4x32-10 */
  uint64_t seed;                   /* Philox key when u == NULL */
  const int64_t* req_id;           /* (B,) counter word: request id of each row (u == NULL) */
  const int64_t* tok_idx;          /* (B,) counter word: index of the token being drawn (u == NULL) */
  int64_t* tok; float* logp;       /* (B,) outputs */
  float* u_out;                    /* optional (B,): the uniform that was used */
  int B, V;
  float cap_a, cap_b, cap_c;       /* softcap a * sigmoid((x + b) / c) */
  float temperature;               /* > 0 draws from softmax(z / T); <= 0 takes argmax (first maximal index) and
                                      logp is log softmax(z)[tok] */
  /* Truncated sampling, sample() of the reference (ultraviolet/model.py:1194-1211), for T > 0: top_k in 1..V-1 keeps the
   * tokens whose value is at least the k-th largest; top_p in (0, 1) then keeps the smallest prefix by probability whose
   * mass reaches top_p (ties of the last kept value all kept).  0 / anything outside (0, 1) switches the filter off.
   * logp stays the log-prob under the untruncated softmax, as the reference records it (model.py:1161-1169). */
  int top_k; float top_p;
  float* thr_out;                  /* optional (B,): the smallest kept exp((z - a) / T) (0 when nothing is filtered) */
  const struct uvmi_sample_commit* commit; /* optional: the rows are the dense rows of a decode step, and the launch also does
                                      uvmi_sched_commit_dense for them (declared with the slot table below) */
} uvmi_sample_args;
int uvmi_fused_sample(const uvmi_sample_args* a, void* stream);
/* Host-side Philox4x32-10 (Random123) for tests and host tooling: out[4] = philox(ctr[4], key[2]). */
void uvmi_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

/* ------------------------------------------------------------------------------------------------------------
 * Fused per-token kernels of the UV-50M step (everything between the GEMMs).  dtype is the activation type
 * (F16 / BF16 / F32).  eps is the RMSNorm epsilon: the reference calls F.rms_norm(x, eps=None)
 * (ultraviolet/model.py:190-191), whose default depends on the torch release (machine epsilon of the input dtype or of
 * fp32), so the caller passes the value its torch uses.
 * ---------------------------------------------------------------------------------------------------------- */

/* x = rmsnorm(table[tok]); n = rmsnorm(x).  Replaces rms_norm_(self.embed(idx)) and the first block's pre-norm
 * (ultraviolet/kernels/fast_decode.py:286, 305).  x_out may be NULL. */
int uvmi_embed_norm(const void* table, int dtype, int64_t vocab, const int64_t* tok, int64_t rows, int d, float eps,
                    void* x_out, void* n_out, void* stream);

/* h = a*x + b*y; n = rmsnorm(h).  Replaces the residual lambdas of Block.finish followed by the next pre-norm
 * (ultraviolet/model.py:567-571; fast_decode.py:305, 332).  h_out may be NULL. */
int uvmi_add_norm(const void* x, const void* y, int dtype, float a, float b, int64_t rows, int d, float eps,
                  void* h_out, void* n_out, void* stream);

/* Attention.qkv after the fused QKV GEMM (ultraviolet/model.py:310-319) plus the decode-time cache append
 * (fast_decode.py:291-294, 315-317) for n token rows: value-embedding gate on v, QK-norm, partial RoPE
 * (half-split pairing) at pos[r], q written in q_dtype for the attention kernel, k / v optionally written
 * unquantized (prefill attention, XSA) and quantized into the int8 cache at row rows[r], slot pos[r] (or
 * pos[r] % S when ring; on a ring only positions > last_pos[r] - S are written).  head_dim 64. */
typedef struct uvmi_qkv_post_args {
  const void* qkv; int dtype;          /* (n, (H + 2 KH) * hd): q heads, then k heads, then v heads */
  const void* xn;                      /* (n, d) normed block input (value-embedding gate reads xn[:, :ve_ch]) */
  const void* ve_table;                /* (vocab, KH * hd) value-embedding table, same dtype; NULL if !has_ve */
  const float* ve_gate;                /* (KH, ve_ch) fp32 */
  const int64_t* tok;                  /* (n,) token ids (value-embedding rows) */
  const int64_t* pos;                  /* (n,) absolute position of each token */
  const int64_t* rows;                 /* (n,) cache row of each token; NULL = identity */
  const int64_t* last_pos;             /* (n,) last position of the token's prompt, or NULL (decode rows) */
  const float* inv_freq;               /* (n_pairs,) RoPE frequencies, fp32 */
  void* q_out; int q_dtype;            /* (n, H, hd) F16, BF16 or F32 */
  void* k_out; void* v_out;            /* (n, KH, hd) in dtype, or NULL */
  int8_t* k_cache; int8_t* v_cache;    /* (B, KH, S, hd) or NULL (no append) */
  uint16_t* k_scale; uint16_t* v_scale;
  int64_t scb, sch, scs, ssb, ssh;     /* cache / scale strides */
  int64_t n, vocab;
  int H, KH, hd, d, ve_ch, n_pairs, S, ring, has_ve, rope;
  float eps;                           /* QK-norm epsilon */
  /* optional inputs of the attention kernel's fused epilogue (Attention.post, model.py:324-333) */
  const float* gate_w; int gate_ch;    /* (H, gate_ch) fp32 output-gate weights */
  float* gate_out;                     /* (n, H) fp32: 2 sigmoid(gate_w[h] . xn[:gate_ch]), rounded as in dtype; or NULL */
  float* vhat_out; float xsa_eps;      /* (n, KH, hd) fp32: v / max(|v|, xsa_eps); or NULL */
  /* optional: uvmi_rope_table's output in dtype's rounding for positions 0 .. rope_positions - 1; tokens at those positions
   * read their cos / sin from it (the same values the kernel would compute), others compute them */
  const float* rope_table; int rope_positions;
  /* optional: the projection output carries the gates' logits behind q, k, v, as the extended projection of the decode
   * step forms them (columns (H + 2 KH) * hd .. : H output-gate logits, then KH value-embedding gate logits, in dtype).
   * qkv_ld: row pitch of qkv in elements (0: (H + 2 KH) * hd).  ext_logits != 0: the logits are read from those columns
   * instead of being computed from xn, gate_w and ve_gate, which may then be NULL. */
  int64_t qkv_ld; int ext_logits;
} uvmi_qkv_post_args;
int uvmi_qkv_post(const uvmi_qkv_post_args* a, void* stream);

/* Attention.post before the output projection (ultraviolet/model.py:321-333): XSA z -= xsa[h] (z . v_hat) v_hat with
 * the unquantized current v (fp32), then z *= 2 sigmoid(gate_w[h] . xn[:gate_ch]).  xsa = tanh(alpha) (H,) fp32 or NULL;
 * gate_w (H, gate_ch) fp32 or NULL.  z (n, H, hd) in z_dtype (F16 / BF16 / F32); out (n, H * hd) in dtype. */
int uvmi_attn_post(const void* z, int z_dtype, const void* v, const void* xn, int dtype, const float* gate_w,
                   const float* xsa, float xsa_eps, int64_t n, int H, int KH, int hd, int d, int gate_ch, void* out,
                   void* stream);

/* SwiGLU after the fused gate/up GEMM (ultraviolet/model.py:388-391): out[r, j] = silu(gu[r, j]) * gu[r, f + j]. */
int uvmi_swiglu(const void* gu, int dtype, int64_t rows, int f, void* out, void* stream);

/* The same with the MLP's pre-norm folded in (ultraviolet/model.py:570 n = norm(h), then 388-391): gu (rows, 2 f) is the
 * gate/up product of the UN-normalised hidden h (rows, d); with rn[r] = rsqrt(mean(h[r]^2) + eps),
 * out[r, j] = silu(rn gu[r, j]) * (rn gu[r, f + j]) - the row scale commutes with the product, so the normalised hidden
 * is never written.  f % 8 == 0, d % 2 == 0. */
int uvmi_swiglu_norm(const void* gu, const void* h, int dtype, int64_t rows, int f, int d, float eps, void* out,
                     void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * On-device continuous batching: the slot table of generate_continuous (ultraviolet/model.py:1283-1350) and
 * StreamGen (scripts/rl_stream.py:55-146) kept in device memory.  All arrays are caller-owned.
 * ---------------------------------------------------------------------------------------------------------- */
typedef struct uvmi_sched_state {
  int64_t* slot_req;    /* (B,) request id bound to the slot, -1 = free */
  int64_t* slot_cnt;    /* (B,) tokens generated so far (the token drawn from the prefill counts) */
  int64_t* slot_limit;  /* (B,) length limit of the request */
  int64_t* slot_tok;    /* (B,) last sampled token = input of the next step */
  int64_t* pos;         /* (B,) next position to write (the KV state's pos) */
  int64_t* starts;      /* (B,) first valid position (the KV state's starts) */
  int32_t* out_tok;     /* (B, max_new) generated tokens per slot */
  float* out_lp;        /* (B, max_new) behaviour log-probs, or NULL */
  int64_t* done_req; int64_t* done_slot; int64_t* done_cnt; /* (done_cap,) completion records, appended in arrival order */
  int32_t* counters;    /* [0] active slots at the last compact, [1] completion records written, [2] bucket overflow flag */
  int64_t max_new; int64_t eos_id; /* eos_id < 0: none */
  int B; int done_cap;
  /* Device-side admission (optional; all NULL / 0 when the host chooses the slots itself).  slot_hold: a slot that retires
   * is held (1) until uvmi_sched_harvest has packed its output row, and only then becomes reusable - uvmi_sched_plan_admit
   * never hands out a held slot.  The admission queue is a ring of q_cap staged prompts, q_stride int64 each:
   * [length, request id, length limit, tokens ...]; q_ctl[0] = prompts staged so far (written by the host after the rows,
   * on the launch stream), q_ctl[1] = prompts admitted so far, q_ctl[2] = prompts admitted by the last plan. */
  int32_t* slot_hold; int64_t* q_buf; int64_t* q_ctl;
  int q_cap; int q_stride;
} uvmi_sched_state;

/* List the active slots (ascending) and gather their token, position, start, request id and token index into dense
 * arrays of length n_bucket; rows past the active count get slot -1 and zeros.  Replaces the host loop over rows of
 * rl_stream.py:105-124 and the device-built index tensors of fast_decode.py:126-134. */
int uvmi_sched_compact(const uvmi_sched_state* s, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c,
                       int64_t* starts_c, int64_t* req_c, int64_t* cnt_c, void* stream);
/* Scatter sampled tokens / log-probs into the slots' output rows, advance count and position, retire rows on EOS,
 * length limit or (retire_p > 0) a Philox Bernoulli draw keyed by (seed, request, token index), park retired rows at
 * position 0 and append completion records.  Replaces buf.scatter_ / cnt.add_ and the harvest test of
 * rl_stream.py:120-143, model.py:1321-1350. */
int uvmi_sched_commit(const uvmi_sched_state* s, int n_bucket, const int64_t* act_slot, const int64_t* new_tok,
                      const float* new_lp, float retire_p, uint64_t seed, void* stream);
/* uvmi_sched_commit that also carries the dense arrays of uvmi_sched_compact to the next step: a row that goes on gets
 * its new token, position + 1 and token index + 1 in place; a row that retires becomes padding where it stands (slot -1,
 * zeros).  The next step then runs on these arrays without a compaction; padding rows may sit between active ones, so
 * the bucket only has to be compacted again after an admission or when it is to shrink. */
int uvmi_sched_commit_dense(const uvmi_sched_state* s, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c,
                            int64_t* starts_c, int64_t* req_c, int64_t* cnt_c, const int64_t* new_tok,
                            const float* new_lp, float retire_p, uint64_t seed, void* stream);
/* uvmi_fused_sample's optional commit: row i of the sampler is dense row i of the step, and the thread that writes the
 * row's token and log-prob then commits them as uvmi_sched_commit_dense does (same retirement draw), which saves the
 * step a launch.  req_c / cnt_c may be the sampler's req_id / tok_idx arrays. */
typedef struct uvmi_sample_commit {
  const uvmi_sched_state* state;
  int64_t* act_slot; int64_t* tok_c; int64_t* pos_c; int64_t* starts_c; int64_t* req_c; int64_t* cnt_c;
  float retire_p; uint64_t seed;
} uvmi_sample_commit;

/* Bind n freshly prefilled requests to slots and record their first sampled token (model.py:1306-1313,
 * rl_stream.py:86-92). */
int uvmi_sched_admit(const uvmi_sched_state* s, int n, const int64_t* slots, const int64_t* req_ids,
                     const int64_t* limits, const int64_t* first_tok, const float* first_lp, void* stream);

/* Per-token tables of the prompts admitted with a step, built on the device from their cu_seqlens (n_adm + 1 entries,
 * non-decreasing; unused trailing entries repeat the total): for packed token i of prompt a, pos_t = adm_start[a] + i -
 * cu[a], row_t = adm_slot[a], last_t = last position of the prompt; tokens at or after cu[n_adm], and prompts with
 * adm_slot < 0, are padding (row -1).  last_idx[a] = packed index of prompt a's last token (0 if unused).  Also sets
 * starts / pos of the admitted slots.  Replaces the host-built index tensors of prefill_packed_host
 * (ultraviolet/kernels/fast_decode.py:210-269) so that a step that admits prompts can be captured in a graph. */
int uvmi_sched_expand(const uvmi_sched_state* s, int n_adm, int n_tokens, const int64_t* cu_seqlens, const int64_t* adm_slot,
                      const int64_t* adm_start, int64_t* pos_t, int64_t* row_t, int64_t* last_t, int64_t* last_idx, void* stream);

/* The admission of a step decided on the device - the free-slot choice and the FIFO queue that the reference keeps in
 * host Python (StreamGen._refill, scripts/rl_stream.py:76-93; generate_continuous' refill, ultraviolet/model.py:1293-1314).
 * Takes prompts from the head of the staged ring while a reusable slot (slot_req < 0, not held) is left, at most admit_cap
 * prompts and n_tokens packed tokens, and binds them to the free slots in ascending slot order.  Writes the step's admission
 * tables - cu_seqlens (admit_cap + 1 entries, unused ones repeat the total), slot (-1 unused), start position (left_pad:
 * longest admitted prompt - own length, else 0), length limit and request id per prompt - and the prompts' tokens packed
 * back to back into tok_packed (n_tokens entries, zero filled), then advances q_ctl[1].  The tables are what
 * uvmi_sched_expand and uvmi_sched_admit take, so a step that admits prompts needs nothing from the host but the launch.
 * One workgroup. */
int uvmi_sched_plan_admit(const uvmi_sched_state* s, int admit_cap, int n_tokens, int left_pad, int64_t* adm_cu, int64_t* adm_slot,
                          int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req, int64_t* tok_packed, void* stream);

/* uvmi_sched_compact, uvmi_sched_plan_admit and uvmi_sched_expand of a step that admits prompts in one launch (one
 * workgroup): everything the step's kernels need - the dense arrays of the decode rows, the admission tables, the packed
 * prompt tokens and their per-token position / cache row / last position tables - without a word from the host.
 * last_c (optional, n_bucket entries): the decode rows' positions once more, as the "last position" column of a pass
 * that runs prompt tokens and decode rows together. */
int uvmi_sched_step_plan(const uvmi_sched_state* s, int n_bucket, int64_t* act_slot, int64_t* tok_c, int64_t* pos_c, int64_t* starts_c,
                         int64_t* req_c, int64_t* cnt_c, int admit_cap, int n_tokens, int left_pad, int64_t* adm_cu, int64_t* adm_slot,
                         int64_t* adm_start, int64_t* adm_limit, int64_t* adm_req, int64_t* tok_packed, int64_t* pos_t, int64_t* row_t,
                         int64_t* last_t, int64_t* last_idx, int64_t* last_c, void* stream);

/* Pack the completion records seen .. min(seen + max_rows, counters[1]) - 1 (seen = records the host has already taken)
 * and the output rows of their slots, so that the host harvests with one copy of the header and one of exactly the
 * finished tokens.  hdr (8 + 4 max_rows int64): [0..2] = counters[0..2], [3] = k, the records packed; then for packed
 * record j: request id, slot, token count (clamped to max_new), offset of its tokens in tok_dst / lp_dst (rows back to
 * back in record order); after the records, at 4 + 4 max_rows: the number of active slots at this point of the stream,
 * q_ctl[1] and q_ctl[2] (0 without a queue).  With slot_hold the packed slots are released for reuse.  tok_dst, lp_dst: max_rows * max_new elements; lp_dst may be NULL.  Replaces the whole-buffer
 * .cpu() and the host loop over rows of StreamGen.chunk (scripts/rl_stream.py:126-143; ultraviolet/model.py:1321-1335). */
int uvmi_sched_harvest(const uvmi_sched_state* s, int64_t seen, int max_rows, int64_t* hdr, int32_t* tok_dst,
                       float* lp_dst, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* UVMI_H */
