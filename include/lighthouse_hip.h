/*
 * lighthouse_hip.h -- C ABI of liblighthouse_hip.so, the MI355X (gfx950) runtime
 * target for Lighthouse's GPU payloads.
 *
 * Lighthouse's Runner JIT-compiles a payload module and calls the resulting native
 * symbol through ctypes with "packed" arguments (lighthouse/execution/runner.py:
 * 196-215): one void* per argument, each pointing at a pointer to a ranked memref
 * descriptor {allocated, aligned, offset, sizes[rank], strides[rank]} with strides
 * in ELEMENTS (lighthouse/utils/memref.py:5-44, lighthouse/utils/torch.py:41-66),
 * or at an int64 for scalars.  This library offers the same calling convention for
 * hand-written kernels instead of JIT'd code (the lh_hip_payload_* functions), plus
 * the plain pointer/size form underneath (lh_hip_gemm, lh_hip_attention, ...), plus
 * the device-memory helpers that replace the JIT'd gpu_alloc/gpu_dealloc/gpu_copy
 * functions of lighthouse/ingress/mlir_gen/gpu_utils.py:6-45.
 *
 * Conventions
 *  - Every function returns 0 on success or a negative lh_status; the message of the
 *    last failure on the calling thread is lh_hip_last_error().  No C++ exception
 *    crosses this boundary.  (The reference's JIT'd functions return void and cannot
 *    report errors; the Python wrapper maps these codes to ValueError/RuntimeError as
 *    lighthouse/execution/runner.py:113,175,179,191 do.)
 *  - All data pointers are DEVICE pointers unless a parameter is named host_*.
 *  - `stream` is a hipStream_t passed as void*; NULL selects the default stream.
 *    Plain-pointer entry points only enqueue work; lh_hip_payload_* entry points
 *    return after the work has finished, like a JIT'd payload call does.
 *  - The caller owns every buffer; no entry point allocates results
 *    (lighthouse/dialects/transform/transform_ext/ops/convert_func_results_to_args.py:14-24).
 *  - Matrices are row-major; `ld*` are leading dimensions in elements.
 *  - Temporary device memory: a few problems need more than their operands (transposed or unaligned
 *    operands run on copies, short-and-wide "decode" problems are cut along K into f32 blocks that a
 *    second kernel adds up).  The plain entry points take it from a pool the library keeps per
 *    (device, stream): calls on different streams never share it, it only grows, and nothing is
 *    freed inside a call (lh_hip_release_scratch() returns it).  The *_ws entry points and the
 *    nanoGPT entry points take a caller workspace instead and never allocate
 *    (lighthouse/dialects/transform/transform_ext/ops/convert_func_results_to_args.py:14-24: the
 *    callee does not allocate).
 */
#ifndef LIGHTHOUSE_HIP_H
#define LIGHTHOUSE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum lh_status {
  LH_OK = 0,
  LH_ERR_INVALID = -1,     /* bad shape / stride / flag / null pointer  -> ValueError   */
  LH_ERR_UNSUPPORTED = -2, /* valid request with no kernel              -> ValueError   */
  LH_ERR_RUNTIME = -3      /* HIP runtime failure                       -> RuntimeError */
} lh_status;

/* Element types (the MLIR element types the payload generators accept). */
typedef enum lh_dtype {
  LH_F32 = 0,
  LH_BF16 = 1,
  LH_F16 = 2,
  LH_F8E4M3 = 3, /* OCP e4m3fn */
  LH_F64 = 4,
  LH_I8 = 5,
  LH_I16 = 6,
  LH_I32 = 7,
  LH_I64 = 8
} lh_dtype;

/* GEMM epilogue / layout flags; names follow generate_gpu_matmul_payload's keyword
 * arguments (lighthouse/ingress/mlir_gen/gpu_matmul_payload.py:5-36). */
#define LH_GEMM_HAS_BIAS 1u
#define LH_GEMM_HAS_RELU 2u
#define LH_GEMM_ACCUMULATE_C 4u
#define LH_GEMM_TRANSPOSE_A 8u
#define LH_GEMM_TRANSPOSE_B 16u
#define LH_GEMM_HAS_GELU 32u /* tanh-GELU on the accumulator instead of ReLU (nanoGPT MLP) */
/* Workgroup-tile request, the counterpart of the wg_m / wg_n schedule parameters
 * (lighthouse/schedule/xegpu/mlp_schedule.py:72-78,142).  AUTO lets the library pick by shape.
 * 16-bit inputs take 256x256, 256x128, 128x256 and 128x128: the tile must divide M and N and
 * needs an untransposed A (B may be stored transposed: the kernels read an [N, K] matrix with
 * aligned rows in place), K % 64 == 0 and 16-byte aligned rows.  f32 inputs take 128x128,
 * 128x64 and 64x64 (M and N need not be multiples): untransposed operands, K % 32 == 0, N % 4 == 0
 * and 16-byte aligned rows.  A request the problem does not meet fails with LH_ERR_INVALID. */
#define LH_GEMM_TILE_MASK 0x700u
#define LH_GEMM_TILE_AUTO 0x000u
#define LH_GEMM_TILE_256x256 0x100u
#define LH_GEMM_TILE_256x128 0x200u
#define LH_GEMM_TILE_128x256 0x300u
#define LH_GEMM_TILE_128x128 0x400u
#define LH_GEMM_TILE_128x64 0x500u
#define LH_GEMM_TILE_64x64 0x600u
/* Cut along K for the 16-bit GEMM ("split K": `splits` workgroup sets each take K / splits columns
 * of A and rows of B and write an f32 block; a second kernel adds the blocks and runs the
 * epilogue), for problems with too few tiles to fill the CUs; the k-dimension counterpart of the
 * tile request above (lighthouse/schedule/xegpu/matmul_params.json holds such per-shape choices).
 * AUTO lets the library decide; NONE forbids the cut; 2 / 4 / 8 request it and need an untransposed A,
 * aligned operands and K / splits a multiple of 64 (runs on 128 x 128 tiles, so it excludes a tile
 * request). */
#define LH_GEMM_SPLITK_MASK 0x3800u
#define LH_GEMM_SPLITK_AUTO 0x0000u
#define LH_GEMM_SPLITK_NONE 0x0800u
#define LH_GEMM_SPLITK_2 0x1000u
#define LH_GEMM_SPLITK_4 0x1800u
#define LH_GEMM_SPLITK_8 0x2000u

/* ---------------------------------------------------------------- runtime ---- */

/* Message of the last error raised on this thread ("" if none). */
const char* lh_hip_last_error(void);

typedef struct lh_device_info {
  char arch[64];            /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
  char name[128];
  int32_t compute_units;
  int32_t clock_khz;        /* engine clock */
  int32_t memory_clock_khz;
  int32_t memory_bus_bits;
  int32_t lds_bytes_per_cu; /* max shared memory per block */
  int32_t wavefront_size;
  int64_t hbm_bytes;
} lh_device_info;

/* Replaces nothing in the reference; feeds the roofline report
 * (the reference keeps vendor constants in lighthouse/schedule/xegpu/xegpu_specs.py:20-35). */
int lh_hip_device_info(lh_device_info* out);
int lh_hip_device_count(int32_t* out);

/* Device memory: replace gpu_alloc_* / gpu_dealloc_* / gpu_copy_* helpers that
 * GPUMemoryManager invokes (lighthouse/execution/memory_manager.py:97-151). */
int lh_hip_alloc(void** dev_ptr, size_t bytes);
int lh_hip_free(void* dev_ptr);
int lh_hip_memcpy_h2d(void* dev_dst, const void* host_src, size_t bytes);
int lh_hip_memcpy_d2h(void* host_dst, const void* dev_src, size_t bytes);
int lh_hip_memcpy_d2d(void* dev_dst, const void* dev_src, size_t bytes);
int lh_hip_memset(void* dev_ptr, int value, size_t bytes);
int lh_hip_sync(void* stream);
/* Waits for the current device and frees the library's pool of temporary buffers on it (no
 * counterpart in the reference, whose JIT'd code frees its temporaries itself:
 * examples/xegpu/nanoGPT_payload.py:407-408). */
int lh_hip_release_scratch(void);

/* --------------------------------------------------- plain pointer kernels ---- */

/*
 * out[M,N] = epilogue(A.B) ; the matmul/MLP-layer payload, emit_mlp_layer
 * (lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:110-156): f32 accumulation from 0 or
 * from `out` (ACCUMULATE_C), + bias[n] extended to f32, conversion to out_dtype, then
 * ReLU.  A is [M,K] (or [K,M] with TRANSPOSE_A), B is [K,N] (or [N,K] with TRANSPOSE_B).
 * ab_dtype in {F32, BF16, F16}; out_dtype F32 or ab_dtype; bias has out_dtype.
 */
int lh_hip_gemm(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
                int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype, uint32_t flags,
                void* stream);

/*
 * lh_hip_gemm with its temporary memory in a caller workspace of at least
 * lh_hip_gemm_workspace_bytes(...) bytes (0 for most problems; the query assumes 16-byte aligned
 * operands).  No allocation happens inside the call; a workspace that is too small fails with
 * LH_ERR_INVALID.  Same role as the workspace of lh_hip_nanogpt_block for callers that manage
 * device memory themselves (GPUMemoryManager, lighthouse/execution/memory_manager.py:97-151).
 */
size_t lh_hip_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                   int32_t ab_dtype, int32_t out_dtype, uint32_t flags);
/*
 * The same query for given operands: an operand that is not 16-byte aligned runs on a padded copy in
 * the workspace, which this variant counts (the pointers are not dereferenced).  lh_hip_gemm_ws and
 * lh_hip_gemm_static compute their need this way and refuse before anything is launched.
 */
size_t lh_hip_gemm_workspace_bytes_for(const void* out, const void* a, const void* b, const void* bias, int64_t M,
                                       int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype,
                                       int32_t out_dtype, uint32_t flags);
int lh_hip_gemm_ws(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype, uint32_t flags,
                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * lh_hip_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, kernels and results as lh_hip_gemm; the temporary memory of the problems that need
 * any (f32 blocks of decode shapes cut along K, copies of transposed or unaligned operands) is a
 * device array of LH_STATIC_SCRATCH_BYTES that is part of the library's device image, so the call
 * performs no hipMalloc / hipFree and uses no allocating library routine.  A problem whose
 * temporaries exceed that size is refused with LH_ERR_INVALID before anything is launched.
 * Nothing in the array needs clearing between calls (every kernel writes what it later reads).
 * All calls on one GPU share the array: calls that overlap in time on one GPU (different streams
 * or threads) race; calls on one stream are safe.
 */
#define LH_STATIC_SCRATCH_BYTES (16u << 20)
int lh_hip_gemm_static(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype, uint32_t flags,
                       void* stream);

/*
 * lh_hip_gemm whose accumulation starts from a separate matrix: out = epilogue(c + A.B), with
 * `c` [M,N] of out_dtype and row stride ldc (ACCUMULATE_C is implied; c may be `out`, which is
 * lh_hip_gemm with the flag).  This is emit_mlp_layer's `acc_tensor` argument in its general
 * form (lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:115,124-127,144); the payload generator
 * itself only ever passes the output matrix (gpu_mlp_payload.py:83-95).  It is what a residual
 * connection x + linear(y) needs when x must survive: the torch ingress lowers that pattern to
 * one call, and the nanoGPT block kernel sequence uses it internally.
 */
int lh_hip_gemm_residual(void* out, const void* c, const void* a, const void* b, const void* bias, int64_t M,
                         int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype,
                         int32_t out_dtype, uint32_t flags, void* stream);

/*
 * fp8 GEMM of the benchmark's quantised configuration (no counterpart in the
 * reference): out[M,N] = out_dtype( (Aq.Bq)_f32 * (scale_a*scale_b) ), Aq [M,K] and
 * Bq [K,N] hold OCP e4m3fn codes; out_dtype BF16 or F32.
 */
int lh_hip_gemm_fp8(void* out, const void* a_q, const void* b_q, float scale_a, float scale_b, int64_t M,
                    int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t out_dtype, void* stream);
/* The same with a caller workspace (see lh_hip_gemm_ws); the decode shapes (M <= 128) always need one. */
size_t lh_hip_gemm_fp8_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                       int32_t out_dtype);
int lh_hip_gemm_fp8_ws(void* out, const void* a_q, const void* b_q, float scale_a, float scale_b, int64_t M,
                       int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t out_dtype,
                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * Fused attention forward, the payload of generate_gpu_attention_payload
 * (lighthouse/ingress/mlir_gen/gpu_attention_payload.py:12-132) in the fused form of
 * ReplaceWithFusedAttentionOp (lighthouse/dialects/transform/transform_ext/ops/
 * replace_with_fused_attention.py:332-455): O = softmax(Q K^T * scale [+ causal mask]) V
 * with f32 running max / sum / accumulator.  Tensors are [Z,H,T,d] with element strides
 * (sz, sh, st) per tensor and unit stride along d, so (T, H*d) projection buffers can be
 * passed as strided views without a copy (examples/xegpu/nanoGPT_payload.py:198-217).
 * dtype in {BF16, F16, F32}; 1 <= d <= 256, any T.  Every problem runs on the matrix cores: with
 * 16-byte accesses when rows are 16-byte aligned and d is a multiple of 8 (16-bit) or 4 (f32), with
 * element accesses otherwise.  A 16-bit problem with few query blocks and a long sequence (fewer
 * 128-row blocks than compute units) has the key range of every block split between workgroups;
 * the partial results (68 KiB per workgroup, at most 35 MiB) live in the library's pool of
 * temporary buffers of the stream, like the K-cut blocks of lh_hip_gemm.  The nanoGPT block and
 * forward entry points, which run on the caller's workspace only, never take that path.
 */
/* `causal` is a word of flags: bit 0 selects the causal mask; the other bits request a kernel
 * variant for 16-bit tensors with head dimension 64, the counterpart of the wg_rows / sg_rows
 * parameters of the reference's fused-attention schedule (examples/xegpu/fused_attention.py:109-145,
 * lighthouse/schedule/xegpu/fused_attention_schedule.py): query rows per wave (64: two 32-row
 * sub-tiles share every K/V fragment, 256-row workgroups; 32: 128-row workgroups, twice as many)
 * and, for the 32-row kernel, the depth of the K/V ring (3 stages: three workgroups per CU; 4: two);
 * LH_ATTN_KSPLIT_2 gives a workgroup of the 64-row kernel two groups of four waves that walk the two
 * halves of the key range side by side and are combined at the end (LH_ATTN_KSPLIT_1: never).
 * 0 lets the library choose by shape.  A request that does not apply fails with LH_ERR_INVALID.
 * LH_ATTN_SCALE_F32 selects where the softmax scale is applied: by default Q is multiplied by
 * scale * log2(e) once and rounded to the element type again (one rounding more than the reference,
 * inside every tolerance of the payload); with this bit Q stays as stored and every score is scaled in
 * f32, as ReplaceWithFusedAttentionOp does (replace_with_fused_attention.py:386), at one more
 * vector instruction per score (about 7 % of the time at [4,16,2048,64]).  The f32 kernel always
 * scales in f32. */
#define LH_ATTN_CAUSAL 0x1
#define LH_ATTN_ROWS_MASK 0x300
#define LH_ATTN_ROWS_32 0x100
#define LH_ATTN_ROWS_64 0x200
#define LH_ATTN_STAGES_MASK 0xC00
#define LH_ATTN_STAGES_3 0x400
#define LH_ATTN_STAGES_4 0x800
#define LH_ATTN_KSPLIT_MASK 0x3000
#define LH_ATTN_KSPLIT_1 0x1000
#define LH_ATTN_KSPLIT_2 0x2000
#define LH_ATTN_SCALE_F32 0x4000
typedef struct lh_strides3 {
  int64_t z, h, t;
} lh_strides3;
int lh_hip_attention(void* out, const void* q, const void* k, const void* v, int64_t Z, int64_t H, int64_t T,
                     int64_t d, lh_strides3 so, lh_strides3 sq, lh_strides3 sk, lh_strides3 sv, float scale,
                     int32_t causal, int32_t dtype, void* stream);
/*
 * lh_hip_attention with its temporary memory in a caller workspace (256-byte aligned) of at least
 * lh_hip_attention_workspace_bytes(...) bytes, for callers that cannot let the library allocate:
 * the only temporaries of an attention call are the partial results of a key range split between
 * workgroups, which the library chooses for 16-bit problems with few query blocks and long
 * sequences (0 bytes for every other problem, the benchmark's among them; a call that requests
 * LH_ATTN_KSPLIT_1, a row count or a ring depth never splits and needs none).  A workspace that is
 * too small fails with LH_ERR_INVALID before anything is launched.  No counterpart in the
 * reference, whose payloads receive every buffer as an argument (lighthouse/execution/runner.py:196-215).
 */
size_t lh_hip_attention_workspace_bytes(int64_t Z, int64_t H, int64_t T, int64_t d, lh_strides3 so, lh_strides3 sq,
                                        lh_strides3 sk, lh_strides3 sv, int32_t causal, int32_t dtype);
int lh_hip_attention_ws(void* out, const void* q, const void* k, const void* v, int64_t Z, int64_t H, int64_t T,
                        int64_t d, lh_strides3 so, lh_strides3 sq, lh_strides3 sk, lh_strides3 sv, float scale,
                        int32_t causal, int32_t dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Row LayerNorm, emit_layer_norm_generics
 * (lighthouse/ingress/mlir_gen/gpu_layer_norm_payload.py:15-87): x [M,N] (x_dtype F32 or
 * BF16), gamma/beta [N] f32, statistics in f32, out [M,N] in out_dtype (F32, BF16 or, from an
 * F32 input, F16; a 16-bit output fuses the cast that follows every LayerNorm in
 * examples/xegpu/nanoGPT_payload.py:299-317).
 */
int lh_hip_layer_norm(void* out, const void* x, const float* gamma, const float* beta, int64_t M, int64_t N,
                      float eps, int32_t x_dtype, int32_t out_dtype, void* stream);

/* Row softmax, generate_gpu_softmax_payload (lighthouse/ingress/mlir_gen/gpu_softmax_payload.py:11-65). */
int lh_hip_softmax(void* out, const void* x, int64_t M, int64_t N, int32_t dtype, void* stream);

/* Elementwise kernels of the nanoGPT payload builder (examples/xegpu/nanoGPT_payload.py:123-181). */
/* out = tanh-GELU(x), n elements (no counterpart in the reference; benchmark's MLP activation). */
int lh_hip_gelu_tanh(void* out, const void* x, int64_t n, int32_t dtype, void* stream);
/* out[m,n] = x[m,n] + bias[n], optional ReLU (Builder.bias :141-163). x, bias, out share dtype. */
int lh_hip_bias_act(void* out, const void* x, const void* bias, int64_t M, int64_t N, int32_t relu,
                    int32_t dtype, void* stream);
/* out = a + b (Builder.add :166-181). */
int lh_hip_add(void* out, const void* a, const void* b, int64_t n, int32_t dtype, void* stream);
/* out = convert(x) between F32/BF16/F16 (Builder.cast_f16 :123-138). */
int lh_hip_cast(void* out, const void* x, int64_t n, int32_t src_dtype, int32_t dst_dtype, void* stream);

/*
 * One pre-LayerNorm GPT-2 block forward, the op sequence of _emit_block_fused
 * (examples/xegpu/nanoGPT_payload.py:299-317): ln1 -> q,k,v projections -> fused attention on
 * (H, T, hs) views -> output projection + bias + residual -> ln2 -> MLP up-projection + bias +
 * activation -> down-projection + bias + residual.  x, y: [B*T, C] f32 residual stream.  Weights are
 * stored [in, out] in `dtype` (F32, BF16 or F16: every matmul input is rounded to it, the rounding
 * points of examples/xegpu/nanoGPT.py:114-126); LayerNorm parameters are f32.
 *
 * Two configurations are covered by `opts` and the parameter struct:
 *  - the benchmark's (opts == NULL): one fused QKV projection [C, 3C] with bias, causal mask,
 *    tanh-GELU, biases of `dtype`;
 *  - the reference's own (examples/xegpu/nanoGPT_payload.py:299-317,333-346): separate w_q / w_k /
 *    w_v [C, C] without bias (w_qkv == NULL), no mask, ReLU, f32 biases.
 * Any bias pointer may be NULL (no bias).  `workspace` must hold
 * lh_hip_nanogpt_block_workspace_bytes(...) bytes; the call allocates nothing.
 */
typedef struct lh_nanogpt_block_params {
  const float* ln1_g;
  const float* ln1_b;
  const void* w_qkv; /* [C, 3C], or NULL with w_q, w_k, w_v set */
  const void* b_qkv; /* [3C] (q | k | v), or NULL */
  const void* w_o;   /* [C, C]  */
  const void* b_o;   /* [C]     */
  const float* ln2_g;
  const float* ln2_b;
  const void* w_fc;   /* [C, hidden] */
  const void* b_fc;   /* [hidden]    */
  const void* w_proj; /* [hidden, C] */
  const void* b_proj; /* [C]     */
  const void* w_q;    /* [C, C] each; used when w_qkv is NULL */
  const void* w_k;
  const void* w_v;
} lh_nanogpt_block_params;
typedef enum lh_activation {
  LH_ACT_GELU_TANH = 0, /* benchmark configuration */
  LH_ACT_RELU = 1       /* Builder.bias(relu=True), examples/xegpu/nanoGPT_payload.py:311 */
} lh_activation;
typedef struct lh_nanogpt_block_opts {
  int32_t causal;     /* 1: causal mask; 0: none (the reference's fused kernel) */
  int32_t activation; /* lh_activation */
  int32_t bias_dtype; /* type of every bias vector: `dtype` or LH_F32 */
  int32_t hidden;     /* MLP width; 0 selects 4 C */
} lh_nanogpt_block_opts;
size_t lh_hip_nanogpt_block_workspace_bytes(int64_t B, int64_t T, int64_t C, int32_t dtype,
                                            const lh_nanogpt_block_opts* opts);
int lh_hip_nanogpt_block(float* y, const float* x, const lh_nanogpt_block_params* p, int64_t B, int64_t T,
                         int64_t C, int64_t n_head, float eps, int32_t dtype, const lh_nanogpt_block_opts* opts,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * n_layer blocks followed by the final LayerNorm and the lm_head projection with bias, the shape
 * of build_gpt_fused_payload (examples/xegpu/nanoGPT_payload.py:318-407; embeddings stay on the
 * host side there too): logits[B*T, vocab] (f32) = LN_f(block_n(...block_1(x))) W_lm + b_lm.
 * Blocks are lh_hip_nanogpt_block's; lm_w [C, vocab] has `dtype`, lm_b [vocab] (or NULL) the bias
 * type of `opts`.  `workspace` must hold lh_hip_nanogpt_forward_workspace_bytes(...) bytes.
 */
size_t lh_hip_nanogpt_forward_workspace_bytes(int64_t B, int64_t T, int64_t C, int64_t vocab, int32_t dtype,
                                              const lh_nanogpt_block_opts* opts);
int lh_hip_nanogpt_forward(float* logits, const float* x, const lh_nanogpt_block_params* blocks, int64_t n_layer,
                           const float* lnf_g, const float* lnf_b, const void* lm_w, const void* lm_b, int64_t B,
                           int64_t T, int64_t C, int64_t n_head, int64_t vocab, float eps, int32_t dtype,
                           const lh_nanogpt_block_opts* opts, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------- packed-argument payloads ---- */

/*
 * The calling convention of a JIT'd `payload` symbol: args[i] points at a pointer to the
 * i-th memref descriptor, output first (lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:44-48,
 * gpu_attention_payload.py:48-50, gpu_layer_norm_payload.py:122-124).  A memref descriptor
 * carries no element type (lighthouse/execution/memory_manager.py:112), so each payload
 * takes an attribute struct with the types and options its generator was called with.
 * These functions validate shapes and strides, run on the library's stream and return
 * after the device finished.
 */
typedef struct lh_matmul_attrs {
  int32_t ab_dtype;
  int32_t out_dtype;
  uint32_t flags; /* LH_GEMM_* */
} lh_matmul_attrs;
/* args: out[M,N], A, B[, bias[N]] */
int lh_hip_payload_matmul(void** args, int32_t nargs, const lh_matmul_attrs* attrs);

/* Multi-layer perceptron, generate_gpu_mlp_payload
 * (lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:10-107): layer i computes
 * epilogue(act_i . W_i) with the matmul payload's epilogue; hidden activations have the A/B type
 * and get the ReLU, the last layer has out_dtype and gets the ReLU only when
 * relu_on_final_layer is set; TRANSPOSE_A applies to the first layer's input only,
 * ACCUMULATE_C to the last layer's output only (the reference accumulates hidden layers into
 * uninitialised tensors, i.e. leaves them undefined).  Hidden activations live in the library's
 * pool of temporary buffers. */
typedef struct lh_mlp_attrs {
  int32_t ab_dtype;
  int32_t out_dtype;  /* result type of the last layer: F32 or the A/B type */
  int32_t bias_dtype; /* type of every bias vector: F32 or the A/B type */
  uint32_t flags;     /* LH_GEMM_HAS_BIAS | HAS_RELU | ACCUMULATE_C | TRANSPOSE_A | TRANSPOSE_B */
  int32_t nlayers;
  int32_t relu_on_final_layer;
} lh_mlp_attrs;
/* args: out[M,N_last], in, W_0 .. W_{n-1}[, bias_0 .. bias_{n-1}] */
int lh_hip_payload_mlp(void** args, int32_t nargs, const lh_mlp_attrs* attrs);

typedef struct lh_matmul_fp8_attrs {
  int32_t out_dtype;
  float scale_a;
  float scale_b;
} lh_matmul_fp8_attrs;
/* args: out[M,N], Aq[M,K], Bq[K,N] */
int lh_hip_payload_matmul_fp8(void** args, int32_t nargs, const lh_matmul_fp8_attrs* attrs);

typedef struct lh_attention_attrs {
  int32_t dtype;
  int32_t causal; /* LH_ATTN_CAUSAL | variant request bits, as for lh_hip_attention */
  float scale; /* <= 0 selects 1/sqrt(d) */
} lh_attention_attrs;
/* args: out, Q, K, V, each rank-4 [Z,H,T,d] */
int lh_hip_payload_attention(void** args, int32_t nargs, const lh_attention_attrs* attrs);

typedef struct lh_layer_norm_attrs {
  int32_t x_dtype;
  int32_t out_dtype;
  float eps;
} lh_layer_norm_attrs;
/* args: out[M,N], x[M,N], gamma[N], beta[N] */
int lh_hip_payload_layer_norm(void** args, int32_t nargs, const lh_layer_norm_attrs* attrs);

typedef struct lh_elementwise_attrs {
  int32_t kind;      /* lh_elementwise_kind */
  int32_t dtype;     /* element type of the operands */
  int32_t dst_dtype; /* CAST only */
  int32_t relu;      /* BIAS only */
} lh_elementwise_attrs;
typedef enum lh_elementwise_kind {
  LH_EW_SOFTMAX = 0, /* args: out[M,N], x[M,N] */
  LH_EW_GELU = 1,    /* args: out, x */
  LH_EW_BIAS = 2,    /* args: out[M,N], x[M,N], bias[N] */
  LH_EW_ADD = 3,     /* args: out, a, b */
  LH_EW_CAST = 4     /* args: out, x */
} lh_elementwise_kind;
int lh_hip_payload_elementwise(void** args, int32_t nargs, const lh_elementwise_attrs* attrs);

typedef struct lh_nanogpt_block_attrs {
  int32_t dtype; /* F32, BF16 or F16: type of the weights and matmul inputs */
  int32_t n_head;
  int32_t B;
  int32_t T;
  float eps;
} lh_nanogpt_block_attrs;
/* The benchmark's block.  args: y[B*T,C], x[B*T,C], ln1_g[C], ln1_b[C], w_qkv[C,3C], b_qkv[3C], w_o[C,C],
 * b_o[C], ln2_g[C], ln2_b[C], w_fc[C,4C], b_fc[4C], w_proj[4C,C], b_proj[C], workspace[bytes] (i8). */
int lh_hip_payload_nanogpt_block(void** args, int32_t nargs, const lh_nanogpt_block_attrs* attrs);

/*
 * The payload of build_gpt_fused_payload (examples/xegpu/nanoGPT_payload.py:318-407) with its own
 * argument list, so that the reference's nanoGPT driver (examples/xegpu/nanoGPT.py:225-297) can
 * call it with the buffers it already builds: out[T,vocab] f32, x[T,C] f32, then per layer
 * g1[C], b1n[C], wq[C,C], wk[C,C], wv[C,C], wp[C,C], bp[C], g2[C], b2n[C], w1[C,hidden], bb1[hidden],
 * w2[hidden,C], bb2[C] (:333-347), then gf_g[C], gf_b[C], lmw[C,vocab], lmb[vocab], and last a
 * workspace[bytes] (i8) of lh_hip_nanogpt_forward_workspace_bytes(1, T, C, vocab, dtype, &opts)
 * with opts = {causal, LH_ACT_RELU, LH_F32, hidden} (the reference frees its temporaries inside the
 * payload, :407-408; here the caller provides them).  Weights have `dtype` (the reference: F16),
 * LayerNorm parameters and biases are f32.  Non-causal unless `causal` is set.
 */
typedef struct lh_gpt_fused_attrs {
  int32_t dtype;
  int32_t n_head;
  int32_t n_layer;
  int32_t causal;
  float eps;
} lh_gpt_fused_attrs;
int lh_hip_payload_gpt_fused(void** args, int32_t nargs, const lh_gpt_fused_attrs* attrs);

/*
 * The `__benchmark` wrapper (WrapInBenchingFuncOp, lighthouse/dialects/transform/
 * transform_ext/ops/wrap_in_benching_func.py:29-65): calls the payload `nwarmup` times
 * untimed, then `nruns` times, each bracketed by a wall clock read with the device idle
 * on both sides; the durations in seconds go to host_times[0..nruns).  `payload` selects
 * the entry point by its name without the "lh_hip_payload_" prefix ("matmul",
 * "matmul_fp8", "attention", "layer_norm", "elementwise", "nanogpt_block", "mlp", "gpt_fused"); `attrs` is that entry point's
 * attribute struct.
 */
int lh_hip_payload_benchmark(const char* payload, void** args, int32_t nargs, const void* attrs,
                             double* host_times, int64_t nruns, int64_t nwarmup);

#ifdef __cplusplus
}
#endif
#endif /* LIGHTHOUSE_HIP_H */
