// C ABI entry points: argument validation, the plain-pointer GEMM calls, the nanoGPT block,
// and the packed-argument (memref descriptor) payload calls with their benchmark wrapper.
#include <chrono>
#include <cstring>
#include <vector>

#include "gemm_common.h"

namespace lh {

static int gemm_common_checks(const char* who, const void* out, const void* a, const void* b, const void* bias,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, uint32_t flags) {
  LH_REQUIRE(out && a && b, "%s: null pointer", who);
  LH_REQUIRE(M > 0 && N > 0 && K > 0, "%s: empty problem M=%lld N=%lld K=%lld", who, (long long)M, (long long)N,
             (long long)K);
  LH_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "%s: dimension exceeds 2^31", who);
  const bool ta = flags & LH_GEMM_TRANSPOSE_A, tb = flags & LH_GEMM_TRANSPOSE_B;
  LH_REQUIRE(lda >= (ta ? M : K), "%s: lda %lld too small", who, (long long)lda);
  LH_REQUIRE(ldb >= (tb ? K : N), "%s: ldb %lld too small", who, (long long)ldb);
  LH_REQUIRE(ldc >= N, "%s: ldc %lld too small", who, (long long)ldc);
  LH_REQUIRE(!(flags & LH_GEMM_HAS_BIAS) || bias != nullptr, "%s: HAS_BIAS set but bias is null", who);
  LH_REQUIRE(!((flags & LH_GEMM_HAS_RELU) && (flags & LH_GEMM_HAS_GELU)), "%s: RELU and GELU are exclusive", who);
  const uint32_t known = LH_GEMM_HAS_BIAS | LH_GEMM_HAS_RELU | LH_GEMM_ACCUMULATE_C | LH_GEMM_TRANSPOSE_A |
                         LH_GEMM_TRANSPOSE_B | LH_GEMM_HAS_GELU | LH_GEMM_TILE_MASK | LH_GEMM_SPLITK_MASK;
  LH_REQUIRE((flags & ~known) == 0, "%s: unknown flag bits 0x%x", who, flags & ~known);
  LH_REQUIRE((flags & LH_GEMM_TILE_MASK) <= LH_GEMM_TILE_64x64, "%s: unknown tile request 0x%x", who,
             flags & LH_GEMM_TILE_MASK);
  LH_REQUIRE((flags & LH_GEMM_SPLITK_MASK) <= LH_GEMM_SPLITK_8, "%s: unknown split-K request 0x%x", who,
             flags & LH_GEMM_SPLITK_MASK);
  LH_REQUIRE((flags & LH_GEMM_SPLITK_MASK) <= LH_GEMM_SPLITK_NONE || (flags & LH_GEMM_TILE_MASK) == LH_GEMM_TILE_AUTO,
             "%s: a split-K request runs on 128 x 128 tiles and excludes a tile request", who);
  return LH_OK;
}

// Internal form with a separate accumulator input, bias type and source of temporary memory.
int gemm_run(void* out, const void* c, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
             int64_t lda, int64_t ldb, int64_t ldc, int ab_dtype, int out_dtype, int bias_dtype, uint32_t flags,
             hipStream_t s, Scratch* ws = nullptr) {
  GemmArgs g;
  g.out = out; g.c = c; g.a = a; g.b = b; g.bias = bias;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.flags = flags; g.out_dt = out_dtype; g.bias_dt = bias_dtype; g.alpha = 1.0f;
  g.ws = ws;
  if (ws) ws->used = 0;  // temporaries of an earlier call on the stream are dead once this one runs
  if (ab_dtype == LH_F32) {
    const uint32_t tile = flags & LH_GEMM_TILE_MASK;
    LH_REQUIRE((flags & LH_GEMM_SPLITK_MASK) == 0, "gemm: split-K requests apply to 16-bit inputs only");
    LH_REQUIRE(tile == LH_GEMM_TILE_AUTO || tile >= LH_GEMM_TILE_128x128,
               "gemm: f32 inputs take the 128x128, 128x64 and 64x64 tiles");
    return gemm32(g, s);
  }
  LH_REQUIRE((flags & LH_GEMM_TILE_MASK) <= LH_GEMM_TILE_128x128,
             "gemm: 16-bit inputs take the 256x256, 256x128, 128x256 and 128x128 tiles");
  return gemm16(g, ab_dtype, s);
}

// Temporary bytes gemm_run would take for this problem: the dispatch code itself is run with launches
// and allocations switched off.  The operand pointers are never dereferenced here; only their
// alignment matters (an operand that is not 16-byte aligned runs on a padded copy, which is part
// of the need).  The overload without pointers assumes aligned operands.
static size_t gemm_need(const void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc, int ab_dtype, int out_dtype, int bias_dtype,
                        uint32_t flags) {
  PlanningScope plan;
  Scratch ws;
  const int rc = gemm_run(const_cast<void*>(out), out, a, b, (flags & LH_GEMM_HAS_BIAS) ? bias : nullptr, M, N, K, lda, ldb,
                          ldc, ab_dtype, out_dtype, bias_dtype, flags, nullptr, &ws);
  return rc ? 0 : ws.need;
}
static size_t gemm_need(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int ab_dtype,
                        int out_dtype, int bias_dtype, uint32_t flags) {
  void* const fake = reinterpret_cast<void*>(uintptr_t(1) << 20);
  return gemm_need(fake, fake, fake, fake, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, bias_dtype, flags);
}

static int gemm8_run(void* out, const void* a_q, const void* b_q, float scale_a, float scale_b, int64_t M, int64_t N,
                     int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t out_dtype, hipStream_t s, Scratch* ws) {
  GemmArgs g;
  g.out = out; g.c = out; g.a = a_q; g.b = b_q; g.bias = nullptr;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.flags = 0; g.out_dt = out_dtype; g.bias_dt = out_dtype;
  g.alpha = scale_a * scale_b;
  g.ws = ws;
  if (ws) ws->used = 0;
  return gemm8(g, s);
}

static int gemm_dtype_checks(const char* who, int32_t ab_dtype, int32_t out_dtype) {
  if (!(ab_dtype == LH_F32 || ab_dtype == LH_BF16 || ab_dtype == LH_F16))
    return fail(LH_ERR_UNSUPPORTED, "%s: unsupported A/B dtype %d", who, ab_dtype);
  if (!(out_dtype == LH_F32 || (out_dtype == ab_dtype)))
    return fail(LH_ERR_UNSUPPORTED, "%s: out dtype %d must be f32 or the A/B dtype %d", who, out_dtype, ab_dtype);
  return LH_OK;
}

static int workspace_checks(const char* who, const void* workspace, size_t workspace_bytes) {
  LH_REQUIRE(workspace != nullptr || workspace_bytes == 0, "%s: null workspace of %zu bytes", who, workspace_bytes);
  LH_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, "%s: workspace must be 256-byte aligned", who);
  return LH_OK;
}

// ---- memref descriptors ------------------------------------------------------------------
struct Memref {
  char* base;  // aligned pointer
  int64_t offset;
  const int64_t* sizes;
  const int64_t* strides;
  void* data(size_t elem) const { return base + offset * (int64_t)elem; }
};

// args[i] points at a pointer to {allocated, aligned, offset, sizes[rank], strides[rank]}.
static bool get_memref(void** args, int i, Memref* m) {
  if (args == nullptr || args[i] == nullptr) return false;
  char* desc = *reinterpret_cast<char**>(args[i]);
  if (desc == nullptr) return false;
  void* aligned;
  std::memcpy(&aligned, desc + sizeof(void*), sizeof(void*));
  std::memcpy(&m->offset, desc + 2 * sizeof(void*), sizeof(int64_t));
  m->base = reinterpret_cast<char*>(aligned);
  m->sizes = reinterpret_cast<const int64_t*>(desc + 2 * sizeof(void*) + sizeof(int64_t));
  return m->base != nullptr;
}
static bool get_memref(void** args, int i, int rank, Memref* m) {
  if (!get_memref(args, i, m)) return false;
  m->strides = m->sizes + rank;
  return true;
}

static int sync_default() {
  LH_HIP_CHECK(hipStreamSynchronize(nullptr));
  return LH_OK;
}

}  // namespace lh

using namespace lh;

extern "C" {

int lh_hip_gemm(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K, int64_t lda,
                int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype, uint32_t flags, void* stream) {
  int rc = gemm_common_checks("lh_hip_gemm", out, a, b, bias, M, N, K, lda, ldb, ldc, flags);
  if (rc) return rc;
  if ((rc = gemm_dtype_checks("lh_hip_gemm", ab_dtype, out_dtype))) return rc;
  return gemm_run(out, out, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags,
                  reinterpret_cast<hipStream_t>(stream));
}

size_t lh_hip_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                   int32_t ab_dtype, int32_t out_dtype, uint32_t flags) {
  void* const fake = reinterpret_cast<void*>(uintptr_t(1) << 20);
  if (gemm_common_checks("lh_hip_gemm_workspace_bytes", fake, fake, fake, fake, M, N, K, lda, ldb, ldc, flags)) return 0;
  if (gemm_dtype_checks("lh_hip_gemm_workspace_bytes", ab_dtype, out_dtype)) return 0;
  return gemm_need(M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags);
}

size_t lh_hip_gemm_workspace_bytes_for(const void* out, const void* a, const void* b, const void* bias, int64_t M,
                                       int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype,
                                       int32_t out_dtype, uint32_t flags) {
  if (gemm_common_checks("lh_hip_gemm_workspace_bytes_for", out, a, b, bias, M, N, K, lda, ldb, ldc, flags)) return 0;
  if (gemm_dtype_checks("lh_hip_gemm_workspace_bytes_for", ab_dtype, out_dtype)) return 0;
  return gemm_need(out, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags);
}

int lh_hip_gemm_ws(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype, uint32_t flags,
                   void* workspace, size_t workspace_bytes, void* stream) {
  int rc = gemm_common_checks("lh_hip_gemm_ws", out, a, b, bias, M, N, K, lda, ldb, ldc, flags);
  if (rc) return rc;
  if ((rc = gemm_dtype_checks("lh_hip_gemm_ws", ab_dtype, out_dtype))) return rc;
  if ((rc = workspace_checks("lh_hip_gemm_ws", workspace, workspace_bytes))) return rc;
  // The need of THESE operands (their alignment included), checked before anything is launched.
  const size_t need = gemm_need(out, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags);
  LH_REQUIRE(need <= workspace_bytes,
             "lh_hip_gemm_ws: workspace too small: this call needs %zu bytes of temporary memory, %zu were given "
             "(lh_hip_gemm_workspace_bytes_for gives the need of operands that are not 16-byte aligned)",
             need, workspace_bytes);
  Scratch ws;
  // An empty workspace still must not fall back to the pool: the base stays non-null.
  ws.base = workspace ? static_cast<char*>(workspace) : reinterpret_cast<char*>(uintptr_t(256));
  ws.bytes = workspace_bytes;
  return gemm_run(out, out, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags,
                  reinterpret_cast<hipStream_t>(stream), &ws);
}

int lh_hip_gemm_static(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype, uint32_t flags,
                       void* stream) {
  int rc = gemm_common_checks("lh_hip_gemm_static", out, a, b, bias, M, N, K, lda, ldb, ldc, flags);
  if (rc) return rc;
  if ((rc = gemm_dtype_checks("lh_hip_gemm_static", ab_dtype, out_dtype))) return rc;
  // What the dispatch takes for these operands (their alignment included), known before anything is launched.
  const size_t need = gemm_need(out, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags);
  LH_REQUIRE(need <= LH_STATIC_SCRATCH_BYTES,
             "lh_hip_gemm_static: this problem needs %zu bytes of temporary memory, the static scratch holds %zu "
             "(use lh_hip_gemm_ws with a workspace of that size)",
             need, (size_t)LH_STATIC_SCRATCH_BYTES);
  Scratch ws;
  if ((rc = static_scratch(&ws.base, &ws.bytes))) return rc;
  return gemm_run(out, out, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype, flags,
                  reinterpret_cast<hipStream_t>(stream), &ws);
}

int lh_hip_gemm_residual(void* out, const void* c, const void* a, const void* b, const void* bias, int64_t M, int64_t N,
                         int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t ab_dtype, int32_t out_dtype,
                         uint32_t flags, void* stream) {
  int rc = gemm_common_checks("lh_hip_gemm_residual", out, a, b, bias, M, N, K, lda, ldb, ldc, flags);
  if (rc) return rc;
  LH_REQUIRE(c != nullptr, "lh_hip_gemm_residual: null accumulator input");
  if ((rc = gemm_dtype_checks("lh_hip_gemm_residual", ab_dtype, out_dtype))) return rc;
  return gemm_run(out, c, a, b, bias, M, N, K, lda, ldb, ldc, ab_dtype, out_dtype, out_dtype,
                  flags | LH_GEMM_ACCUMULATE_C, reinterpret_cast<hipStream_t>(stream));
}

int lh_hip_gemm_fp8(void* out, const void* a_q, const void* b_q, float scale_a, float scale_b, int64_t M, int64_t N,
                    int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t out_dtype, void* stream) {
  int rc = gemm_common_checks("lh_hip_gemm_fp8", out, a_q, b_q, nullptr, M, N, K, lda, ldb, ldc, 0);
  if (rc) return rc;
  if (!(out_dtype == LH_BF16 || out_dtype == LH_F32))
    return fail(LH_ERR_UNSUPPORTED, "lh_hip_gemm_fp8: out dtype %d must be bf16 or f32", out_dtype);
  return gemm8_run(out, a_q, b_q, scale_a, scale_b, M, N, K, lda, ldb, ldc, out_dtype,
                   reinterpret_cast<hipStream_t>(stream), nullptr);
}

size_t lh_hip_gemm_fp8_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                       int32_t out_dtype) {
  void* const fake = reinterpret_cast<void*>(uintptr_t(1) << 20);
  if (gemm_common_checks("lh_hip_gemm_fp8_workspace_bytes", fake, fake, fake, nullptr, M, N, K, lda, ldb, ldc, 0)) return 0;
  if (!(out_dtype == LH_BF16 || out_dtype == LH_F32)) return 0;
  PlanningScope plan;
  Scratch ws;
  const int rc = gemm8_run(fake, fake, fake, 1.0f, 1.0f, M, N, K, lda, ldb, ldc, out_dtype, nullptr, &ws);
  return rc ? 0 : ws.need;
}

int lh_hip_gemm_fp8_ws(void* out, const void* a_q, const void* b_q, float scale_a, float scale_b, int64_t M, int64_t N,
                       int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int32_t out_dtype, void* workspace,
                       size_t workspace_bytes, void* stream) {
  int rc = gemm_common_checks("lh_hip_gemm_fp8_ws", out, a_q, b_q, nullptr, M, N, K, lda, ldb, ldc, 0);
  if (rc) return rc;
  if (!(out_dtype == LH_BF16 || out_dtype == LH_F32))
    return fail(LH_ERR_UNSUPPORTED, "lh_hip_gemm_fp8_ws: out dtype %d must be bf16 or f32", out_dtype);
  if ((rc = workspace_checks("lh_hip_gemm_fp8_ws", workspace, workspace_bytes))) return rc;
  Scratch ws;
  ws.base = workspace ? static_cast<char*>(workspace) : reinterpret_cast<char*>(uintptr_t(256));
  ws.bytes = workspace_bytes;
  return gemm8_run(out, a_q, b_q, scale_a, scale_b, M, N, K, lda, ldb, ldc, out_dtype,
                   reinterpret_cast<hipStream_t>(stream), &ws);
}

// ---- nanoGPT block -------------------------------------------------------------------------
static size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

struct BlockConfig {
  bool causal;
  int activation, bias_dtype;
  int64_t hidden;
};
static int block_config(const char* who, const lh_nanogpt_block_opts* o, int64_t C, int32_t dtype, BlockConfig* c) {
  c->causal = o ? o->causal != 0 : true;
  c->activation = o ? o->activation : LH_ACT_GELU_TANH;
  c->bias_dtype = o ? o->bias_dtype : dtype;
  c->hidden = (o && o->hidden > 0) ? o->hidden : 4 * C;
  LH_REQUIRE(dtype == LH_F32 || dtype == LH_BF16 || dtype == LH_F16, "%s: dtype must be f32, bf16 or f16", who);
  LH_REQUIRE(c->activation == LH_ACT_GELU_TANH || c->activation == LH_ACT_RELU, "%s: unknown activation %d", who,
             c->activation);
  LH_REQUIRE(c->bias_dtype == dtype || c->bias_dtype == LH_F32, "%s: bias type must be f32 or the weight type", who);
  return LH_OK;
}

// The block's fixed buffers, then the temporaries of whichever of its GEMMs needs most.
static size_t block_fixed_bytes(size_t rows, int64_t C, int64_t hidden, size_t e) {
  return align256(rows * C * e)         /* LayerNorm output */
         + align256(rows * 3 * C * e)   /* q | k | v */
         + align256(rows * C * e)       /* attention output */
         + align256(rows * C * 4)       /* residual stream after attention */
         + align256(rows * hidden * e); /* MLP hidden */
}
static size_t block_gemm_need(int64_t rows, int64_t C, int64_t hidden, int32_t dtype, int bias_dt) {
  const uint32_t bias = LH_GEMM_HAS_BIAS;
  size_t need = gemm_need(rows, 3 * C, C, C, 3 * C, 3 * C, dtype, dtype, bias_dt, bias);
  auto upto = [&](size_t n) { if (n > need) need = n; };
  upto(gemm_need(rows, C, C, C, C, 3 * C, dtype, dtype, bias_dt, bias));  // separate q / k / v projections
  upto(gemm_need(rows, C, C, C, C, C, dtype, LH_F32, bias_dt, bias | LH_GEMM_ACCUMULATE_C));
  upto(gemm_need(rows, hidden, C, C, hidden, hidden, dtype, dtype, bias_dt, bias | LH_GEMM_HAS_GELU));
  upto(gemm_need(rows, C, hidden, hidden, C, C, dtype, LH_F32, bias_dt, bias | LH_GEMM_ACCUMULATE_C));
  return align256(need);
}

size_t lh_hip_nanogpt_block_workspace_bytes(int64_t B, int64_t T, int64_t C, int32_t dtype,
                                            const lh_nanogpt_block_opts* opts) {
  BlockConfig cfg;
  if (B <= 0 || T <= 0 || C <= 0 || block_config("lh_hip_nanogpt_block_workspace_bytes", opts, C, dtype, &cfg)) return 0;
  return block_fixed_bytes((size_t)B * T, C, cfg.hidden, dtype_size(dtype)) +
         block_gemm_need(B * T, C, cfg.hidden, dtype, cfg.bias_dtype);
}

int lh_hip_nanogpt_block(float* y, const float* x, const lh_nanogpt_block_params* p, int64_t B, int64_t T, int64_t C,
                         int64_t n_head, float eps, int32_t dtype, const lh_nanogpt_block_opts* opts, void* workspace,
                         size_t workspace_bytes, void* stream) {
  LH_REQUIRE(y && x && p && workspace, "lh_hip_nanogpt_block: null pointer");
  BlockConfig cfg;
  if (int rc = block_config("lh_hip_nanogpt_block", opts, C, dtype, &cfg)) return rc;
  LH_REQUIRE(B > 0 && T > 0 && C > 0 && n_head > 0 && C % n_head == 0, "lh_hip_nanogpt_block: bad shape");
  LH_REQUIRE(p->ln1_g && p->ln1_b && p->ln2_g && p->ln2_b && p->w_o && p->w_fc && p->w_proj,
             "lh_hip_nanogpt_block: null parameter");
  LH_REQUIRE(p->w_qkv || (p->w_q && p->w_k && p->w_v), "lh_hip_nanogpt_block: w_qkv or all of w_q, w_k, w_v must be set");
  LH_REQUIRE(workspace_bytes >= lh_hip_nanogpt_block_workspace_bytes(B, T, C, dtype, opts),
             "lh_hip_nanogpt_block: workspace too small (%zu bytes)", workspace_bytes);
  LH_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, "lh_hip_nanogpt_block: workspace must be 256-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const size_t e = dtype_size(dtype), eb = dtype_size(cfg.bias_dtype);
  const int64_t rows = B * T, hs = C / n_head, hidden = cfg.hidden;
  const int bdt = cfg.bias_dtype;
  char* w = reinterpret_cast<char*>(workspace);
  void* ln = w;            w += align256((size_t)rows * C * e);
  void* qkv = w;           w += align256((size_t)rows * 3 * C * e);
  void* att = w;           w += align256((size_t)rows * C * e);
  float* a = (float*)w;    w += align256((size_t)rows * C * 4);
  void* hid = w;           w += align256((size_t)rows * hidden * e);
  Scratch ws;  // temporaries of the GEMMs: the rest of the workspace
  ws.base = w;
  ws.bytes = workspace_bytes - (size_t)(w - reinterpret_cast<char*>(workspace));
  auto bias_flag = [](const void* b) -> uint32_t { return b ? LH_GEMM_HAS_BIAS : 0u; };
  int rc;
  // ln1 = LN(x), rounded to the matmul input type.
  if ((rc = layer_norm(ln, x, p->ln1_g, p->ln1_b, rows, C, eps, LH_F32, dtype, false, s))) return rc;
  if (p->w_qkv) {
    // qkv = ln1 Wqkv + bqkv
    if ((rc = gemm_run(qkv, nullptr, ln, p->w_qkv, p->b_qkv, rows, 3 * C, C, C, 3 * C, 3 * C, dtype, dtype, bdt,
                       bias_flag(p->b_qkv), s, &ws)))
      return rc;
  } else {
    // q, k, v = ln1 Wq, ln1 Wk, ln1 Wv into the three column blocks of the same buffer
    const void* wsep[3] = {p->w_q, p->w_k, p->w_v};
    for (int i = 0; i < 3; ++i) {
      const void* bi = p->b_qkv ? static_cast<const char*>(p->b_qkv) + (size_t)i * C * eb : nullptr;
      if ((rc = gemm_run(static_cast<char*>(qkv) + (size_t)i * C * e, nullptr, ln, wsep[i], bi, rows, C, C, C, C, 3 * C,
                         dtype, dtype, bdt, bias_flag(bi), s, &ws)))
        return rc;
    }
  }
  // Attention on (B, H, T, hs) strided views of the (B*T, 3C) projection buffer.
  {
    lh_strides3 sqkv = {T * 3 * C, hs, 3 * C};
    lh_strides3 so = {T * C, hs, C};
    const char* qp = reinterpret_cast<const char*>(qkv);
    NoAttentionScratchScope own_workspace_only;  // (the block's temporaries all come from `workspace`)
    if ((rc = lh_hip_attention(att, qp, qp + (size_t)C * e, qp + (size_t)2 * C * e, B, n_head, T, hs, so, sqkv, sqkv,
                               sqkv, 0.0f, cfg.causal ? 1 : 0, dtype, s)))
      return rc;
  }
  // a = x + att Wo + bo
  if ((rc = gemm_run(a, x, att, p->w_o, p->b_o, rows, C, C, C, C, C, dtype, LH_F32, bdt,
                     bias_flag(p->b_o) | LH_GEMM_ACCUMULATE_C, s, &ws)))
    return rc;
  // ln2 = LN(a)
  if ((rc = layer_norm(ln, a, p->ln2_g, p->ln2_b, rows, C, eps, LH_F32, dtype, false, s))) return rc;
  // h = act(ln2 W1 + b1)
  const uint32_t act = cfg.activation == LH_ACT_RELU ? LH_GEMM_HAS_RELU : LH_GEMM_HAS_GELU;
  if ((rc = gemm_run(hid, nullptr, ln, p->w_fc, p->b_fc, rows, hidden, C, C, hidden, hidden, dtype, dtype, bdt,
                     bias_flag(p->b_fc) | act, s, &ws)))
    return rc;
  // y = a + h W2 + b2
  return gemm_run(y, a, hid, p->w_proj, p->b_proj, rows, C, hidden, hidden, C, C, dtype, LH_F32, bdt,
                  bias_flag(p->b_proj) | LH_GEMM_ACCUMULATE_C, s, &ws);
}

static size_t forward_head_need(int64_t rows, int64_t C, int64_t vocab, int32_t dtype, int bias_dt) {
  return align256(gemm_need(rows, vocab, C, C, vocab, vocab, dtype, LH_F32, bias_dt, LH_GEMM_HAS_BIAS));
}

size_t lh_hip_nanogpt_forward_workspace_bytes(int64_t B, int64_t T, int64_t C, int64_t vocab, int32_t dtype,
                                              const lh_nanogpt_block_opts* opts) {
  BlockConfig cfg;
  if (B <= 0 || T <= 0 || C <= 0 || vocab <= 0 ||
      block_config("lh_hip_nanogpt_forward_workspace_bytes", opts, C, dtype, &cfg))
    return 0;
  const size_t rows = (size_t)B * T;
  return lh_hip_nanogpt_block_workspace_bytes(B, T, C, dtype, opts) + 2 * align256(rows * C * 4) /* residual streams */
         + forward_head_need(B * T, C, vocab, dtype, cfg.bias_dtype);
}

int lh_hip_nanogpt_forward(float* logits, const float* x, const lh_nanogpt_block_params* blocks, int64_t n_layer,
                           const float* lnf_g, const float* lnf_b, const void* lm_w, const void* lm_b, int64_t B,
                           int64_t T, int64_t C, int64_t n_head, int64_t vocab, float eps, int32_t dtype,
                           const lh_nanogpt_block_opts* opts, void* workspace, size_t workspace_bytes, void* stream) {
  LH_REQUIRE(logits && x && lnf_g && lnf_b && lm_w && workspace, "lh_hip_nanogpt_forward: null pointer");
  LH_REQUIRE(n_layer >= 0 && (n_layer == 0 || blocks), "lh_hip_nanogpt_forward: bad layer list");
  BlockConfig cfg;
  if (int rc = block_config("lh_hip_nanogpt_forward", opts, C, dtype, &cfg)) return rc;
  LH_REQUIRE(B > 0 && T > 0 && C > 0 && vocab > 0, "lh_hip_nanogpt_forward: bad shape");
  LH_REQUIRE(workspace_bytes >= lh_hip_nanogpt_forward_workspace_bytes(B, T, C, vocab, dtype, opts),
             "lh_hip_nanogpt_forward: workspace too small (%zu bytes)", workspace_bytes);
  LH_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, "lh_hip_nanogpt_forward: workspace must be 256-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t rows = B * T;
  const size_t block_ws = lh_hip_nanogpt_block_workspace_bytes(B, T, C, dtype, opts);
  char* w = reinterpret_cast<char*>(workspace);
  float* h[2] = {reinterpret_cast<float*>(w + block_ws),
                 reinterpret_cast<float*>(w + block_ws + align256((size_t)rows * C * 4))};
  const float* cur = x;
  for (int64_t l = 0; l < n_layer; ++l) {
    float* nxt = h[l & 1];
    int rc = lh_hip_nanogpt_block(nxt, cur, &blocks[l], B, T, C, n_head, eps, dtype, opts, workspace, block_ws, stream);
    if (rc) return rc;
    cur = nxt;
  }
  // hf = LN_f(h) rounded to the matmul input type (first area of the block workspace), then lm_head.
  int rc = layer_norm(workspace, cur, lnf_g, lnf_b, rows, C, eps, LH_F32, dtype, false, s);
  if (rc) return rc;
  Scratch ws;
  ws.base = w + block_ws + 2 * align256((size_t)rows * C * 4);
  ws.bytes = workspace_bytes - (size_t)(ws.base - w);
  return gemm_run(logits, nullptr, workspace, lm_w, lm_b, rows, vocab, C, C, vocab, vocab, dtype, LH_F32, cfg.bias_dtype,
                  lm_b ? LH_GEMM_HAS_BIAS : 0, s, &ws);
}

// ---- packed-argument payloads -------------------------------------------------------------

int lh_hip_payload_matmul(void** args, int32_t nargs, const lh_matmul_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_matmul: null argument");
  const bool has_bias = at->flags & LH_GEMM_HAS_BIAS;
  LH_REQUIRE(nargs == (has_bias ? 4 : 3), "lh_hip_payload_matmul: expected %d arguments, got %d", has_bias ? 4 : 3,
             nargs);
  Memref o, a, b, bias;
  LH_REQUIRE(get_memref(args, 0, 2, &o) && get_memref(args, 1, 2, &a) && get_memref(args, 2, 2, &b),
             "lh_hip_payload_matmul: bad memref descriptor");
  const bool ta = at->flags & LH_GEMM_TRANSPOSE_A, tb = at->flags & LH_GEMM_TRANSPOSE_B;
  const int64_t M = o.sizes[0], N = o.sizes[1];
  const int64_t K = ta ? a.sizes[0] : a.sizes[1];
  LH_REQUIRE((ta ? a.sizes[1] : a.sizes[0]) == M, "lh_hip_payload_matmul: A shape does not match out rows");
  LH_REQUIRE((tb ? b.sizes[1] : b.sizes[0]) == K && (tb ? b.sizes[0] : b.sizes[1]) == N,
             "lh_hip_payload_matmul: B shape [%lld,%lld] does not match K=%lld N=%lld", (long long)b.sizes[0],
             (long long)b.sizes[1], (long long)K, (long long)N);
  LH_REQUIRE(o.strides[1] == 1 && a.strides[1] == 1 && b.strides[1] == 1,
             "lh_hip_payload_matmul: innermost stride must be 1");
  const void* bias_p = nullptr;
  if (has_bias) {
    LH_REQUIRE(get_memref(args, 3, 1, &bias), "lh_hip_payload_matmul: bad bias descriptor");
    LH_REQUIRE(bias.sizes[0] == N && bias.strides[0] == 1, "lh_hip_payload_matmul: bias must be contiguous [N]");
    bias_p = bias.data(dtype_size(at->out_dtype));
  }
  int rc = lh_hip_gemm(o.data(dtype_size(at->out_dtype)), a.data(dtype_size(at->ab_dtype)),
                       b.data(dtype_size(at->ab_dtype)), bias_p, M, N, K, a.strides[0], b.strides[0], o.strides[0],
                       at->ab_dtype, at->out_dtype, at->flags, nullptr);
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_mlp(void** args, int32_t nargs, const lh_mlp_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_mlp: null argument");
  const int n = at->nlayers;
  LH_REQUIRE(n >= 1 && n <= 64, "lh_hip_payload_mlp: nlayers %d out of range", n);
  const bool has_bias = at->flags & LH_GEMM_HAS_BIAS;
  LH_REQUIRE(nargs == 2 + n * (has_bias ? 2 : 1), "lh_hip_payload_mlp: expected %d arguments, got %d",
             2 + n * (has_bias ? 2 : 1), nargs);
  LH_REQUIRE((at->flags & ~(LH_GEMM_HAS_BIAS | LH_GEMM_HAS_RELU | LH_GEMM_ACCUMULATE_C | LH_GEMM_TRANSPOSE_A |
                            LH_GEMM_TRANSPOSE_B)) == 0,
             "lh_hip_payload_mlp: unsupported flag bits 0x%x", at->flags);
  LH_REQUIRE(at->ab_dtype == LH_F32 || at->ab_dtype == LH_BF16 || at->ab_dtype == LH_F16,
             "lh_hip_payload_mlp: unsupported A/B dtype %d", at->ab_dtype);
  LH_REQUIRE(at->out_dtype == LH_F32 || at->out_dtype == at->ab_dtype,
             "lh_hip_payload_mlp: result type must be f32 or the A/B type");
  LH_REQUIRE(!has_bias || at->bias_dtype == LH_F32 || at->bias_dtype == at->ab_dtype,
             "lh_hip_payload_mlp: bias type must be f32 or the A/B type");
  const bool ta = at->flags & LH_GEMM_TRANSPOSE_A, tb = at->flags & LH_GEMM_TRANSPOSE_B;
  const size_t eab = dtype_size(at->ab_dtype), eout = dtype_size(at->out_dtype);
  Memref o, in;
  LH_REQUIRE(get_memref(args, 0, 2, &o) && get_memref(args, 1, 2, &in), "lh_hip_payload_mlp: bad memref descriptor");
  LH_REQUIRE(o.strides[1] == 1 && in.strides[1] == 1, "lh_hip_payload_mlp: innermost stride must be 1");
  const int64_t M = ta ? in.sizes[1] : in.sizes[0];
  LH_REQUIRE(o.sizes[0] == M, "lh_hip_payload_mlp: output rows %lld != batch %lld", (long long)o.sizes[0], (long long)M);
  int64_t width = ta ? in.sizes[0] : in.sizes[1];
  int64_t max_hidden = 0;
  Memref w[64], bias[64];
  for (int i = 0; i < n; ++i) {
    LH_REQUIRE(get_memref(args, 2 + i, 2, &w[i]) && w[i].strides[1] == 1, "lh_hip_payload_mlp: bad weight %d", i);
    const int64_t k = tb ? w[i].sizes[1] : w[i].sizes[0], nn = tb ? w[i].sizes[0] : w[i].sizes[1];
    LH_REQUIRE(k == width, "lh_hip_payload_mlp: weight %d has %lld input features, expected %lld", i, (long long)k,
               (long long)width);
    if (has_bias) {
      LH_REQUIRE(get_memref(args, 2 + n + i, 1, &bias[i]) && bias[i].sizes[0] == nn && bias[i].strides[0] == 1,
                 "lh_hip_payload_mlp: bias %d must be contiguous [%lld]", i, (long long)nn);
    }
    width = nn;
    if (i + 1 < n && nn > max_hidden) max_hidden = nn;
  }
  LH_REQUIRE(o.sizes[1] == width, "lh_hip_payload_mlp: output has %lld columns, last layer %lld", (long long)o.sizes[1],
             (long long)width);
  const size_t half = ((size_t)M * max_hidden * eab + 255) & ~(size_t)255;
  // Hidden activations: two halves of a pool buffer used alternately.
  char* hidden_buf = nullptr;
  if (n > 1) {
    void* taken = nullptr;
    if (int rc = scratch_take(nullptr, nullptr, kScratchMlp, 2 * half, "lh_hip_payload_mlp", &taken)) return rc;
    hidden_buf = static_cast<char*>(taken);
  }
  const void* act = in.data(eab);
  int64_t lda = in.strides[0];
  int64_t K = ta ? in.sizes[0] : in.sizes[1];
  for (int i = 0; i < n; ++i) {
    const bool last = i + 1 == n;
    const int64_t N = tb ? w[i].sizes[0] : w[i].sizes[1];
    uint32_t flags = (at->flags & LH_GEMM_TRANSPOSE_B) | (has_bias ? LH_GEMM_HAS_BIAS : 0);
    if (i == 0 && ta) flags |= LH_GEMM_TRANSPOSE_A;
    if ((at->flags & LH_GEMM_HAS_RELU) && (!last || at->relu_on_final_layer)) flags |= LH_GEMM_HAS_RELU;
    if (last && (at->flags & LH_GEMM_ACCUMULATE_C)) flags |= LH_GEMM_ACCUMULATE_C;
    void* dst = last ? o.data(eout) : static_cast<void*>(hidden_buf + (i & 1) * half);
    const int out_dt = last ? at->out_dtype : at->ab_dtype;
    const void* bias_p = has_bias ? bias[i].data(dtype_size(at->bias_dtype)) : nullptr;
    const int64_t ldc = last ? o.strides[0] : N;
    int rc = gemm_common_checks("lh_hip_payload_mlp", dst, act, w[i].data(eab), bias_p, M, N, K, lda, w[i].strides[0],
                                ldc, flags);
    if (rc) return rc;
    rc = gemm_run(dst, dst, act, w[i].data(eab), bias_p, M, N, K, lda, w[i].strides[0], ldc, at->ab_dtype, out_dt,
                  at->bias_dtype, flags, nullptr);
    if (rc) return rc;
    act = dst;
    lda = N;
    K = N;
  }
  return sync_default();
}

int lh_hip_payload_matmul_fp8(void** args, int32_t nargs, const lh_matmul_fp8_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_matmul_fp8: null argument");
  LH_REQUIRE(nargs == 3, "lh_hip_payload_matmul_fp8: expected 3 arguments, got %d", nargs);
  Memref o, a, b;
  LH_REQUIRE(get_memref(args, 0, 2, &o) && get_memref(args, 1, 2, &a) && get_memref(args, 2, 2, &b),
             "lh_hip_payload_matmul_fp8: bad memref descriptor");
  const int64_t M = o.sizes[0], N = o.sizes[1], K = a.sizes[1];
  LH_REQUIRE(a.sizes[0] == M && b.sizes[0] == K && b.sizes[1] == N, "lh_hip_payload_matmul_fp8: shape mismatch");
  LH_REQUIRE(o.strides[1] == 1 && a.strides[1] == 1 && b.strides[1] == 1,
             "lh_hip_payload_matmul_fp8: innermost stride must be 1");
  int rc = lh_hip_gemm_fp8(o.data(dtype_size(at->out_dtype)), a.data(1), b.data(1), at->scale_a, at->scale_b, M, N, K,
                           a.strides[0], b.strides[0], o.strides[0], at->out_dtype, nullptr);
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_attention(void** args, int32_t nargs, const lh_attention_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_attention: null argument");
  LH_REQUIRE(nargs == 4, "lh_hip_payload_attention: expected 4 arguments, got %d", nargs);
  Memref m[4];
  for (int i = 0; i < 4; ++i)
    LH_REQUIRE(get_memref(args, i, 4, &m[i]), "lh_hip_payload_attention: bad memref descriptor %d", i);
  for (int i = 1; i < 4; ++i)
    for (int r = 0; r < 4; ++r)
      LH_REQUIRE(m[i].sizes[r] == m[0].sizes[r], "lh_hip_payload_attention: shape mismatch in argument %d", i);
  lh_strides3 st[4];
  for (int i = 0; i < 4; ++i) {
    LH_REQUIRE(m[i].strides[3] == 1, "lh_hip_payload_attention: innermost stride must be 1");
    st[i] = lh_strides3{m[i].strides[0], m[i].strides[1], m[i].strides[2]};
  }
  const size_t e = dtype_size(at->dtype);
  int rc = lh_hip_attention(m[0].data(e), m[1].data(e), m[2].data(e), m[3].data(e), m[0].sizes[0], m[0].sizes[1],
                            m[0].sizes[2], m[0].sizes[3], st[0], st[1], st[2], st[3], at->scale, at->causal, at->dtype,
                            nullptr);
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_layer_norm(void** args, int32_t nargs, const lh_layer_norm_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_layer_norm: null argument");
  LH_REQUIRE(nargs == 4, "lh_hip_payload_layer_norm: expected 4 arguments, got %d", nargs);
  Memref o, x, g, b;
  LH_REQUIRE(get_memref(args, 0, 2, &o) && get_memref(args, 1, 2, &x) && get_memref(args, 2, 1, &g) &&
                 get_memref(args, 3, 1, &b),
             "lh_hip_payload_layer_norm: bad memref descriptor");
  const int64_t M = o.sizes[0], N = o.sizes[1];
  LH_REQUIRE(x.sizes[0] == M && x.sizes[1] == N && g.sizes[0] == N && b.sizes[0] == N,
             "lh_hip_payload_layer_norm: shape mismatch");
  LH_REQUIRE(o.strides[1] == 1 && x.strides[1] == 1 && o.strides[0] == N && x.strides[0] == N && g.strides[0] == 1 &&
                 b.strides[0] == 1,
             "lh_hip_payload_layer_norm: buffers must be contiguous");
  int rc = lh_hip_layer_norm(o.data(dtype_size(at->out_dtype)), x.data(dtype_size(at->x_dtype)),
                             reinterpret_cast<const float*>(g.data(4)), reinterpret_cast<const float*>(b.data(4)), M, N,
                             at->eps, at->x_dtype, at->out_dtype, nullptr);
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_elementwise(void** args, int32_t nargs, const lh_elementwise_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_elementwise: null argument");
  const int want = (at->kind == LH_EW_BIAS || at->kind == LH_EW_ADD) ? 3 : 2;
  LH_REQUIRE(nargs == want, "lh_hip_payload_elementwise: expected %d arguments, got %d", want, nargs);
  Memref o, x, y;
  LH_REQUIRE(get_memref(args, 0, 2, &o) && get_memref(args, 1, 2, &x), "lh_hip_payload_elementwise: bad descriptor");
  const int64_t M = o.sizes[0], N = o.sizes[1];
  LH_REQUIRE(x.sizes[0] == M && x.sizes[1] == N, "lh_hip_payload_elementwise: shape mismatch");
  LH_REQUIRE(o.strides[1] == 1 && x.strides[1] == 1 && o.strides[0] == N && x.strides[0] == N,
             "lh_hip_payload_elementwise: buffers must be contiguous");
  const size_t e = dtype_size(at->dtype);
  int rc;
  switch (at->kind) {
    case LH_EW_SOFTMAX: rc = lh_hip_softmax(o.data(e), x.data(e), M, N, at->dtype, nullptr); break;
    case LH_EW_GELU: rc = lh_hip_gelu_tanh(o.data(e), x.data(e), M * N, at->dtype, nullptr); break;
    case LH_EW_BIAS:
      LH_REQUIRE(get_memref(args, 2, 1, &y) && y.sizes[0] == N && y.strides[0] == 1,
                 "lh_hip_payload_elementwise: bias must be contiguous [N]");
      rc = lh_hip_bias_act(o.data(e), x.data(e), y.data(e), M, N, at->relu, at->dtype, nullptr);
      break;
    case LH_EW_ADD:
      LH_REQUIRE(get_memref(args, 2, 2, &y) && y.sizes[0] == M && y.sizes[1] == N && y.strides[1] == 1 &&
                     y.strides[0] == N,
                 "lh_hip_payload_elementwise: second operand must be contiguous [M,N]");
      rc = lh_hip_add(o.data(e), x.data(e), y.data(e), M * N, at->dtype, nullptr);
      break;
    case LH_EW_CAST:
      rc = lh_hip_cast(o.data(dtype_size(at->dst_dtype)), x.data(e), M * N, at->dtype, at->dst_dtype, nullptr);
      break;
    default: return fail(LH_ERR_INVALID, "lh_hip_payload_elementwise: unknown kind %d", at->kind);
  }
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_nanogpt_block(void** args, int32_t nargs, const lh_nanogpt_block_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_nanogpt_block: null argument");
  LH_REQUIRE(nargs == 15, "lh_hip_payload_nanogpt_block: expected 15 arguments, got %d", nargs);
  Memref y, x, v[12], ws;
  LH_REQUIRE(get_memref(args, 0, 2, &y) && get_memref(args, 1, 2, &x) && get_memref(args, 14, 1, &ws),
             "lh_hip_payload_nanogpt_block: bad memref descriptor");
  static const int ranks[12] = {1, 1, 2, 1, 2, 1, 1, 1, 2, 1, 2, 1};
  for (int i = 0; i < 12; ++i)
    LH_REQUIRE(get_memref(args, 2 + i, ranks[i], &v[i]), "lh_hip_payload_nanogpt_block: bad descriptor %d", 2 + i);
  const int64_t rows = y.sizes[0], C = y.sizes[1];
  LH_REQUIRE(rows == (int64_t)at->B * at->T && x.sizes[0] == rows && x.sizes[1] == C,
             "lh_hip_payload_nanogpt_block: x / y shape does not match B*T x C");
  LH_REQUIRE(y.strides[0] == C && y.strides[1] == 1 && x.strides[0] == C && x.strides[1] == 1,
             "lh_hip_payload_nanogpt_block: x and y must be contiguous");
  const int64_t want[12][2] = {{C, 0}, {C, 0}, {C, 3 * C}, {3 * C, 0}, {C, C}, {C, 0},
                               {C, 0}, {C, 0}, {C, 4 * C}, {4 * C, 0}, {4 * C, C}, {C, 0}};
  for (int i = 0; i < 12; ++i) {
    LH_REQUIRE(v[i].sizes[0] == want[i][0] && (ranks[i] == 1 || v[i].sizes[1] == want[i][1]),
               "lh_hip_payload_nanogpt_block: parameter %d has the wrong shape", 2 + i);
    LH_REQUIRE(v[i].strides[ranks[i] - 1] == 1 && (ranks[i] == 1 || v[i].strides[0] == v[i].sizes[1]),
               "lh_hip_payload_nanogpt_block: parameter %d must be contiguous", 2 + i);
  }
  const size_t e = dtype_size(at->dtype);
  lh_nanogpt_block_params p;
  p.ln1_g = (const float*)v[0].data(4); p.ln1_b = (const float*)v[1].data(4);
  p.w_qkv = v[2].data(e); p.b_qkv = v[3].data(e);
  p.w_o = v[4].data(e); p.b_o = v[5].data(e);
  p.ln2_g = (const float*)v[6].data(4); p.ln2_b = (const float*)v[7].data(4);
  p.w_fc = v[8].data(e); p.b_fc = v[9].data(e);
  p.w_proj = v[10].data(e); p.b_proj = v[11].data(e);
  p.w_q = p.w_k = p.w_v = nullptr;
  int rc = lh_hip_nanogpt_block((float*)y.data(4), (const float*)x.data(4), &p, at->B, at->T, C, at->n_head, at->eps,
                                at->dtype, nullptr, ws.data(1), (size_t)ws.sizes[0], nullptr);
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_gpt_fused(void** args, int32_t nargs, const lh_gpt_fused_attrs* at) {
  LH_REQUIRE(args && at, "lh_hip_payload_gpt_fused: null argument");
  LH_REQUIRE(at->n_layer >= 0 && at->n_layer <= 1024, "lh_hip_payload_gpt_fused: n_layer %d out of range", at->n_layer);
  const int L = at->n_layer;
  LH_REQUIRE(nargs == 2 + 13 * L + 4 + 1, "lh_hip_payload_gpt_fused: expected %d arguments, got %d", 2 + 13 * L + 5, nargs);
  Memref out, x, ws;
  LH_REQUIRE(get_memref(args, 0, 2, &out) && get_memref(args, 1, 2, &x) && get_memref(args, nargs - 1, 1, &ws),
             "lh_hip_payload_gpt_fused: bad memref descriptor");
  const int64_t T = x.sizes[0], C = x.sizes[1], vocab = out.sizes[1];
  LH_REQUIRE(out.sizes[0] == T, "lh_hip_payload_gpt_fused: out has %lld rows, x %lld", (long long)out.sizes[0], (long long)T);
  LH_REQUIRE(out.strides[1] == 1 && out.strides[0] == vocab && x.strides[1] == 1 && x.strides[0] == C,
             "lh_hip_payload_gpt_fused: out and x must be contiguous");
  const size_t e = dtype_size(at->dtype);
  LH_REQUIRE(e == 2 || e == 4, "lh_hip_payload_gpt_fused: unsupported dtype %d", at->dtype);
  // A contiguous vector [n] or matrix [r, c] argument; returns its data pointer through `ptr`.
  auto vec = [&](int i, int64_t n, size_t es, const void** ptr) -> bool {
    Memref m;
    if (!get_memref(args, i, 1, &m) || m.sizes[0] != n || m.strides[0] != 1) return false;
    *ptr = m.data(es);
    return true;
  };
  auto mat = [&](int i, int64_t r, int64_t c, const void** ptr) -> bool {
    Memref m;
    if (!get_memref(args, i, 2, &m) || m.sizes[0] != r || m.sizes[1] != c || m.strides[1] != 1 || m.strides[0] != c)
      return false;
    *ptr = m.data(e);
    return true;
  };
  int64_t hidden = 4 * C;
  if (L > 0) {
    Memref w1;
    LH_REQUIRE(get_memref(args, 2 + 9, 2, &w1), "lh_hip_payload_gpt_fused: bad descriptor of w1");
    hidden = w1.sizes[1];
  }
  std::vector<lh_nanogpt_block_params> blocks((size_t)(L > 0 ? L : 1));
  for (int l = 0; l < L; ++l) {
    const int b = 2 + 13 * l;
    lh_nanogpt_block_params& p = blocks[(size_t)l];
    const void *g1, *b1n, *g2, *b2n;
    p.w_qkv = nullptr;
    p.b_qkv = nullptr;
    const bool ok = vec(b + 0, C, 4, &g1) && vec(b + 1, C, 4, &b1n) && mat(b + 2, C, C, &p.w_q) &&
                    mat(b + 3, C, C, &p.w_k) && mat(b + 4, C, C, &p.w_v) && mat(b + 5, C, C, &p.w_o) &&
                    vec(b + 6, C, 4, &p.b_o) && vec(b + 7, C, 4, &g2) && vec(b + 8, C, 4, &b2n) &&
                    mat(b + 9, C, hidden, &p.w_fc) && vec(b + 10, hidden, 4, &p.b_fc) &&
                    mat(b + 11, hidden, C, &p.w_proj) && vec(b + 12, C, 4, &p.b_proj);
    LH_REQUIRE(ok, "lh_hip_payload_gpt_fused: a parameter of layer %d has the wrong shape or is not contiguous", l);
    p.ln1_g = (const float*)g1; p.ln1_b = (const float*)b1n; p.ln2_g = (const float*)g2; p.ln2_b = (const float*)b2n;
  }
  const int t = 2 + 13 * L;
  const void *gf_g, *gf_b, *lmw, *lmb;
  LH_REQUIRE(vec(t, C, 4, &gf_g) && vec(t + 1, C, 4, &gf_b) && mat(t + 2, C, vocab, &lmw) && vec(t + 3, vocab, 4, &lmb),
             "lh_hip_payload_gpt_fused: ln_f / lm_head parameter has the wrong shape or is not contiguous");
  lh_nanogpt_block_opts opts = {at->causal, LH_ACT_RELU, LH_F32, (int32_t)hidden};
  int rc = lh_hip_nanogpt_forward((float*)out.data(4), (const float*)x.data(4), blocks.data(), L, (const float*)gf_g,
                                  (const float*)gf_b, lmw, lmb, 1, T, C, at->n_head, vocab, at->eps, at->dtype, &opts,
                                  ws.data(1), (size_t)ws.sizes[0], nullptr);
  if (rc) return rc;
  return sync_default();
}

int lh_hip_payload_benchmark(const char* payload, void** args, int32_t nargs, const void* attrs, double* host_times,
                             int64_t nruns, int64_t nwarmup) {
  LH_REQUIRE(payload && args && attrs, "lh_hip_payload_benchmark: null argument");
  LH_REQUIRE(nruns >= 0 && nwarmup >= 0 && (nruns == 0 || host_times), "lh_hip_payload_benchmark: bad run counts");
  int kind;
  if (!std::strcmp(payload, "matmul")) kind = 0;
  else if (!std::strcmp(payload, "matmul_fp8")) kind = 1;
  else if (!std::strcmp(payload, "attention")) kind = 2;
  else if (!std::strcmp(payload, "layer_norm")) kind = 3;
  else if (!std::strcmp(payload, "elementwise")) kind = 4;
  else if (!std::strcmp(payload, "nanogpt_block")) kind = 5;
  else if (!std::strcmp(payload, "mlp")) kind = 6;
  else if (!std::strcmp(payload, "gpt_fused")) kind = 7;
  else return fail(LH_ERR_INVALID, "lh_hip_payload_benchmark: unknown payload '%s'", payload);
  auto call = [&]() -> int {
    switch (kind) {
      case 0: return lh_hip_payload_matmul(args, nargs, reinterpret_cast<const lh_matmul_attrs*>(attrs));
      case 1: return lh_hip_payload_matmul_fp8(args, nargs, reinterpret_cast<const lh_matmul_fp8_attrs*>(attrs));
      case 2: return lh_hip_payload_attention(args, nargs, reinterpret_cast<const lh_attention_attrs*>(attrs));
      case 3: return lh_hip_payload_layer_norm(args, nargs, reinterpret_cast<const lh_layer_norm_attrs*>(attrs));
      case 4: return lh_hip_payload_elementwise(args, nargs, reinterpret_cast<const lh_elementwise_attrs*>(attrs));
      case 5: return lh_hip_payload_nanogpt_block(args, nargs, reinterpret_cast<const lh_nanogpt_block_attrs*>(attrs));
      case 6: return lh_hip_payload_mlp(args, nargs, reinterpret_cast<const lh_mlp_attrs*>(attrs));
      default: return lh_hip_payload_gpt_fused(args, nargs, reinterpret_cast<const lh_gpt_fused_attrs*>(attrs));
    }
  };
  for (int64_t i = 0; i < nwarmup; ++i) {
    int rc = call();
    if (rc) return rc;
  }
  for (int64_t i = 0; i < nruns; ++i) {
    auto t0 = std::chrono::steady_clock::now();
    int rc = call();
    auto t1 = std::chrono::steady_clock::now();
    if (rc) return rc;
    host_times[i] = std::chrono::duration<double>(t1 - t0).count();
  }
  return LH_OK;
}

}  // extern "C"
