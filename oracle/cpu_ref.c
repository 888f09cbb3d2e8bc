/*
 * CPU restatement of the loop nests Lighthouse's default CPU lowering produces
 * for the GPU payloads (TEST INFRASTRUCTURE: checker and timed CPU baseline only;
 * never linked into or called from the shipped library).
 *
 * lh-run appends `convert-linalg-to-loops` + the LLVM lowering to every pipeline
 * (lighthouse/lh_run.py:103-107), i.e. each linalg op becomes a plain scalar
 * loop nest: i-j-k for linalg.matmul with a separate f32 multiply and add, one
 * loop nest per elementwise op.  The functions below keep that loop order and
 * those rounding points.  `threads` > 1 parallelises the outermost row loop with
 * OpenMP, the analogue of the `convert-scf-to-openmp` stage of
 * lighthouse/pipeline/descriptors/x86_64/lower.yaml:6.
 *
 * Build: gcc -O3 -march=native -ffp-contract=off -fopenmp -shared -fPIC cpu_ref.c -o libcpu_ref.so -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LHREF_BIAS 1
#define LHREF_RELU 2
#define LHREF_ACCUMULATE_C 4
#define LHREF_GELU 32

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* arith.truncf f32->bf16: round to nearest even, quiet NaN. */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float gelu_tanh_f32(float x) {
  const float k = 0.7978845608028654f; /* sqrt(2/pi) */
  float inner = k * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(inner));
}

/* OCP e4m3fn code -> float */
static float e4m3_table[256];
static int e4m3_ready = 0;
static void e4m3_init(void) {
  if (e4m3_ready) return;
  for (int c = 0; c < 256; ++c) {
    int e = (c >> 3) & 15, m = c & 7;
    float v;
    if (e == 15 && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m / 8.0f, -6);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    e4m3_table[c] = (c & 0x80) ? -v : v;
  }
  e4m3_ready = 1;
}

/*
 * f32 matmul payload: out = relu?(A.B (+out) (+bias)).
 * emit_mlp_layer, lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:110-156; the
 * generic-form fixture test/opt/pipeline-check.mlir:27-46 has the same three steps.
 */
int lhref_matmul_f32(float* out, const float* a, const float* b, const float* bias, int64_t M, int64_t N,
                     int64_t K, uint32_t flags, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      float acc = (flags & LHREF_ACCUMULATE_C) ? out[i * N + j] : 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float p = a[i * K + k] * b[k * N + j];
        acc = acc + p;
      }
      if (flags & LHREF_BIAS) acc = bias[j] + acc;
      if (flags & LHREF_GELU) acc = gelu_tanh_f32(acc);
      if (flags & LHREF_RELU) acc = acc > 0.0f ? acc : (acc != acc ? acc : 0.0f);
      out[i * N + j] = acc;
    }
  }
  return 0;
}

/*
 * bf16 A/B, f32 accumulation, bf16 bias extended to f32, result truncated to bf16,
 * ReLU applied in bf16 (gpu_mlp_payload.py:142-151 order: bias, convert, relu).
 */
int lhref_matmul_bf16(uint16_t* out, const uint16_t* a, const uint16_t* b, const uint16_t* bias, int64_t M,
                      int64_t N, int64_t K, uint32_t flags, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      float acc = (flags & LHREF_ACCUMULATE_C) ? bf16_to_f32(out[i * N + j]) : 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float p = bf16_to_f32(a[i * K + k]) * bf16_to_f32(b[k * N + j]);
        acc = acc + p;
      }
      if (flags & LHREF_BIAS) acc = bf16_to_f32(bias[j]) + acc;
      if (flags & LHREF_GELU) acc = gelu_tanh_f32(acc);
      uint16_t r = f32_to_bf16(acc);
      if ((flags & LHREF_RELU) && (r & 0x8000) && (r & 0x7fff) <= 0x7f80) r = 0;
      out[i * N + j] = r;
    }
  }
  return 0;
}

/*
 * The same two payloads cache-tiled: the CPU analogue of the reference's optimising matmul
 * pipeline (pack, tile, register-tile, vectorise: lighthouse/pipeline/descriptors/x86_64/matmul/
 * f32.yaml:1-17) with the OpenMP stage of x86_64/lower.yaml:6 over row blocks.  Each thread takes
 * blocks of TM rows; for a block and a strip of TN columns the f32 accumulators live in a
 * thread-private tile and K is walked in chunks of TK (the TK x TN piece of B stays in the cache
 * across the block's rows; the innermost loop runs along columns and vectorises).  Every output
 * element still adds its products one at a time in increasing k, multiply and add separate, so the
 * results equal the plain loop nests' bit for bit.
 */
#define LHREF_TM 32
#define LHREF_TN 512
#define LHREF_TK 128

int lhref_matmul_f32_tiled(float* out, const float* a, const float* b, const float* bias, int64_t M, int64_t N,
                           int64_t K, uint32_t flags, int threads) {
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
  for (int64_t i0 = 0; i0 < M; i0 += LHREF_TM) {
    float acc[LHREF_TM][LHREF_TN];
    const int64_t mi = (M - i0 < LHREF_TM) ? M - i0 : LHREF_TM;
    for (int64_t j0 = 0; j0 < N; j0 += LHREF_TN) {
      const int64_t nj = (N - j0 < LHREF_TN) ? N - j0 : LHREF_TN;
      for (int64_t i = 0; i < mi; ++i)
        for (int64_t j = 0; j < nj; ++j) acc[i][j] = (flags & LHREF_ACCUMULATE_C) ? out[(i0 + i) * N + j0 + j] : 0.0f;
      for (int64_t k0 = 0; k0 < K; k0 += LHREF_TK) {
        const int64_t nk = (K - k0 < LHREF_TK) ? K - k0 : LHREF_TK;
        for (int64_t i = 0; i < mi; ++i)
          for (int64_t k = 0; k < nk; ++k) {
            const float av = a[(i0 + i) * K + k0 + k];
            const float* brow = b + (k0 + k) * N + j0;
            for (int64_t j = 0; j < nj; ++j) {
              float p = av * brow[j];
              acc[i][j] = acc[i][j] + p;
            }
          }
      }
      for (int64_t i = 0; i < mi; ++i)
        for (int64_t j = 0; j < nj; ++j) {
          float v = acc[i][j];
          if (flags & LHREF_BIAS) v = bias[j0 + j] + v;
          if (flags & LHREF_GELU) v = gelu_tanh_f32(v);
          if (flags & LHREF_RELU) v = v > 0.0f ? v : (v != v ? v : 0.0f);
          out[(i0 + i) * N + j0 + j] = v;
        }
    }
  }
  return 0;
}

int lhref_matmul_bf16_tiled(uint16_t* out, const uint16_t* a, const uint16_t* b, const uint16_t* bias, int64_t M,
                            int64_t N, int64_t K, uint32_t flags, int threads) {
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
  for (int64_t i0 = 0; i0 < M; i0 += LHREF_TM) {
    float acc[LHREF_TM][LHREF_TN];
    float bt[LHREF_TK][LHREF_TN]; /* the B piece extended to f32 once per block */
    const int64_t mi = (M - i0 < LHREF_TM) ? M - i0 : LHREF_TM;
    for (int64_t j0 = 0; j0 < N; j0 += LHREF_TN) {
      const int64_t nj = (N - j0 < LHREF_TN) ? N - j0 : LHREF_TN;
      for (int64_t i = 0; i < mi; ++i)
        for (int64_t j = 0; j < nj; ++j)
          acc[i][j] = (flags & LHREF_ACCUMULATE_C) ? bf16_to_f32(out[(i0 + i) * N + j0 + j]) : 0.0f;
      for (int64_t k0 = 0; k0 < K; k0 += LHREF_TK) {
        const int64_t nk = (K - k0 < LHREF_TK) ? K - k0 : LHREF_TK;
        for (int64_t k = 0; k < nk; ++k)
          for (int64_t j = 0; j < nj; ++j) bt[k][j] = bf16_to_f32(b[(k0 + k) * N + j0 + j]);
        for (int64_t i = 0; i < mi; ++i)
          for (int64_t k = 0; k < nk; ++k) {
            const float av = bf16_to_f32(a[(i0 + i) * K + k0 + k]);
            for (int64_t j = 0; j < nj; ++j) {
              float p = av * bt[k][j];
              acc[i][j] = acc[i][j] + p;
            }
          }
      }
      for (int64_t i = 0; i < mi; ++i)
        for (int64_t j = 0; j < nj; ++j) {
          float v = acc[i][j];
          if (flags & LHREF_BIAS) v = bf16_to_f32(bias[j0 + j]) + v;
          if (flags & LHREF_GELU) v = gelu_tanh_f32(v);
          uint16_t r = f32_to_bf16(v);
          if ((flags & LHREF_RELU) && (r & 0x8000) && (r & 0x7fff) <= 0x7f80) r = 0;
          out[(i0 + i) * N + j0 + j] = r;
        }
    }
  }
  return 0;
}

/* fp8 e4m3 GEMM with per-tensor scales: bf16((Aq.Bq)_f32 * (sa*sb)). */
int lhref_matmul_fp8(uint16_t* out, const uint8_t* a, const uint8_t* b, float scale_a, float scale_b, int64_t M,
                     int64_t N, int64_t K, int threads) {
  e4m3_init();
  const float s = scale_a * scale_b;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) acc = acc + e4m3_table[a[i * K + k]] * e4m3_table[b[k * N + j]];
      out[i * N + j] = f32_to_bf16(acc * s);
    }
  }
  return 0;
}

/*
 * Attention payload, one (batch*head) problem after another, contiguous [BH,T,d].
 * Op sequence of generate_gpu_attention_payload
 * (lighthouse/ingress/mlir_gen/gpu_attention_payload.py:78-125): scores = Q.K^T,
 * scaled, row softmax (max, exp, sum, divide), times V; statistics in f32 as in
 * the fused rewrite (replace_with_fused_attention.py:332-344).  `causal` adds -inf
 * above the diagonal (examples/xegpu/nanoGPT.py:102-109).  elt: 0 = f32 storage,
 * 1 = bf16 storage (uint16) with probabilities rounded to bf16 before P.V.
 */
int lhref_attention(void* out_, const void* q_, const void* k_, const void* v_, int64_t BH, int64_t T,
                    int64_t d, float scale, int causal, int elt, int threads) {
#pragma omp parallel for num_threads(threads) schedule(dynamic, 8) collapse(2)
  for (int64_t bh = 0; bh < BH; ++bh) {
    for (int64_t i = 0; i < T; ++i) {
      float* s = (float*)malloc(sizeof(float) * (size_t)T);
      float* o = (float*)malloc(sizeof(float) * (size_t)d);
      const int64_t base = bh * T * d;
      int64_t jend = causal ? i + 1 : T;
      float m = -INFINITY;
      for (int64_t j = 0; j < jend; ++j) {
        float acc = 0.0f;
        for (int64_t c = 0; c < d; ++c) {
          float qv = elt ? bf16_to_f32(((const uint16_t*)q_)[base + i * d + c]) : ((const float*)q_)[base + i * d + c];
          float kv = elt ? bf16_to_f32(((const uint16_t*)k_)[base + j * d + c]) : ((const float*)k_)[base + j * d + c];
          acc = acc + qv * kv;
        }
        s[j] = acc * scale;
        m = s[j] > m ? s[j] : m;
      }
      float l = 0.0f;
      for (int64_t j = 0; j < jend; ++j) {
        s[j] = expf(s[j] - m);
        l = l + s[j];
      }
      for (int64_t c = 0; c < d; ++c) o[c] = 0.0f;
      for (int64_t j = 0; j < jend; ++j) {
        float p = elt ? bf16_to_f32(f32_to_bf16(s[j])) : s[j];
        for (int64_t c = 0; c < d; ++c) {
          float vv = elt ? bf16_to_f32(((const uint16_t*)v_)[base + j * d + c]) : ((const float*)v_)[base + j * d + c];
          o[c] = o[c] + p * vv;
        }
      }
      for (int64_t c = 0; c < d; ++c) {
        float r = o[c] / l;
        if (elt) ((uint16_t*)out_)[base + i * d + c] = f32_to_bf16(r);
        else ((float*)out_)[base + i * d + c] = r;
      }
      free(s);
      free(o);
    }
  }
  return 0;
}

/*
 * Row LayerNorm, the three loop nests of emit_layer_norm_generics
 * (lighthouse/ingress/mlir_gen/gpu_layer_norm_payload.py:15-87): row sum, sum of
 * squared centred values with mean = sum * (1/N), then
 * (x-mean) * rsqrt(var*(1/N)+eps) * gamma + beta.  (1/N) is a pre-rounded f32 constant.
 */
int lhref_layer_norm_f32(float* out, const float* x, const float* gamma, const float* beta, int64_t M, int64_t N,
                         float eps, int threads) {
  const float inv_n = (float)(1.0 / (double)N);
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    float s = 0.0f;
    for (int64_t j = 0; j < N; ++j) s = x[i * N + j] + s;
    float mean = s * inv_n;
    float v = 0.0f;
    for (int64_t j = 0; j < N; ++j) {
      float c = x[i * N + j] - mean;
      v = c * c + v;
    }
    float inv_std = 1.0f / sqrtf(v * inv_n + eps);
    for (int64_t j = 0; j < N; ++j) out[i * N + j] = (x[i * N + j] - mean) * inv_std * gamma[j] + beta[j];
  }
  return 0;
}

/* Elementwise tanh-GELU in f32. */
int lhref_gelu_tanh_f32(float* out, const float* x, int64_t n, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = gelu_tanh_f32(x[i]);
  return 0;
}

/* Row softmax in f32 (lighthouse/ingress/mlir_gen/gpu_softmax_payload.py:46-55). */
int lhref_softmax_f32(float* out, const float* x, int64_t M, int64_t N, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    float m = -INFINITY;
    for (int64_t j = 0; j < N; ++j) m = x[i * N + j] > m ? x[i * N + j] : m;
    float l = 0.0f;
    for (int64_t j = 0; j < N; ++j) {
      out[i * N + j] = expf(x[i * N + j] - m);
      l = l + out[i * N + j];
    }
    for (int64_t j = 0; j < N; ++j) out[i * N + j] = out[i * N + j] / l;
  }
  return 0;
}
