// Argument block and register epilogue shared by the GEMM kernels.
#pragma once

#include "common.h"

namespace lh {

struct GemmArgs {
  void* out;
  const void* c;  // accumulator input for ACCUMULATE_C (out_dt typed; may alias out)
  const void* a;
  const void* b;
  const void* bias;
  int M, N, K;
  int64_t lda, ldb, ldc;
  uint32_t flags;
  int out_dt;
  int bias_dt;  // element type of bias
  float alpha;  // accumulator scale applied first (1 for the unquantised payloads)
  // Split-K launches of the 16-bit direct kernel: `splits` problems of K columns each, problem sp reads
  // A from column sp K, B from row sp K and writes its own M x ldc block of `out`.
  int splits = 1;
  // Source of the call's temporary device memory; nullptr: the library's pool of the stream.
  Scratch* ws = nullptr;
  // 16-bit direct kernel, 128 x 128 tile: main loop with one barrier per 64 k (set by the launcher
  // when more than one workgroup falls on a compute unit).
  int one_barrier = 0;
};

// Epilogue for 4 consecutive columns of one row.
template <int DT>
__device__ __forceinline__ void epilogue4(const GemmArgs& g, int m, int n, float v0, float v1, float v2, float v3) {
  float v[4] = {v0 * g.alpha, v1 * g.alpha, v2 * g.alpha, v3 * g.alpha};
  const int64_t off = (int64_t)m * g.ldc + n;
  if (g.flags & LH_GEMM_ACCUMULATE_C) {
    if (g.out_dt == LH_F32) {
      f32x4 c = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(g.c) + off);
      v[0] += c[0]; v[1] += c[1]; v[2] += c[2]; v[3] += c[3];
    } else {
      u32x2 c = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g.c) + off);
      v[0] += unpack_lo<DT>(c[0]); v[1] += unpack_hi<DT>(c[0]);
      v[2] += unpack_lo<DT>(c[1]); v[3] += unpack_hi<DT>(c[1]);
    }
  }
  if (g.flags & LH_GEMM_HAS_BIAS) {
    if (g.bias_dt == LH_F32) {
      f32x4 bb = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(g.bias) + n);
      v[0] += bb[0]; v[1] += bb[1]; v[2] += bb[2]; v[3] += bb[3];
    } else {
      u32x2 bb = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g.bias) + n);
      v[0] += unpack_lo<DT>(bb[0]); v[1] += unpack_hi<DT>(bb[0]);
      v[2] += unpack_lo<DT>(bb[1]); v[3] += unpack_hi<DT>(bb[1]);
    }
  }
  if (g.flags & LH_GEMM_HAS_GELU) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
  }
  const bool relu = (g.flags & LH_GEMM_HAS_RELU) != 0;
  if (g.out_dt == LH_F32) {
    if (relu) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = relu_nan(v[e]);
    }
    f32x4 o = {v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(g.out) + off) = o;
  } else {
    if (relu) {
      // ReLU is applied after the conversion (gpu_mlp_payload.py:147-151); max(x,0) and
      // rounding commute for every input (0 is representable and rounding is monotone).
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = relu_nan(v[e]);
    }
    u32x2 o = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
    *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(g.out) + off) = o;
  }
}

// Bias of 4 consecutive columns as f32 (zeros without a bias).
template <int DT>
__device__ __forceinline__ f32x4 bias4(const GemmArgs& g, int n) {
  f32x4 r = {0.0f, 0.0f, 0.0f, 0.0f};
  if (g.flags & LH_GEMM_HAS_BIAS) {
    if (g.bias_dt == LH_F32) {
      r = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(g.bias) + n);
    } else {
      u32x2 bb = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g.bias) + n);
      r = f32x4{unpack_lo<DT>(bb[0]), unpack_hi<DT>(bb[0]), unpack_lo<DT>(bb[1]), unpack_hi<DT>(bb[1])};
    }
  }
  return r;
}

// ---- epilogue variants fixed at compile time ----------------------------------------------
// epilogue4 tests the flags of the call for every group of 4 elements.  In a tile
// kernel whose epilogue is unrolled over the tile that is a handful of scalar branches around a
// few vector instructions, a hundred times over, in code that runs once per tile and is cold in
// the instruction cache each time: the 256 x 256 bf16 tile spent 5.2 us converting and staging
// 128 KiB of output that way, 2.5 us without the tests.  The tile kernels therefore choose ONE
// variant per tile (epi_dispatch: a chain of wave-uniform branches at the top of the epilogue)
// and run straight-line code specialised for it; EpiAny keeps the run-time tests for the
// combinations that have no variant of their own.  Same operations in the same order either way
// (a scale of exactly 1 is skipped: x * 1 == x bit for bit).
template <bool ALPHA, bool BIAS, int ACT>  // ACT: 0 none, 1 ReLU, 2 tanh-GELU
struct EpiFixed {
  static constexpr bool kAny = false, kAlpha = ALPHA, kBias = BIAS;
  static constexpr int kAct = ACT;
};
struct EpiAny {
  static constexpr bool kAny = true, kAlpha = true, kBias = true;
  static constexpr int kAct = -1;
};
template <typename E>
__device__ __forceinline__ bool epi_has_bias(const GemmArgs& g) {
  if constexpr (E::kAny) return (g.flags & LH_GEMM_HAS_BIAS) != 0;
  else return E::kBias;
}
// Scale, bias and activation on 4 values, in epilogue4's order.
template <typename E>
__device__ __forceinline__ void epi_apply4(const GemmArgs& g, const f32x4& bias, float (&v)[4]) {
  if constexpr (E::kAny) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= g.alpha;
    if (g.flags & LH_GEMM_HAS_BIAS) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += bias[e];
    }
    if (g.flags & LH_GEMM_HAS_GELU) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
    }
    if (g.flags & LH_GEMM_HAS_RELU) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = relu_nan(v[e]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if constexpr (E::kAlpha) v[e] *= g.alpha;
      if constexpr (E::kBias) v[e] += bias[e];
      if constexpr (E::kAct == 2) v[e] = gelu_tanh(v[e]);
      if constexpr (E::kAct == 1) v[e] = relu_nan(v[e]);
    }
  }
}
// 4 accumulator values -> two packed dwords of a 16-bit output (no accumulator input).
template <int DT, typename E>
__device__ __forceinline__ u32x2 epi_pack4(const GemmArgs& g, const f32x4& bias, const f32x4& a) {
  float v[4] = {a[0], a[1], a[2], a[3]};
  epi_apply4<E>(g, bias, v);
  return u32x2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
}
// Calls f with the variant of the call: unscaled accumulators without a bias, with a bias, with a
// bias followed by ReLU or GELU, scaled accumulators without a bias (the fp8 payload); anything
// else takes EpiAny.
template <typename F>
__device__ __forceinline__ void epi_dispatch(const GemmArgs& g, F&& f) {
  const uint32_t k = g.flags & (LH_GEMM_HAS_BIAS | LH_GEMM_HAS_GELU | LH_GEMM_HAS_RELU);
  if (g.alpha == 1.0f) {
    if (k == 0) return f(EpiFixed<false, false, 0>{});
    if (k == LH_GEMM_HAS_BIAS) return f(EpiFixed<false, true, 0>{});
    if (k == (LH_GEMM_HAS_BIAS | LH_GEMM_HAS_RELU)) return f(EpiFixed<false, true, 1>{});
    if (k == (LH_GEMM_HAS_BIAS | LH_GEMM_HAS_GELU)) return f(EpiFixed<false, true, 2>{});
  } else if (k == 0) {
    return f(EpiFixed<true, false, 0>{});
  }
  f(EpiAny{});
}
// The same without the activation variants, for epilogues that also specialise on the output
// type and the accumulator input (residual adds, f32 outputs, split-K blocks).
template <typename F>
__device__ __forceinline__ void epi_dispatch_linear(const GemmArgs& g, F&& f) {
  const uint32_t k = g.flags & (LH_GEMM_HAS_BIAS | LH_GEMM_HAS_GELU | LH_GEMM_HAS_RELU);
  if (g.alpha == 1.0f) {
    if (k == 0) return f(EpiFixed<false, false, 0>{});
    if (k == LH_GEMM_HAS_BIAS) return f(EpiFixed<false, true, 0>{});
  }
  f(EpiAny{});
}
// epilogue4 with the variant, the output type and the presence of an accumulator input fixed.
template <int DT, typename E, bool OUT32, bool HAS_C>
__device__ __forceinline__ void epi_store4(const GemmArgs& g, int m, int n, const f32x4& bias, const f32x4& a) {
  float v[4] = {a[0], a[1], a[2], a[3]};
  const int64_t off = (int64_t)m * g.ldc + n;
  if constexpr (HAS_C) {
    // (the accumulator input is added to the scaled accumulator before the bias, as in epilogue4)
    if constexpr (E::kAlpha) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] *= g.alpha;
    }
    if constexpr (OUT32) {
      const f32x4 c = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(g.c) + off);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += c[e];
    } else {
      const u32x2 c = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g.c) + off);
      v[0] += unpack_lo<DT>(c[0]); v[1] += unpack_hi<DT>(c[0]);
      v[2] += unpack_lo<DT>(c[1]); v[3] += unpack_hi<DT>(c[1]);
    }
    if constexpr (E::kAny) {
      if (g.flags & LH_GEMM_HAS_BIAS) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += bias[e];
      }
      if (g.flags & LH_GEMM_HAS_GELU) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
      }
      if (g.flags & LH_GEMM_HAS_RELU) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = relu_nan(v[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (E::kBias) v[e] += bias[e];
        if constexpr (E::kAct == 2) v[e] = gelu_tanh(v[e]);
        if constexpr (E::kAct == 1) v[e] = relu_nan(v[e]);
      }
    }
  } else {
    epi_apply4<E>(g, bias, v);
  }
  if constexpr (OUT32)
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(g.out) + off) = f32x4{v[0], v[1], v[2], v[3]};
  else
    *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(g.out) + off) = u32x2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
}

// Transposed operands (A stored [K,M], B stored [N,K]) of a problem the direct kernels would
// otherwise take are first transposed into temporary memory (one extra pass over that
// operand, about a tenth of a 4096^3 problem's time) instead of running the slower kernels that
// read them in place.  Returns 0 and rewrites `g` on success, 1 when the problem does not qualify.
template <int ELEM_BYTES>
inline int untranspose_operands(GemmArgs& g, int k_multiple, int n_multiple, hipStream_t s) {
  const bool ta = g.flags & LH_GEMM_TRANSPOSE_A, tb = g.flags & LH_GEMM_TRANSPOSE_B;
  if (!(ta || tb) || g.K % k_multiple != 0 || g.N % n_multiple != 0) return 1;
  const size_t a_bytes = ta ? ((size_t)g.M * g.K * ELEM_BYTES + 255) / 256 * 256 : 0;
  const size_t b_bytes = tb ? (size_t)g.K * g.N * ELEM_BYTES : 0;
  void* taken = nullptr;
  if (int rc = scratch_take(g.ws, s, kScratchTranspose, a_bytes + b_bytes, "gemm (transposed operands)", &taken)) return rc;
  char* buf = static_cast<char*>(taken);
  if (ta) {  // stored [K, M] -> [M, K]
    if (int rc = transpose_matrix(buf, g.a, g.K, g.M, g.lda, g.K, ELEM_BYTES, s)) return rc;
    g.a = buf;
    g.lda = g.K;
  }
  if (tb) {  // stored [N, K] -> [K, N]
    if (int rc = transpose_matrix(buf + a_bytes, g.b, g.N, g.K, g.ldb, g.N, ELEM_BYTES, s)) return rc;
    g.b = buf + a_bytes;
    g.ldb = g.N;
  }
  g.flags &= ~(uint32_t)(LH_GEMM_TRANSPOSE_A | LH_GEMM_TRANSPOSE_B);
  return 0;
}

// A problem whose K or N the direct kernels cannot take (K not a multiple of the k-step, N not a
// multiple of the vector width, or rows that are not 16-byte aligned) runs on them all the same:
// A and B are copied into temporary matrices padded with zeros, the kernel writes a padded
// result, and that is copied back (bf16 4096 x 4100 x 4096: 2012 -> about 200 us; the generic
// kernel it replaces reads element by element).  `run` launches the padded problem.  Returns 1
// when nothing needs padding, a negative status on failure.
template <int ELEM_BYTES, typename Run>
inline int gemm_padded(const GemmArgs& g, int k_multiple, int n_multiple, hipStream_t s, Run run) {
  const bool ta = g.flags & LH_GEMM_TRANSPOSE_A, tb = g.flags & LH_GEMM_TRANSPOSE_B;
  const int out_bytes = g.out_dt == LH_F32 ? 4 : 2, bias_bytes = g.bias_dt == LH_F32 ? 4 : 2;
  const int Kp = (g.K + k_multiple - 1) / k_multiple * k_multiple;
  const int Np = (g.N + n_multiple - 1) / n_multiple * n_multiple;
  const bool has_bias = g.flags & LH_GEMM_HAS_BIAS, acc = g.flags & LH_GEMM_ACCUMULATE_C;
  // (a transposed operand is copied in any case: the copy is where it gets untransposed)
  const bool pad_a = ta || Kp != g.K || g.lda % (16 / ELEM_BYTES) != 0 || !aligned16(g.a);
  const bool pad_b = tb || Kp != g.K || Np != g.N || g.ldb % (16 / ELEM_BYTES) != 0 || !aligned16(g.b);
  const bool pad_c = Np != g.N || g.ldc % n_multiple != 0 || !aligned16(g.out) || (acc && !aligned16(g.c));
  const bool pad_bias = has_bias && (Np != g.N || !aligned16(g.bias));
  if (!(pad_a || pad_b || pad_c || pad_bias)) return 1;
  auto round256 = [](size_t b) { return (b + 255) / 256 * 256; };
  const size_t a_bytes = pad_a ? round256((size_t)g.M * Kp * ELEM_BYTES) : 0;
  const size_t b_bytes = pad_b ? round256((size_t)Kp * Np * ELEM_BYTES) : 0;
  const size_t c_bytes = pad_c ? round256((size_t)g.M * Np * out_bytes) : 0;
  const size_t bias_bytes_total = pad_bias ? round256((size_t)Np * bias_bytes) : 0;
  void* taken = nullptr;
  if (int rc = scratch_take(g.ws, s, kScratchPad, a_bytes + b_bytes + c_bytes + bias_bytes_total, "gemm (padded operands)",
                            &taken))
    return rc;
  char* buf = static_cast<char*>(taken);
  GemmArgs p = g;
  p.K = Kp;
  p.N = Np;
  if (pad_a) {
    if (ta) {  // stored [K, M]: zeros first (the padding), then the transposed matrix on top
      if (Kp != g.K)
        if (int rc = pad_copy_matrix(buf, Kp, g.M, Kp, g.a, g.lda, 0, 0, ELEM_BYTES, s)) return rc;
      if (int rc = transpose_matrix(buf, g.a, g.K, g.M, g.lda, Kp, ELEM_BYTES, s)) return rc;
    } else if (int rc = pad_copy_matrix(buf, Kp, g.M, Kp, g.a, g.lda, g.M, g.K, ELEM_BYTES, s)) {
      return rc;
    }
    p.a = buf;
    p.lda = Kp;
  }
  if (pad_b) {
    char* bp = buf + a_bytes;
    if (tb) {  // stored [N, K]
      if (Kp != g.K || Np != g.N)
        if (int rc = pad_copy_matrix(bp, Np, Kp, Np, g.b, g.ldb, 0, 0, ELEM_BYTES, s)) return rc;
      if (int rc = transpose_matrix(bp, g.b, g.N, g.K, g.ldb, Np, ELEM_BYTES, s)) return rc;
    } else if (int rc = pad_copy_matrix(bp, Np, Kp, Np, g.b, g.ldb, g.K, g.N, ELEM_BYTES, s)) {
      return rc;
    }
    p.b = bp;
    p.ldb = Np;
  }
  p.flags &= ~(uint32_t)(LH_GEMM_TRANSPOSE_A | LH_GEMM_TRANSPOSE_B);
  if (pad_c) {
    char* cp = buf + a_bytes + b_bytes;
    if (acc)
      if (int rc = pad_copy_matrix(cp, Np, g.M, Np, g.c, g.ldc, g.M, g.N, out_bytes, s)) return rc;
    p.out = cp;
    p.c = cp;
    p.ldc = Np;
  }
  if (pad_bias) {
    char* bp = buf + a_bytes + b_bytes + c_bytes;
    if (int rc = pad_copy_matrix(bp, Np, 1, Np, g.bias, g.N, 1, g.N, bias_bytes, s)) return rc;
    p.bias = bp;
  }
  if (int rc = run(p)) return rc;
  if (pad_c) return pad_copy_matrix(g.out, g.ldc, g.M, g.N, p.out, Np, g.M, g.N, out_bytes, s);
  return LH_OK;
}

// Sum over the f32 blocks of a split-K launch for 4 consecutive columns: p + sp * step, sp = 0 ..
// splits - 1, added in that order.  `deep`: up to 8 loads are in flight before the first add, for the
// small reductions (a few MiB spread over every CU) that are bound by latency alone; large ones
// are faster with one block at a time (8 streams several MiB apart: 41 -> 43 us at 256 x 8192 x 8).
__device__ __forceinline__ f32x4 splitk_sum4(const float* p, int64_t step, int splits, bool deep) {
  f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
  if (!deep) {
    for (int sp = 0; sp < splits; ++sp) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(p + sp * step);
      v[0] += t[0]; v[1] += t[1]; v[2] += t[2]; v[3] += t[3];
    }
    return v;
  }
  int sp = 0;
  for (; sp + 8 <= splits; sp += 8) {
    f32x4 t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) t[u] = *reinterpret_cast<const f32x4*>(p + (sp + u) * step);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      v[0] += t[u][0]; v[1] += t[u][1]; v[2] += t[u][2]; v[3] += t[u][3];
    }
  }
  for (; sp < splits; ++sp) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p + sp * step);
    v[0] += t[0]; v[1] += t[1]; v[2] += t[2]; v[3] += t[3];
  }
  return v;
}

// Workgroup size of a reduce kernel over `groups` 4-column groups: one wave per workgroup while
// that still gives every CU only a few of them (decode batches up to 32 rows of 8192), else 256.
static inline int reduce_block(int64_t groups) { return groups <= 64 * 1024 ? 64 : 256; }

// One output element, any alignment (edge tiles and the generic kernels).
template <int DT>
__device__ __forceinline__ void epilogue1(const GemmArgs& g, int m, int n, float x) {
  const int64_t off = (int64_t)m * g.ldc + n;
  x *= g.alpha;
  if (g.flags & LH_GEMM_ACCUMULATE_C)
    x += (g.out_dt == LH_F32) ? reinterpret_cast<const float*>(g.c)[off] : load_as_f32<DT>(g.c, off);
  if (g.flags & LH_GEMM_HAS_BIAS)
    x += (g.bias_dt == LH_F32) ? reinterpret_cast<const float*>(g.bias)[n] : load_as_f32<DT>(g.bias, n);
  if (g.flags & LH_GEMM_HAS_GELU) x = gelu_tanh(x);
  if (g.flags & LH_GEMM_HAS_RELU) x = relu_nan(x);
  if (g.out_dt == LH_F32) reinterpret_cast<float*>(g.out)[off] = x;
  else store_from_f32<DT>(g.out, off, x);
}

int gemm16(const GemmArgs& g, int ab_dtype, hipStream_t s);
int gemm32(const GemmArgs& g, hipStream_t s);
int gemm8(const GemmArgs& g, hipStream_t s);

}  // namespace lh
