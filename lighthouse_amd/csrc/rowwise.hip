// Bandwidth-bound row and elementwise kernels: LayerNorm, softmax, tanh-GELU, bias(+ReLU),
// residual add, conversion.  One pass over HBM each: a row lives in registers between the
// reduction passes, every global access is 8 or 16 bytes per lane and contiguous across the
// wave.
#include "common.h"

namespace lh {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// 4 consecutive elements as floats.
template <int DT>
__device__ __forceinline__ f32x4 load4(const void* p, int64_t i) {
  if constexpr (DT == LH_F32) {
    return *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p) + i);
  } else {
    u32x2 w = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(p) + i);
    return f32x4{unpack_lo<DT>(w[0]), unpack_hi<DT>(w[0]), unpack_lo<DT>(w[1]), unpack_hi<DT>(w[1])};
  }
}
template <int DT>
__device__ __forceinline__ void store4(void* p, int64_t i, f32x4 v) {
  if constexpr (DT == LH_F32) {
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p) + i) = v;
  } else {
    u32x2 w = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
    *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(p) + i) = w;
  }
}

// The same through a non-temporal store.  A stand-alone bandwidth kernel whose output nothing on the
// device reads next leaves less dirty data in the L2s for the end-of-kernel write-back (LayerNorm
// [8192, 768] f32 -> f32 12.5 -> 11.1 us, f32 -> bf16 9.0 -> 8.4 us, GELU [8192, 3072] 37.7 -> 35.4 us
// on rotating buffers); inside the nanoGPT block, where the next GEMM reads the rows at once, it
// cost 1 % and is not used.
template <int DT>
__device__ __forceinline__ void store4_streaming(void* p, int64_t i, f32x4 v) {
  if constexpr (DT == LH_F32) {
    __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p) + i));
  } else {
    u32x2 w = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(p) + i));
  }
}

// LayerNorm, one wave per row, N = VPL * 256 exactly; the three loop nests of
// emit_layer_norm_generics (lighthouse/ingress/mlir_gen/gpu_layer_norm_payload.py:15-87)
// evaluated on the register-resident row: sum -> mean = sum * (1/N); sum of squared centred
// values -> var = that * (1/N); (x - mean) * rsqrt(var + eps) * gamma + beta.
// A wave takes RPW rows (r, r + rows/RPW ...): all of them, gamma and beta are requested up
// front, so that the loads of a later row and the stores of an earlier one overlap.
// GUARD: N is any multiple of 4 up to 256 VPL; element groups past the end are neither loaded,
// counted nor stored (hidden sizes such as 384, 640 or 1280).
// STREAM: non-temporal stores (a template parameter: as a run-time choice the compiler merges the two
// stores into a plain one).
template <int XDT, int ODT, int VPL, int RPW, bool GUARD = false, bool STREAM = false>
__global__ void __launch_bounds__(256) layer_norm_vec(void* out, const void* x, const float* gamma, const float* beta,
                                                      int M, int N, float eps, float inv_n) {
  const int lane = threadIdx.x & 63;
  const int slots = (M + RPW - 1) / RPW;  // waves in the grid that have work
  const int slot = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (slot >= slots) return;
  f32x4 v[RPW][VPL];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int row = min(slot + r * slots, M - 1);  // a row past the end repeats the last one and is not stored
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      v[r][i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (!GUARD || (i * 64 + lane) * 4 < N) v[r][i] = load4<XDT>(x, (int64_t)row * N + (i * 64 + lane) * 4);
    }
  }
  f32x4 g[VPL], b[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    g[i] = b[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (!GUARD || (i * 64 + lane) * 4 < N) {
      g[i] = *reinterpret_cast<const f32x4*>(gamma + (i * 64 + lane) * 4);
      b[i] = *reinterpret_cast<const f32x4*>(beta + (i * 64 + lane) * 4);
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int row = slot + r * slots;
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) s += (v[r][i][0] + v[r][i][1]) + (v[r][i][2] + v[r][i][3]);
    const float mean = wave_sum(s) * inv_n;
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      if (GUARD && (i * 64 + lane) * 4 >= N) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float c = v[r][i][e] - mean;
        q += c * c;
      }
    }
    const float inv_std = rsqrtf(wave_sum(q) * inv_n + eps);
    if (row < M) {
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        if (GUARD && (i * 64 + lane) * 4 >= N) continue;
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (v[r][i][e] - mean) * inv_std * g[i][e] + b[i][e];
        if constexpr (STREAM) store4_streaming<ODT>(out, (int64_t)row * N + (i * 64 + lane) * 4, o);
        else store4<ODT>(out, (int64_t)row * N + (i * 64 + lane) * 4, o);
      }
    }
  }
}

// Any N: one wave per row, three passes over the row (re-read from cache).
template <int XDT, int ODT>
__global__ void __launch_bounds__(256) layer_norm_generic(void* out, const void* x, const float* gamma,
                                                          const float* beta, int M, int N, float eps, float inv_n) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int64_t base = (int64_t)row * N;
  float s = 0.0f;
  for (int j = lane; j < N; j += 64) s += load_as_f32<XDT>(x, base + j);
  const float mean = wave_sum(s) * inv_n;
  float q = 0.0f;
  for (int j = lane; j < N; j += 64) {
    float c = load_as_f32<XDT>(x, base + j) - mean;
    q += c * c;
  }
  const float inv_std = rsqrtf(wave_sum(q) * inv_n + eps);
  for (int j = lane; j < N; j += 64)
    store_from_f32<ODT>(out, base + j, (load_as_f32<XDT>(x, base + j) - mean) * inv_std * gamma[j] + beta[j]);
}

// Row softmax with the row resident in registers (N = 256 VPL): one read and one write per
// element, one exp per element.
template <int DT, int VPL, bool GUARD = false>
__global__ void __launch_bounds__(256) softmax_rows_vec(void* out, const void* x, int M, int N) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int64_t base = (int64_t)row * N;
  f32x4 v[VPL];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    v[i] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};  // (GUARD: groups past the end count as exp(-inf) = 0)
    if (!GUARD || (i * 64 + lane) * 4 < N) v[i] = load4<DT>(x, base + (i * 64 + lane) * 4);
    mx = fmaxf(fmaxf(mx, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
  }
  mx = wave_max(mx);
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < VPL; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[i][e] = expf(v[i][e] - mx);
      s += v[i][e];
    }
  s = wave_sum(s);
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = v[i][e] / s;
    if (!GUARD || (i * 64 + lane) * 4 < N) store4<DT>(out, base + (i * 64 + lane) * 4, o);
  }
}

// Row softmax (lighthouse/ingress/mlir_gen/gpu_softmax_payload.py:46-55), one wave per row.
template <int DT>
__global__ void __launch_bounds__(256) softmax_rows(void* out, const void* x, int M, int N) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int64_t base = (int64_t)row * N;
  float mx = -INFINITY;
  for (int j = lane; j < N; j += 64) mx = fmaxf(mx, load_as_f32<DT>(x, base + j));
  mx = wave_max(mx);
  float s = 0.0f;
  for (int j = lane; j < N; j += 64) s += expf(load_as_f32<DT>(x, base + j) - mx);
  s = wave_sum(s);
  for (int j = lane; j < N; j += 64) store_from_f32<DT>(out, base + j, expf(load_as_f32<DT>(x, base + j) - mx) / s);
}

// Long rows (N >= 1024 outside the register-resident cases): one workgroup of 256 threads per row,
// the same three passes with block-wide reductions; the row comes from HBM once and from the cache
// twice.  VEC: rows start 16-byte aligned and N % 4 == 0, 4 elements per access.  One wave per row
// leaves a 50000-column row to 64 lanes and a short matrix to a handful of waves.
__device__ __forceinline__ float block_reduce(float v, bool is_max, float* red) {
  v = is_max ? wave_max(v) : wave_sum(v);
  __syncthreads();  // `red` may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  const float a = red[0], b = red[1], c = red[2], d = red[3];
  return is_max ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
}

template <int XDT, int ODT, bool VEC>
__global__ void __launch_bounds__(256) layer_norm_block(void* out, const void* x, const float* gamma, const float* beta,
                                                        int M, int N, float eps, float inv_n) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * N;
  const int tid = threadIdx.x;
  float s = 0.0f;
  if constexpr (VEC) {
    for (int j = 4 * tid; j < N; j += 1024) {
      const f32x4 v = load4<XDT>(x, base + j);
      s += (v[0] + v[1]) + (v[2] + v[3]);
    }
  } else {
    for (int j = tid; j < N; j += 256) s += load_as_f32<XDT>(x, base + j);
  }
  const float mean = block_reduce(s, false, red) * inv_n;
  float q = 0.0f;
  if constexpr (VEC) {
    for (int j = 4 * tid; j < N; j += 1024) {
      const f32x4 v = load4<XDT>(x, base + j);
#pragma unroll
      for (int e = 0; e < 4; ++e) q += (v[e] - mean) * (v[e] - mean);
    }
  } else {
    for (int j = tid; j < N; j += 256) {
      const float c = load_as_f32<XDT>(x, base + j) - mean;
      q += c * c;
    }
  }
  const float inv_std = rsqrtf(block_reduce(q, false, red) * inv_n + eps);
  if constexpr (VEC) {
    for (int j = 4 * tid; j < N; j += 1024) {
      const f32x4 v = load4<XDT>(x, base + j);
      const f32x4 g = *reinterpret_cast<const f32x4*>(gamma + j), b = *reinterpret_cast<const f32x4*>(beta + j);
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (v[e] - mean) * inv_std * g[e] + b[e];
      store4<ODT>(out, base + j, o);
    }
  } else {
    for (int j = tid; j < N; j += 256)
      store_from_f32<ODT>(out, base + j, (load_as_f32<XDT>(x, base + j) - mean) * inv_std * gamma[j] + beta[j]);
  }
}

// Rows of up to 16384 elements (N % 4 == 0, aligned) stay in the workgroup's registers between
// the passes: 16 groups of 4 elements per thread at most, one read and one write per element.
constexpr int kBlockRegGroups = 16;

template <int XDT, int ODT>
__global__ void __launch_bounds__(256) layer_norm_block_reg(void* out, const void* x, const float* gamma,
                                                            const float* beta, int M, int N, float eps, float inv_n) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * N;
  const int j0 = 4 * threadIdx.x;
  f32x4 v[kBlockRegGroups];
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < kBlockRegGroups; ++i) {
    v[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (j0 + 1024 * i < N) {
      v[i] = load4<XDT>(x, base + j0 + 1024 * i);
      s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
    }
  }
  const float mean = block_reduce(s, false, red) * inv_n;
  float q = 0.0f;
#pragma unroll
  for (int i = 0; i < kBlockRegGroups; ++i)
    if (j0 + 1024 * i < N) {
#pragma unroll
      for (int e = 0; e < 4; ++e) q += (v[i][e] - mean) * (v[i][e] - mean);
    }
  const float inv_std = rsqrtf(block_reduce(q, false, red) * inv_n + eps);
#pragma unroll
  for (int i = 0; i < kBlockRegGroups; ++i)
    if (j0 + 1024 * i < N) {
      const int j = j0 + 1024 * i;
      const f32x4 g = *reinterpret_cast<const f32x4*>(gamma + j), b = *reinterpret_cast<const f32x4*>(beta + j);
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (v[i][e] - mean) * inv_std * g[e] + b[e];
      store4<ODT>(out, base + j, o);
    }
}

template <int DT>
__global__ void __launch_bounds__(256) softmax_block_reg(void* out, const void* x, int M, int N) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * N;
  const int j0 = 4 * threadIdx.x;
  f32x4 v[kBlockRegGroups];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < kBlockRegGroups; ++i)
    if (j0 + 1024 * i < N) {
      v[i] = load4<DT>(x, base + j0 + 1024 * i);
      mx = fmaxf(fmaxf(mx, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
    }
  mx = block_reduce(mx, true, red);
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < kBlockRegGroups; ++i)
    if (j0 + 1024 * i < N) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[i][e] = expf(v[i][e] - mx);
        s += v[i][e];
      }
    }
  s = block_reduce(s, false, red);
#pragma unroll
  for (int i = 0; i < kBlockRegGroups; ++i)
    if (j0 + 1024 * i < N) {
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = v[i][e] / s;
      store4<DT>(out, base + j0 + 1024 * i, o);
    }
}

template <int DT, bool VEC>
__global__ void __launch_bounds__(256) softmax_block(void* out, const void* x, int M, int N) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * N;
  const int tid = threadIdx.x;
  float mx = -INFINITY;
  if constexpr (VEC) {
    for (int j = 4 * tid; j < N; j += 1024) {
      const f32x4 v = load4<DT>(x, base + j);
      mx = fmaxf(fmaxf(mx, fmaxf(v[0], v[1])), fmaxf(v[2], v[3]));
    }
  } else {
    for (int j = tid; j < N; j += 256) mx = fmaxf(mx, load_as_f32<DT>(x, base + j));
  }
  mx = block_reduce(mx, true, red);
  float s = 0.0f;
  if constexpr (VEC) {
    for (int j = 4 * tid; j < N; j += 1024) {
      const f32x4 v = load4<DT>(x, base + j);
#pragma unroll
      for (int e = 0; e < 4; ++e) s += expf(v[e] - mx);
    }
  } else {
    for (int j = tid; j < N; j += 256) s += expf(load_as_f32<DT>(x, base + j) - mx);
  }
  s = block_reduce(s, false, red);
  if constexpr (VEC) {
    for (int j = 4 * tid; j < N; j += 1024) {
      const f32x4 v = load4<DT>(x, base + j);
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = expf(v[e] - mx) / s;
      store4<DT>(out, base + j, o);
    }
  } else {
    for (int j = tid; j < N; j += 256) store_from_f32<DT>(out, base + j, expf(load_as_f32<DT>(x, base + j) - mx) / s);
  }
}

enum { EW_GELU = 0, EW_ADD = 1, EW_BIAS = 2, EW_BIAS_RELU = 3 };

// n4 groups of 4 elements; `N` is the row length for the bias kinds.
template <int DT, int KIND>
__global__ void __launch_bounds__(256) elementwise4(void* out, const void* a, const void* b, int64_t n4, int N) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
    f32x4 x = load4<DT>(a, i * 4);
    f32x4 o;
    if constexpr (KIND == EW_GELU) {
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = gelu_tanh(x[e]);
    } else if constexpr (KIND == EW_ADD) {
      f32x4 y = load4<DT>(b, i * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = x[e] + y[e];
    } else {
      f32x4 y = load4<DT>(b, (i * 4) % N);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        o[e] = x[e] + y[e];
        if constexpr (KIND == EW_BIAS_RELU) o[e] = relu_nan(o[e]);
      }
    }
    store4_streaming<DT>(out, i * 4, o);
  }
}

template <int DT, int KIND>
__global__ void __launch_bounds__(256) elementwise1(void* out, const void* a, const void* b, int64_t n, int N) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    float x = load_as_f32<DT>(a, i), o;
    if constexpr (KIND == EW_GELU) o = gelu_tanh(x);
    else if constexpr (KIND == EW_ADD) o = x + load_as_f32<DT>(b, i);
    else {
      o = x + load_as_f32<DT>(b, i % N);
      if constexpr (KIND == EW_BIAS_RELU) o = relu_nan(o);
    }
    store_from_f32<DT>(out, i, o);
  }
}

template <int SDT, int DDT>
__global__ void __launch_bounds__(256) cast_kernel(void* out, const void* x, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t n4 = n / 4;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride)
    store4<DDT>(out, i * 4, load4<SDT>(x, i * 4));
  for (int64_t i = n4 * 4 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
    store_from_f32<DDT>(out, i, load_as_f32<SDT>(x, i));
}

static inline unsigned ew_grid(int64_t work) {
  int64_t b = (work + 255) / 256;
  if (b < 1) b = 1;
  const int64_t cap = 256 * 16;  // 16 workgroups per CU, grid-stride beyond that
  return (unsigned)(b > cap ? cap : b);
}

// Smallest instantiated count of 4-element groups per lane that covers a row of N elements.
static inline int row_groups_rounded(int N) {
  const int need = (N + 255) / 256;
  const int have[] = {1, 2, 3, 4, 6, 8, 12, 16};
  for (int v : have)
    if (v >= need) return v;
  return 0;
}

template <int XDT, int ODT>
static int layer_norm_launch(void* out, const void* x, const float* gamma, const float* beta, int M, int N, float eps,
                             bool streaming, hipStream_t s) {
  const float inv_n = (float)(1.0 / (double)N);
  dim3 grid((M + 3) / 4), block(256);
  const bool vec = N % 256 == 0 && aligned16(out) && aligned16(x) && aligned16(gamma) && aligned16(beta);
  // Two rows per wave once every CU would otherwise hold 16 waves or more (and rows of at most
  // 1024 elements, to stay within 64 registers of row data).
  const bool two = (int64_t)M >= 16ll * 2 * num_cus() && N <= 1024;
  const dim3 grid2((((M + 1) / 2) + 3) / 4);
#define LH_LN_CASE(V)                                                                                                 \
  case V:                                                                                                             \
    if (two && V <= 4) {                                                                                              \
      if (streaming)                                                                                                  \
        LH_LAUNCH((layer_norm_vec<XDT, ODT, V, V <= 4 ? 2 : 1, false, true>), grid2, block, 0, s, out, x, gamma, beta, M, \
                  N, eps, inv_n);                                                                                     \
      else                                                                                                            \
        LH_LAUNCH((layer_norm_vec<XDT, ODT, V, V <= 4 ? 2 : 1>), grid2, block, 0, s, out, x, gamma, beta, M, N, eps,  \
                  inv_n);                                                                                             \
    } else if (streaming) {                                                                                           \
      LH_LAUNCH((layer_norm_vec<XDT, ODT, V, 1, false, true>), grid, block, 0, s, out, x, gamma, beta, M, N, eps,     \
                inv_n);                                                                                               \
    } else {                                                                                                          \
      LH_LAUNCH((layer_norm_vec<XDT, ODT, V, 1>), grid, block, 0, s, out, x, gamma, beta, M, N, eps, inv_n);          \
    }                                                                                                                 \
    return check_launch("layer_norm_vec");
  if (vec) {
    switch (N / 256) {
      LH_LN_CASE(1) LH_LN_CASE(2) LH_LN_CASE(3) LH_LN_CASE(4) LH_LN_CASE(6) LH_LN_CASE(8) LH_LN_CASE(12) LH_LN_CASE(16)
      default: break;
    }
  }
#undef LH_LN_CASE
  const bool vec4 = N % 4 == 0 && aligned16(out) && aligned16(x) && aligned16(gamma) && aligned16(beta);
  // Any other row of whole 4-element groups up to 4096 elements: the next register count up, guarded.
  if (vec4 && N >= 64 && N <= 4096) {
#define LH_LN_GUARD(V)                                                                                                \
  case V:                                                                                                             \
    LH_LAUNCH((layer_norm_vec<XDT, ODT, V, 1, true>), grid, block, 0, s, out, x, gamma, beta, M, N, eps,      \
                       inv_n);                                                                                        \
    return check_launch("layer_norm_vec (guarded)");
    switch (row_groups_rounded(N)) {
      LH_LN_GUARD(1) LH_LN_GUARD(2) LH_LN_GUARD(3) LH_LN_GUARD(4) LH_LN_GUARD(6) LH_LN_GUARD(8) LH_LN_GUARD(12)
      LH_LN_GUARD(16)
      default: break;
    }
#undef LH_LN_GUARD
  }
  if (N >= 1024 || (vec4 && N >= 512)) {
    if (vec4 && N <= 1024 * kBlockRegGroups)
      LH_LAUNCH((layer_norm_block_reg<XDT, ODT>), dim3(M), block, 0, s, out, x, gamma, beta, M, N, eps, inv_n);
    else if (vec4)
      LH_LAUNCH((layer_norm_block<XDT, ODT, true>), dim3(M), block, 0, s, out, x, gamma, beta, M, N, eps, inv_n);
    else
      LH_LAUNCH((layer_norm_block<XDT, ODT, false>), dim3(M), block, 0, s, out, x, gamma, beta, M, N, eps,
                         inv_n);
    return check_launch("layer_norm_block");
  }
  LH_LAUNCH((layer_norm_generic<XDT, ODT>), grid, block, 0, s, out, x, gamma, beta, M, N, eps, inv_n);
  return check_launch("layer_norm_generic");
}

template <int DT, int KIND>
static int ew_launch(void* out, const void* a, const void* b, int64_t n, int N, hipStream_t s) {
  const bool vec = n % 4 == 0 && (KIND < EW_BIAS || N % 4 == 0) && aligned16(out) && aligned16(a) &&
                   (b == nullptr || aligned16(b));
  if (vec) LH_LAUNCH((elementwise4<DT, KIND>), dim3(ew_grid(n / 4)), dim3(256), 0, s, out, a, b, n / 4, N);
  else LH_LAUNCH((elementwise1<DT, KIND>), dim3(ew_grid(n)), dim3(256), 0, s, out, a, b, n, N);
  return check_launch("elementwise");
}

template <int KIND>
static int ew_dispatch(void* out, const void* a, const void* b, int64_t n, int N, int dt, hipStream_t s) {
  switch (dt) {
    case LH_F32: return ew_launch<LH_F32, KIND>(out, a, b, n, N, s);
    case LH_BF16: return ew_launch<LH_BF16, KIND>(out, a, b, n, N, s);
    case LH_F16: return ew_launch<LH_F16, KIND>(out, a, b, n, N, s);
    default: return fail(LH_ERR_UNSUPPORTED, "elementwise: unsupported dtype %d", dt);
  }
}

}  // namespace lh

using namespace lh;

extern "C" {

int lh_hip_layer_norm(void* out, const void* x, const float* gamma, const float* beta, int64_t M, int64_t N, float eps,
                      int32_t x_dtype, int32_t out_dtype, void* stream) {
  return lh::layer_norm(out, x, gamma, beta, M, N, eps, x_dtype, out_dtype, /*streaming=*/true, stream);
}
}  // extern "C"

namespace lh {
int layer_norm(void* out, const void* x, const float* gamma, const float* beta, int64_t M, int64_t N, float eps,
               int32_t x_dtype, int32_t out_dtype, bool streaming, void* stream) {
  LH_REQUIRE(out && x && gamma && beta, "lh_hip_layer_norm: null pointer");
  LH_REQUIRE(M > 0 && N > 0 && M < (1ll << 31) && N < (1ll << 31), "lh_hip_layer_norm: bad shape %lld x %lld",
             (long long)M, (long long)N);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (x_dtype == LH_F32 && out_dtype == LH_F32)
    return layer_norm_launch<LH_F32, LH_F32>(out, x, gamma, beta, (int)M, (int)N, eps, streaming, s);
  if (x_dtype == LH_F32 && out_dtype == LH_BF16)
    return layer_norm_launch<LH_F32, LH_BF16>(out, x, gamma, beta, (int)M, (int)N, eps, streaming, s);
  if (x_dtype == LH_F32 && out_dtype == LH_F16)
    return layer_norm_launch<LH_F32, LH_F16>(out, x, gamma, beta, (int)M, (int)N, eps, streaming, s);
  if (x_dtype == LH_BF16 && out_dtype == LH_BF16)
    return layer_norm_launch<LH_BF16, LH_BF16>(out, x, gamma, beta, (int)M, (int)N, eps, streaming, s);
  if (x_dtype == LH_BF16 && out_dtype == LH_F32)
    return layer_norm_launch<LH_BF16, LH_F32>(out, x, gamma, beta, (int)M, (int)N, eps, streaming, s);
  return fail(LH_ERR_UNSUPPORTED, "lh_hip_layer_norm: unsupported dtypes x=%d out=%d", x_dtype, out_dtype);
}
}  // namespace lh

extern "C" {

int lh_hip_softmax(void* out, const void* x, int64_t M, int64_t N, int32_t dtype, void* stream) {
  LH_REQUIRE(out && x, "lh_hip_softmax: null pointer");
  LH_REQUIRE(M > 0 && N > 0 && M < (1ll << 31) && N < (1ll << 31), "lh_hip_softmax: bad shape");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)((M + 3) / 4)), block(256);
  if (N % 256 == 0 && N <= 4096 && aligned16(out) && aligned16(x)) {
#define LH_SM_CASE(DT, V)                                                                            \
  case V:                                                                                            \
    LH_LAUNCH((softmax_rows_vec<DT, V>), grid, block, 0, s, out, x, (int)M, (int)N);        \
    return check_launch("softmax_rows_vec");
#define LH_SM_DTYPE(DT)                                                                              \
  switch (N / 256) {                                                                                 \
    LH_SM_CASE(DT, 1) LH_SM_CASE(DT, 2) LH_SM_CASE(DT, 3) LH_SM_CASE(DT, 4) LH_SM_CASE(DT, 6)        \
    LH_SM_CASE(DT, 8) LH_SM_CASE(DT, 12) LH_SM_CASE(DT, 16)                                          \
    default: break;                                                                                  \
  }
    if (dtype == LH_F32) { LH_SM_DTYPE(LH_F32) }
    else if (dtype == LH_BF16) { LH_SM_DTYPE(LH_BF16) }
    else if (dtype == LH_F16) { LH_SM_DTYPE(LH_F16) }
#undef LH_SM_DTYPE
#undef LH_SM_CASE
  }
  const bool vec = N % 4 == 0 && aligned16(out) && aligned16(x);
  if (vec && N >= 64 && N <= 4096) {
#define LH_SM_GUARD(DT, V)                                                                           \
  case V:                                                                                            \
    LH_LAUNCH((softmax_rows_vec<DT, V, true>), grid, block, 0, s, out, x, (int)M, (int)N);  \
    return check_launch("softmax_rows_vec (guarded)");
#define LH_SM_GUARD_DTYPE(DT)                                                                        \
  switch (row_groups_rounded((int)N)) {                                                              \
    LH_SM_GUARD(DT, 1) LH_SM_GUARD(DT, 2) LH_SM_GUARD(DT, 3) LH_SM_GUARD(DT, 4) LH_SM_GUARD(DT, 6)   \
    LH_SM_GUARD(DT, 8) LH_SM_GUARD(DT, 12) LH_SM_GUARD(DT, 16)                                       \
    default: break;                                                                                  \
  }
    if (dtype == LH_F32) { LH_SM_GUARD_DTYPE(LH_F32) }
    else if (dtype == LH_BF16) { LH_SM_GUARD_DTYPE(LH_BF16) }
    else if (dtype == LH_F16) { LH_SM_GUARD_DTYPE(LH_F16) }
#undef LH_SM_GUARD_DTYPE
#undef LH_SM_GUARD
  }
  if (N >= 1024 || (vec && N >= 512)) {
    const dim3 rows((unsigned)M);
#define LH_SMB_CASE(DT)                                                                                    \
  case DT:                                                                                                 \
    if (vec && N <= 1024 * kBlockRegGroups)                                                                \
      LH_LAUNCH((softmax_block_reg<DT>), rows, block, 0, s, out, x, (int)M, (int)N);              \
    else if (vec) LH_LAUNCH((softmax_block<DT, true>), rows, block, 0, s, out, x, (int)M, (int)N); \
    else LH_LAUNCH((softmax_block<DT, false>), rows, block, 0, s, out, x, (int)M, (int)N);        \
    return check_launch("softmax_block");
    switch (dtype) {
      LH_SMB_CASE(LH_F32) LH_SMB_CASE(LH_BF16) LH_SMB_CASE(LH_F16)
      default: return fail(LH_ERR_UNSUPPORTED, "lh_hip_softmax: unsupported dtype %d", dtype);
    }
#undef LH_SMB_CASE
  }
  switch (dtype) {
    case LH_F32: LH_LAUNCH(softmax_rows<LH_F32>, grid, block, 0, s, out, x, (int)M, (int)N); break;
    case LH_BF16: LH_LAUNCH(softmax_rows<LH_BF16>, grid, block, 0, s, out, x, (int)M, (int)N); break;
    case LH_F16: LH_LAUNCH(softmax_rows<LH_F16>, grid, block, 0, s, out, x, (int)M, (int)N); break;
    default: return fail(LH_ERR_UNSUPPORTED, "lh_hip_softmax: unsupported dtype %d", dtype);
  }
  return check_launch("softmax_rows");
}

int lh_hip_gelu_tanh(void* out, const void* x, int64_t n, int32_t dtype, void* stream) {
  LH_REQUIRE(out && x && n > 0, "lh_hip_gelu_tanh: bad arguments");
  return ew_dispatch<EW_GELU>(out, x, nullptr, n, 1, dtype, reinterpret_cast<hipStream_t>(stream));
}

int lh_hip_bias_act(void* out, const void* x, const void* bias, int64_t M, int64_t N, int32_t relu, int32_t dtype,
                    void* stream) {
  LH_REQUIRE(out && x && bias && M > 0 && N > 0 && N < (1ll << 31), "lh_hip_bias_act: bad arguments");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (relu) return ew_dispatch<EW_BIAS_RELU>(out, x, bias, M * N, (int)N, dtype, s);
  return ew_dispatch<EW_BIAS>(out, x, bias, M * N, (int)N, dtype, s);
}

int lh_hip_add(void* out, const void* a, const void* b, int64_t n, int32_t dtype, void* stream) {
  LH_REQUIRE(out && a && b && n > 0, "lh_hip_add: bad arguments");
  return ew_dispatch<EW_ADD>(out, a, b, n, 1, dtype, reinterpret_cast<hipStream_t>(stream));
}

int lh_hip_cast(void* out, const void* x, int64_t n, int32_t src, int32_t dst, void* stream) {
  LH_REQUIRE(out && x && n > 0, "lh_hip_cast: bad arguments");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool al = aligned16(out) && aligned16(x);
  if (!al) return fail(LH_ERR_INVALID, "lh_hip_cast: buffers must be 16-byte aligned");
  dim3 grid(ew_grid(n / 4 + 1)), block(256);
#define LH_CAST(S, D)                                                         \
  if (src == S && dst == D) {                                                 \
    LH_LAUNCH((cast_kernel<S, D>), grid, block, 0, s, out, x, n);    \
    return check_launch("cast_kernel");                                       \
  }
  LH_CAST(LH_F32, LH_BF16) LH_CAST(LH_F32, LH_F16) LH_CAST(LH_BF16, LH_F32) LH_CAST(LH_F16, LH_F32)
  LH_CAST(LH_F32, LH_F32) LH_CAST(LH_BF16, LH_BF16) LH_CAST(LH_F16, LH_F16)
#undef LH_CAST
  return fail(LH_ERR_UNSUPPORTED, "lh_hip_cast: unsupported conversion %d -> %d", src, dst);
}

}  // extern "C"
