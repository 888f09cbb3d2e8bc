// GEMM for 16-bit inputs (bf16 / f16) with f32 accumulation on the gfx950 matrix cores and
// the fused bias / activation / conversion epilogue of the matmul payload
// (emit_mlp_layer, lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:110-156).
//
// Fast kernel (shapes that are multiples of the tile): workgroup tile BM x BN x 64, A and B
// panels double-buffered in LDS, v_mfma_f32_32x32x16 tiles, one barrier per k-step.  The MFMA
// is issued with the B panel as its first operand and the A panel as its second, so the
// accumulator of a lane holds 4 consecutive columns n of one row m and the epilogue stores
// 8 or 16 contiguous bytes per lane.  A row-major B ([K,N], n contiguous) is transposed in
// registers (v_perm_b32) on its way into LDS so both LDS panels are k-contiguous and every
// MFMA operand is a single 16-byte LDS read.
//
// Generic kernel: any shape, stride and transpose combination, 64 x 64 x 32 tiles with
// bounds-checked scalar loads.
#include "gemm_common.h"

namespace lh {

template <int DT>
struct Mfma16;
template <>
struct Mfma16<LH_BF16> {
  __device__ static __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  }
};
template <>
struct Mfma16<LH_F16> {
  __device__ static __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
  }
};

constexpr int kBK = 64;
constexpr int kLdsStride = kBK + 8;  // elements; 144-byte rows keep 16-byte reads of 16 rows conflict free

template <int BM, int BN>
constexpr size_t gemm16_lds_bytes() {
  return (size_t)2 * (BM + BN) * kLdsStride * sizeof(uint16_t);
}

template <int DT, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KC>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64) gemm16_fast(GemmArgs g) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_CH = BM * (kBK / 8) / NT;  // 16-byte chunks of the A panel per thread
  constexpr int B_CH = BN * (kBK / 8) / NT;  // same for a k-contiguous B panel
  constexpr int B_UN = (kBK / 8) * (BN / 4) / NT;  // 8k x 4n units per thread for a row-major B
  static_assert(A_CH >= 1 && B_CH >= 1 && B_UN >= 1, "tile too small for the thread count");

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* As = smem;
  uint16_t* Bs = smem + 2 * BM * kLdsStride;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WTM;
  const int wn0 = (wave % WAVES_N) * WTN;

  // Tile assignment: XCD-contiguous ids, then groups of 4 tile rows.
  const int tiles_m = g.M / BM, tiles_n = g.N / BN;
  int id = xcd_remap(blockIdx.x, gridDim.x);
  constexpr int GROUP_M = 4;
  const int group_size = GROUP_M * tiles_n;
  const int first_m = (id / group_size) * GROUP_M;
  const int gm = min(tiles_m - first_m, GROUP_M);
  const int tile_m = first_m + (id % group_size) % gm;
  const int tile_n = (id % group_size) / gm;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const uint16_t* A = reinterpret_cast<const uint16_t*>(g.a);
  const uint16_t* B = reinterpret_cast<const uint16_t*>(g.b);

  u32x4 ra[A_CH];
  u32x4 rbk[B_KC ? B_CH : 1];
  u32x2 rbn[B_KC ? 1 : B_UN][8];

  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      int c = tid + i * NT;
      int row = c >> 3, kc = c & 7;
      ra[i] = *reinterpret_cast<const u32x4*>(A + (int64_t)(m0 + row) * g.lda + k0 + kc * 8);
    }
    if constexpr (B_KC) {
#pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        int c = tid + i * NT;
        int row = c >> 3, kc = c & 7;
        rbk[i] = *reinterpret_cast<const u32x4*>(B + (int64_t)(n0 + row) * g.ldb + k0 + kc * 8);
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_UN; ++i) {
        int u = tid + i * NT;
        int ngrp = u % (BN / 4), kgrp = u / (BN / 4);
        const uint16_t* p = B + (int64_t)(k0 + kgrp * 8) * g.ldb + n0 + ngrp * 4;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) rbn[i][kk] = *reinterpret_cast<const u32x2*>(p + (int64_t)kk * g.ldb);
      }
    }
  };

  auto store_lds = [&](int buf) {
    uint16_t* as = As + buf * BM * kLdsStride;
    uint16_t* bs = Bs + buf * BN * kLdsStride;
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      int c = tid + i * NT;
      int row = c >> 3, kc = c & 7;
      *reinterpret_cast<u32x4*>(as + row * kLdsStride + kc * 8) = ra[i];
    }
    if constexpr (B_KC) {
#pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        int c = tid + i * NT;
        int row = c >> 3, kc = c & 7;
        *reinterpret_cast<u32x4*>(bs + row * kLdsStride + kc * 8) = rbk[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < B_UN; ++i) {
        int u = tid + i * NT;
        int ngrp = u % (BN / 4), kgrp = u / (BN / 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // Column j of the 8 x 4 register block becomes a k-contiguous row of 8 values.
          const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
          u32x4 w;
#pragma unroll
          for (int d = 0; d < 4; ++d)
            w[d] = __builtin_amdgcn_perm(rbn[i][2 * d + 1][j >> 1], rbn[i][2 * d][j >> 1], sel);
          *reinterpret_cast<u32x4*>(bs + (ngrp * 4 + j) * kLdsStride + kgrp * 8) = w;
        }
      }
    }
  };

  f32x16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int nk = g.K / kBK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;

  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global((kt + 1) * kBK);

    const uint16_t* as = As + buf * BM * kLdsStride + (wm0 + frag_row) * kLdsStride + frag_k;
    const uint16_t* bs = Bs + buf * BN * kLdsStride + (wn0 + frag_row) * kLdsStride + frag_k;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      u32x4 fb[TN], fa[TM];
#pragma unroll
      for (int i = 0; i < TN; ++i) fb[i] = *reinterpret_cast<const u32x4*>(bs + i * 32 * kLdsStride + ks * 16);
#pragma unroll
      for (int j = 0; j < TM; ++j) fa[j] = *reinterpret_cast<const u32x4*>(as + j * 32 * kLdsStride + ks * 16);
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) acc[i][j] = Mfma16<DT>::mma(fb[i], fa[j], acc[i][j]);
    }

    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }

  // acc[i][j][4q+e] = C[m0+wm0+32j+lane%32][n0+wn0+32i+8q+4(lane/32)+e]
  const int m_base = m0 + wm0 + (lane & 31);
  const int n_base = n0 + wn0 + 4 * (lane >> 5);
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        epilogue4<DT>(g, m_base + 32 * j, n_base + 32 * i + 8 * q, acc[i][j][4 * q], acc[i][j][4 * q + 1],
                      acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
}

// Any shape / stride / transpose; 64 x 64 x 32 tiles, 256 threads, bounds-checked.
template <int DT>
__global__ void __launch_bounds__(256) gemm16_generic(GemmArgs g) {
  constexpr int BM = 64, BN = 64, BK = 32, STR = BK + 8;
  __shared__ __attribute__((aligned(16))) uint16_t As[BM * STR];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[BN * STR];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const uint16_t* A = reinterpret_cast<const uint16_t*>(g.a);
  const uint16_t* B = reinterpret_cast<const uint16_t*>(g.b);
  const bool ta = (g.flags & LH_GEMM_TRANSPOSE_A) != 0, tb = (g.flags & LH_GEMM_TRANSPOSE_B) != 0;
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  for (int k0 = 0; k0 < g.K; k0 += BK) {
    for (int e = tid; e < BM * BK; e += 256) {
      // Thread order follows the contiguous dimension of the stored operand.
      int r, c;
      if (ta) { r = e % BM; c = e / BM; } else { r = e / BK; c = e % BK; }
      int m = m0 + r, k = k0 + c;
      uint16_t v = 0;
      if (m < g.M && k < g.K) v = ta ? A[(int64_t)k * g.lda + m] : A[(int64_t)m * g.lda + k];
      As[r * STR + c] = v;
    }
    for (int e = tid; e < BN * BK; e += 256) {
      int r, c;
      if (tb) { r = e / BK; c = e % BK; } else { r = e % BN; c = e / BN; }
      int n = n0 + r, k = k0 + c;
      uint16_t v = 0;
      if (n < g.N && k < g.K) v = tb ? B[(int64_t)n * g.ldb + k] : B[(int64_t)k * g.ldb + n];
      Bs[r * STR + c] = v;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      u32x4 fb = *reinterpret_cast<const u32x4*>(&Bs[(wn0 + (lane & 31)) * STR + ks * 16 + (lane >> 5) * 8]);
      u32x4 fa = *reinterpret_cast<const u32x4*>(&As[(wm0 + (lane & 31)) * STR + ks * 16 + (lane >> 5) * 8]);
      acc = Mfma16<DT>::mma(fb, fa, acc);
    }
    __syncthreads();
  }
  const int m = m0 + wm0 + (lane & 31);
  if (m >= g.M) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    int n = n0 + wn0 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
    if (n >= g.N) continue;
    epilogue1<DT>(g, m, n, acc[v]);
  }
}

template <int DT, int BM, int BN, int WAVES_M, int WAVES_N, bool B_KC>
static int launch_fast(const GemmArgs& g, hipStream_t s) {
  auto kern = gemm16_fast<DT, BM, BN, WAVES_M, WAVES_N, B_KC>;
  constexpr size_t lds = gemm16_lds_bytes<BM, BN>();
  static bool configured = false;
  if (!configured) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  dim3 grid((g.M / BM) * (g.N / BN));
  hipLaunchKernelGGL(kern, grid, dim3(WAVES_M * WAVES_N * 64), lds, s, g);
  return check_launch("gemm16_fast");
}

template <int DT>
static int gemm16_dispatch(const GemmArgs& g, hipStream_t s) {
  const bool ta = g.flags & LH_GEMM_TRANSPOSE_A, tb = g.flags & LH_GEMM_TRANSPOSE_B;
  const bool vec_ok = !ta && g.K % kBK == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 && g.ldc % 4 == 0 &&
                      aligned16(g.a) && aligned16(g.b) && aligned16(g.out) &&
                      (!(g.flags & LH_GEMM_HAS_BIAS) || aligned16(g.bias));
  if (vec_ok) {
    const int cus = 256;
    const bool big = g.M % 256 == 0 && g.N % 256 == 0 && (int64_t)(g.M / 256) * (g.N / 256) >= cus;
    if (big) {
      return tb ? launch_fast<DT, 256, 256, 2, 4, true>(g, s) : launch_fast<DT, 256, 256, 2, 4, false>(g, s);
    }
    if (g.M % 128 == 0 && g.N % 128 == 0) {
      return tb ? launch_fast<DT, 128, 128, 2, 2, true>(g, s) : launch_fast<DT, 128, 128, 2, 2, false>(g, s);
    }
  }
  dim3 grid((g.N + 63) / 64, (g.M + 63) / 64);
  hipLaunchKernelGGL(gemm16_generic<DT>, grid, dim3(256), 0, s, g);
  return check_launch("gemm16_generic");
}

int gemm16(const GemmArgs& g, int ab_dtype, hipStream_t s) {
  if (ab_dtype == LH_BF16) return gemm16_dispatch<LH_BF16>(g, s);
  return gemm16_dispatch<LH_F16>(g, s);
}

}  // namespace lh
