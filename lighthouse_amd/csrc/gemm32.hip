// f32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32, full f32 products and
// accumulation) with the fused epilogue of the matmul payload
// (emit_mlp_layer, lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:110-156; the f32
// generic-form fixture test/opt/pipeline-check.mlir:27-46).
//
// Fast kernel: workgroup tile BM x BN x 32, 4 waves (2 x 2), A panel [m][k] and B panel
// [k][n] double-buffered in LDS in their global orientation.  The MFMA takes one f32 per
// lane and operand; a lane reads 4 consecutive k of its A row with one 16-byte LDS read and
// issues 4 MFMAs, and reads the 4 matching B rows with 4-byte reads that are contiguous
// across the lanes of a half wave.  As in the 16-bit kernel the B panel is the first MFMA
// operand, so a lane's accumulator holds 4 consecutive columns of one row.
#include "gemm_common.h"

namespace lh {

constexpr int kBK32 = 32;
constexpr int kAStride32 = kBK32 + 4;  // floats; 144-byte rows: 16-byte reads of 16 rows are conflict free

template <int BM, int BN>
__global__ void __launch_bounds__(256) gemm32_fast(GemmArgs g) {
  constexpr int NT = 256;
  constexpr int BSTR = BN + 8;  // rows 4 apart land 32 banks apart
  constexpr int WTM = BM / 2, WTN = BN / 2, TM = WTM / 32, TN = WTN / 32;
  constexpr int A_CH = BM * (kBK32 / 4) / NT;
  constexpr int B_CH = kBK32 * (BN / 4) / NT;
  extern __shared__ __attribute__((aligned(16))) float smem32[];
  float(*As)[BM * kAStride32] = reinterpret_cast<float(*)[BM * kAStride32]>(smem32);
  float(*Bs)[kBK32 * BSTR] = reinterpret_cast<float(*)[kBK32 * BSTR]>(smem32 + 2 * BM * kAStride32);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * WTM, wn0 = (wave & 1) * WTN;
  const int tiles_n = g.N / BN;
  const int id = xcd_remap(blockIdx.x, gridDim.x);
  const int m0 = (id / tiles_n) * BM, n0 = (id % tiles_n) * BN;
  const float* A = reinterpret_cast<const float*>(g.a);
  const float* B = reinterpret_cast<const float*>(g.b);

  f32x4 ra[A_CH], rb[B_CH];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      int c = tid + i * NT, row = c >> 3, kc = c & 7;
      ra[i] = *reinterpret_cast<const f32x4*>(A + (int64_t)(m0 + row) * g.lda + k0 + kc * 4);
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      int c = tid + i * NT, row = c / (BN / 4), nc = c % (BN / 4);
      rb[i] = *reinterpret_cast<const f32x4*>(B + (int64_t)(k0 + row) * g.ldb + n0 + nc * 4);
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      int c = tid + i * NT, row = c >> 3, kc = c & 7;
      *reinterpret_cast<f32x4*>(&As[buf][row * kAStride32 + kc * 4]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      int c = tid + i * NT, row = c / (BN / 4), nc = c % (BN / 4);
      *reinterpret_cast<f32x4*>(&Bs[buf][row * BSTR + nc * 4]) = rb[i];
    }
  };

  f32x16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int nk = g.K / kBK32;
  load_global(0);
  store_lds(0);
  __syncthreads();
  const int r32 = lane & 31, h = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global((kt + 1) * kBK32);
#pragma unroll
    for (int kk = 0; kk < kBK32 / 8; ++kk) {
      // The lane's k indices for the next 4 MFMAs are kk*8 + 4h + t, t = 0..3.
      f32x4 fa[TM];
      float fb[TN][4];
#pragma unroll
      for (int j = 0; j < TM; ++j)
        fa[j] = *reinterpret_cast<const f32x4*>(&As[buf][(wm0 + 32 * j + r32) * kAStride32 + kk * 8 + 4 * h]);
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int t = 0; t < 4; ++t) fb[i][t] = Bs[buf][(kk * 8 + 4 * h + t) * BSTR + wn0 + 32 * i + r32];
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
          for (int j = 0; j < TM; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[i][t], fa[j][t], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }

  const int m_base = m0 + wm0 + r32;
  const int n_base = n0 + wn0 + 4 * h;
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        epilogue4<LH_F32>(g, m_base + 32 * j, n_base + 32 * i + 8 * q, acc[i][j][4 * q], acc[i][j][4 * q + 1],
                          acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
}

// Any shape / stride / transpose; 64 x 64 x 16 tiles, bounds-checked scalar loads.
__global__ void __launch_bounds__(256) gemm32_generic(GemmArgs g) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float As[BM * (BK + 1)];
  __shared__ float Bs[BK * (BN + 1)];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const float* A = reinterpret_cast<const float*>(g.a);
  const float* B = reinterpret_cast<const float*>(g.b);
  const bool ta = (g.flags & LH_GEMM_TRANSPOSE_A) != 0, tb = (g.flags & LH_GEMM_TRANSPOSE_B) != 0;
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  for (int k0 = 0; k0 < g.K; k0 += BK) {
    for (int e = tid; e < BM * BK; e += 256) {
      int r, c;
      if (ta) { r = e % BM; c = e / BM; } else { r = e / BK; c = e % BK; }
      int m = m0 + r, k = k0 + c;
      float v = 0.0f;
      if (m < g.M && k < g.K) v = ta ? A[(int64_t)k * g.lda + m] : A[(int64_t)m * g.lda + k];
      As[r * (BK + 1) + c] = v;
    }
    for (int e = tid; e < BN * BK; e += 256) {
      int r, c;  // r = n, c = k
      if (tb) { r = e / BK; c = e % BK; } else { r = e % BN; c = e / BN; }
      int n = n0 + r, k = k0 + c;
      float v = 0.0f;
      if (n < g.N && k < g.K) v = tb ? B[(int64_t)n * g.ldb + k] : B[(int64_t)k * g.ldb + n];
      Bs[c * (BN + 1) + r] = v;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
      int k = ks * 2 + (lane >> 5);
      float fb = Bs[k * (BN + 1) + wn0 + (lane & 31)];
      float fa = As[(wm0 + (lane & 31)) * (BK + 1) + k];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb, fa, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  const int m = m0 + wm0 + (lane & 31);
  if (m >= g.M) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    int n = n0 + wn0 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
    if (n >= g.N) continue;
    epilogue1<LH_F32>(g, m, n, acc[v]);
  }
}

template <int BM, int BN>
static int launch_fast32(const GemmArgs& g, hipStream_t s) {
  auto kern = gemm32_fast<BM, BN>;
  constexpr size_t lds = (size_t)2 * (BM * kAStride32 + kBK32 * (BN + 8)) * sizeof(float);
  static bool configured = false;
  if (!configured) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3((g.M / BM) * (g.N / BN)), dim3(256), lds, s, g);
  return check_launch("gemm32_fast");
}

int gemm32(const GemmArgs& g, hipStream_t s) {
  const bool trans = g.flags & (LH_GEMM_TRANSPOSE_A | LH_GEMM_TRANSPOSE_B);
  const bool vec_ok = !trans && g.K % kBK32 == 0 && g.lda % 4 == 0 && g.ldb % 4 == 0 && g.ldc % 4 == 0 &&
                      aligned16(g.a) && aligned16(g.b) && aligned16(g.out) &&
                      (!(g.flags & LH_GEMM_HAS_BIAS) || aligned16(g.bias));
  if (vec_ok && g.M % 128 == 0 && g.N % 128 == 0 && (int64_t)(g.M / 128) * (g.N / 128) >= 512) {
    return launch_fast32<128, 128>(g, s);
  }
  if (vec_ok && g.M % 64 == 0 && g.N % 64 == 0) {
    return launch_fast32<64, 64>(g, s);
  }
  dim3 grid((g.N + 63) / 64, (g.M + 63) / 64);
  hipLaunchKernelGGL(gemm32_generic, grid, dim3(256), 0, s, g);
  return check_launch("gemm32_generic");
}

}  // namespace lh
