// fp8 (OCP e4m3fn) GEMM with per-tensor scales on the gfx950 matrix cores:
// out = out_dtype((Aq . Bq)_f32 * (scale_a * scale_b)).  The benchmark's quantised
// configuration; the reference has no fp8 payload.
//
// Large kernel: workgroup tile 256 x 256 x 128, 8 waves, v_mfma_f32_32x32x64_f8f6f4, A and B
// panels double-buffered in LDS with k contiguous; the row-major B ([K,N]) is transposed in
// registers with byte permutes on its way into LDS.  The MFMA pairs equal (lane half,
// register, byte) positions of its two operands, so any k order inside a 64-wide k-step is
// valid as long as both panels use the same one; both are read as 32 contiguous bytes.
//
// Skinny kernel (M <= 16, the decode shape): HBM-bound streaming of B; v_mfma_f32_16x16x128,
// split over K across workgroups with f32 partials reduced by a second small kernel.
#include "gemm_common.h"

namespace lh {

__device__ __forceinline__ f32x16 mfma_f8_32(i32x8 a, i32x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma_f8_16(i32x8 a, i32x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// Transpose a 4 x 4 byte block held as 4 dwords (row r = dword r) in place.
__device__ __forceinline__ void transpose4x4_bytes(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
  uint32_t t01l = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
  uint32_t t01h = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
  uint32_t t23l = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
  uint32_t t23h = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
  r0 = __builtin_amdgcn_perm(t23l, t01l, 0x05040100u);
  r1 = __builtin_amdgcn_perm(t23l, t01l, 0x07060302u);
  r2 = __builtin_amdgcn_perm(t23h, t01h, 0x05040100u);
  r3 = __builtin_amdgcn_perm(t23h, t01h, 0x07060302u);
}

constexpr int kBK8 = 128;
constexpr int kStride8 = kBK8 + 16;  // bytes per LDS row

template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64) gemm8_fast(GemmArgs g) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N, TM = WTM / 32, TN = WTN / 32;
  constexpr int A_CH = BM * (kBK8 / 16) / NT;          // 16-byte chunks per thread
  constexpr int B_UN = (kBK8 / 16) * (BN / 4) / NT;    // 16k x 4n units per thread
  static_assert(A_CH >= 1 && B_UN >= 1, "tile too small");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem8[];
  uint8_t* As = smem8;
  uint8_t* Bs = smem8 + 2 * BM * kStride8;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
  const int tiles_m = g.M / BM, tiles_n = g.N / BN;
  const int id = xcd_remap(blockIdx.x, gridDim.x);
  constexpr int GROUP_M = 4;
  const int group_size = GROUP_M * tiles_n;
  const int first_m = (id / group_size) * GROUP_M;
  const int gm = min(tiles_m - first_m, GROUP_M);
  const int m0 = (first_m + (id % group_size) % gm) * BM;
  const int n0 = ((id % group_size) / gm) * BN;
  const uint8_t* A = reinterpret_cast<const uint8_t*>(g.a);
  const uint8_t* B = reinterpret_cast<const uint8_t*>(g.b);

  u32x4 ra[A_CH];
  uint32_t rb[B_UN][16];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      int c = tid + i * NT, row = c >> 3, kc = c & 7;
      ra[i] = *reinterpret_cast<const u32x4*>(A + (int64_t)(m0 + row) * g.lda + k0 + kc * 16);
    }
#pragma unroll
    for (int i = 0; i < B_UN; ++i) {
      int u = tid + i * NT, ngrp = u % (BN / 4), kgrp = u / (BN / 4);
      const uint8_t* p = B + (int64_t)(k0 + kgrp * 16) * g.ldb + n0 + ngrp * 4;
#pragma unroll
      for (int kk = 0; kk < 16; ++kk) rb[i][kk] = *reinterpret_cast<const uint32_t*>(p + (int64_t)kk * g.ldb);
    }
  };
  auto store_lds = [&](int buf) {
    uint8_t* as = As + buf * BM * kStride8;
    uint8_t* bs = Bs + buf * BN * kStride8;
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      int c = tid + i * NT, row = c >> 3, kc = c & 7;
      *reinterpret_cast<u32x4*>(as + row * kStride8 + kc * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_UN; ++i) {
      int u = tid + i * NT, ngrp = u % (BN / 4), kgrp = u / (BN / 4);
#pragma unroll
      for (int q = 0; q < 4; ++q) transpose4x4_bytes(rb[i][4 * q], rb[i][4 * q + 1], rb[i][4 * q + 2], rb[i][4 * q + 3]);
      // rb[i][4q + j] now holds column j, k rows 4q..4q+3.
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x4 w = {rb[i][j], rb[i][4 + j], rb[i][8 + j], rb[i][12 + j]};
        *reinterpret_cast<u32x4*>(bs + (ngrp * 4 + j) * kStride8 + kgrp * 16) = w;
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

  const int nk = g.K / kBK8;
  load_global(0);
  store_lds(0);
  __syncthreads();
  const int r32 = lane & 31, h = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global((kt + 1) * kBK8);
    const uint8_t* as = As + buf * BM * kStride8 + (wm0 + r32) * kStride8 + 32 * h;
    const uint8_t* bs = Bs + buf * BN * kStride8 + (wn0 + r32) * kStride8 + 32 * h;
#pragma unroll
    for (int ks = 0; ks < kBK8 / 64; ++ks) {
      i32x8 fb[TN], fa[TM];
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        i32x4 lo = *reinterpret_cast<const i32x4*>(bs + i * 32 * kStride8 + ks * 64);
        i32x4 hi = *reinterpret_cast<const i32x4*>(bs + i * 32 * kStride8 + ks * 64 + 16);
        fb[i] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        i32x4 lo = *reinterpret_cast<const i32x4*>(as + j * 32 * kStride8 + ks * 64);
        i32x4 hi = *reinterpret_cast<const i32x4*>(as + j * 32 * kStride8 + ks * 64 + 16);
        fa[j] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) acc[i][j] = mfma_f8_32(fb[i], fa[j], acc[i][j]);
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
        epilogue4<LH_BF16>(g, m_base + 32 * j, n_base + 32 * i + 8 * q, acc[i][j][4 * q], acc[i][j][4 * q + 1],
                           acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
}

// Any shape: 32 x 32 x 64 tile per wave, one wave per workgroup tile of 32 x 32,
// bounds-checked byte loads (zero padding: code 0 is +0).
__global__ void __launch_bounds__(64) gemm8_generic(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) uint8_t As[32 * 80];
  __shared__ __attribute__((aligned(16))) uint8_t Bs[32 * 80];
  const int lane = threadIdx.x, r32 = lane & 31, h = lane >> 5;
  const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
  const uint8_t* A = reinterpret_cast<const uint8_t*>(g.a);
  const uint8_t* B = reinterpret_cast<const uint8_t*>(g.b);
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  for (int k0 = 0; k0 < g.K; k0 += 64) {
    for (int e = lane; e < 32 * 64; e += 64) {
      int r = e / 64, c = e % 64;
      int m = m0 + r, k = k0 + c;
      As[r * 80 + c] = (m < g.M && k < g.K) ? A[(int64_t)m * g.lda + k] : (uint8_t)0;
    }
    for (int e = lane; e < 32 * 64; e += 64) {
      int r = e % 32, c = e / 32;  // r = n (contiguous in memory), c = k
      int n = n0 + r, k = k0 + c;
      Bs[r * 80 + c] = (n < g.N && k < g.K) ? B[(int64_t)k * g.ldb + n] : (uint8_t)0;
    }
    __syncthreads();
    i32x4 alo = *reinterpret_cast<const i32x4*>(&As[r32 * 80 + 32 * h]);
    i32x4 ahi = *reinterpret_cast<const i32x4*>(&As[r32 * 80 + 32 * h + 16]);
    i32x4 blo = *reinterpret_cast<const i32x4*>(&Bs[r32 * 80 + 32 * h]);
    i32x4 bhi = *reinterpret_cast<const i32x4*>(&Bs[r32 * 80 + 32 * h + 16]);
    i32x8 fa = {alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
    i32x8 fb = {blo[0], blo[1], blo[2], blo[3], bhi[0], bhi[1], bhi[2], bhi[3]};
    acc = mfma_f8_32(fb, fa, acc);
    __syncthreads();
  }
  const int m = m0 + r32;
  if (m >= g.M) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    int n = n0 + 8 * (v >> 2) + 4 * h + (v & 3);
    if (n >= g.N) continue;
    epilogue1<LH_BF16>(g, m, n, acc[v]);
  }
}

// ---- skinny (decode) path ---------------------------------------------------------------
// Workgroup: 256 threads, tile 16 (padded M) x 128 n x 128 k per step, over a K chunk.
// partial[split][16][N] f32.  Wave w owns columns 32 w .. 32 w + 31 (two 16-wide MFMA tiles).
constexpr int kSkinnyBN = 128;

__global__ void __launch_bounds__(256) gemm8_skinny(GemmArgs g, float* partial, int k_chunk) {
  __shared__ __attribute__((aligned(16))) uint8_t As[2][16 * kStride8];
  __shared__ __attribute__((aligned(16))) uint8_t Bs[2][kSkinnyBN * kStride8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * kSkinnyBN;
  const int kbeg = blockIdx.y * k_chunk;
  const uint8_t* A = reinterpret_cast<const uint8_t*>(g.a);
  const uint8_t* B = reinterpret_cast<const uint8_t*>(g.b);

  // Loader: B tile 128 k x 128 n = 256 units of 16k x 4n (one per thread); A tile 16 x 128 =
  // 128 chunks of 16 bytes (threads 0..127; rows >= M read as zero).
  const int ngrp = tid % (kSkinnyBN / 4), kgrp = tid / (kSkinnyBN / 4);
  const int a_row = tid >> 3, a_kc = tid & 7;
  uint32_t rb[16];
  u32x4 ra = {0, 0, 0, 0};
  auto load_global = [&](int k0) {
    const uint8_t* p = B + (int64_t)(k0 + kgrp * 16) * g.ldb + n0 + ngrp * 4;
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) rb[kk] = *reinterpret_cast<const uint32_t*>(p + (int64_t)kk * g.ldb);
    if (tid < 128 && a_row < g.M) ra = *reinterpret_cast<const u32x4*>(A + (int64_t)a_row * g.lda + k0 + a_kc * 16);
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 4; ++q) transpose4x4_bytes(rb[4 * q], rb[4 * q + 1], rb[4 * q + 2], rb[4 * q + 3]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 w = {rb[j], rb[4 + j], rb[8 + j], rb[12 + j]};
      *reinterpret_cast<u32x4*>(&Bs[buf][(ngrp * 4 + j) * kStride8 + kgrp * 16]) = w;
    }
    if (tid < 128) *reinterpret_cast<u32x4*>(&As[buf][a_row * kStride8 + a_kc * 16]) = ra;
  };

  f32x4 acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[i][v] = 0.0f;
  const int nk = k_chunk / kBK8;
  load_global(kbeg);
  store_lds(0);
  __syncthreads();
  const int r16 = lane & 15, qd = lane >> 4;  // row/col within the MFMA tile, k quarter
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global(kbeg + (kt + 1) * kBK8);
    i32x4 alo = *reinterpret_cast<const i32x4*>(&As[buf][r16 * kStride8 + 32 * qd]);
    i32x4 ahi = *reinterpret_cast<const i32x4*>(&As[buf][r16 * kStride8 + 32 * qd + 16]);
    i32x8 fa = {alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint8_t* bp = &Bs[buf][(wave * 32 + 16 * i + r16) * kStride8 + 32 * qd];
      i32x4 blo = *reinterpret_cast<const i32x4*>(bp);
      i32x4 bhi = *reinterpret_cast<const i32x4*>(bp + 16);
      i32x8 fb = {blo[0], blo[1], blo[2], blo[3], bhi[0], bhi[1], bhi[2], bhi[3]};
      // First operand = B panel: the accumulator of lane (m = r16, quarter qd) holds
      // columns n = 4 qd + v of row m.
      acc[i] = mfma_f8_16(fb, fa, acc[i]);
    }
    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }
  float* dst = partial + ((int64_t)blockIdx.y * 16 + r16) * g.N + n0 + wave * 32 + 4 * qd;
#pragma unroll
  for (int i = 0; i < 2; ++i) *reinterpret_cast<f32x4*>(dst + 16 * i) = acc[i];
}

__global__ void __launch_bounds__(256) gemm8_skinny_reduce(GemmArgs g, const float* partial, int splits) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)g.M * g.N) return;
  const int m = (int)(idx / g.N), n = (int)(idx % g.N);
  float s = 0.0f;
  for (int sp = 0; sp < splits; ++sp) s += partial[((int64_t)sp * 16 + m) * g.N + n];
  epilogue1<LH_BF16>(g, m, n, s);
}

static float* g_partial = nullptr;
static size_t g_partial_bytes = 0;

template <int BM, int BN, int WAVES_M, int WAVES_N>
static int launch_fast8(const GemmArgs& g, hipStream_t s) {
  auto kern = gemm8_fast<BM, BN, WAVES_M, WAVES_N>;
  constexpr size_t lds = (size_t)2 * (BM + BN) * kStride8;
  static bool configured = false;
  if (!configured) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3((g.M / BM) * (g.N / BN)), dim3(WAVES_M * WAVES_N * 64), lds, s, g);
  return check_launch("gemm8_fast");
}

int gemm8(const GemmArgs& g, hipStream_t s) {
  const bool vec_ok = g.K % kBK8 == 0 && g.lda % 16 == 0 && g.ldb % 4 == 0 && g.ldc % 4 == 0 && aligned16(g.a) &&
                      aligned16(g.b) && aligned16(g.out);
  if (vec_ok && g.M <= 16 && g.N % kSkinnyBN == 0) {
    // Split K so that about 512 workgroups stream B.
    int splits = 1;
    const int nblk = g.N / kSkinnyBN;
    while (nblk * splits < 512 && (g.K / kBK8) % (splits * 2) == 0 && splits < 64) splits *= 2;
    const size_t need = (size_t)splits * 16 * g.N * sizeof(float);
    if (need > g_partial_bytes) {
      if (g_partial) LH_HIP_CHECK(hipFree(g_partial));
      g_partial = nullptr;
      g_partial_bytes = 0;
      LH_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&g_partial), need));
      g_partial_bytes = need;
    }
    hipLaunchKernelGGL(gemm8_skinny, dim3(nblk, splits), dim3(256), 0, s, g, g_partial, g.K / splits);
    int rc = check_launch("gemm8_skinny");
    if (rc) return rc;
    const int64_t total = (int64_t)g.M * g.N;
    hipLaunchKernelGGL(gemm8_skinny_reduce, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, g, g_partial,
                       splits);
    return check_launch("gemm8_skinny_reduce");
  }
  if (vec_ok && g.M % 256 == 0 && g.N % 256 == 0 && (int64_t)(g.M / 256) * (g.N / 256) >= 128)
    return launch_fast8<256, 256, 2, 4>(g, s);
  if (vec_ok && g.M % 128 == 0 && g.N % 128 == 0) return launch_fast8<128, 128, 2, 2>(g, s);
  dim3 grid((g.N + 31) / 32, (g.M + 31) / 32);
  hipLaunchKernelGGL(gemm8_generic, grid, dim3(64), 0, s, g);
  return check_launch("gemm8_generic");
}

}  // namespace lh
