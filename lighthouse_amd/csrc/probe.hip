// Benchmark-side helper, built into a library of its own (liblighthouse_probe.so) that only
// bench.py loads; it is not part of liblighthouse_hip.so or of its C ABI.
// Measurement aid: the rate of a register-only MFMA loop (no LDS, no global traffic in the timed
// part) on every SIMD of the device, with all-zero or random operands.  The matrix cores' clock
// under load depends on how much the operand bits toggle, so this is the ceiling a GEMM of the same
// element type can reach on the same kind of data, to be read next to the published peak.
#include <vector>

#include "common.h"

namespace lh {

// 8 waves per workgroup, one workgroup per CU; each wave keeps the accumulators of a 128 x 64
// sub-tile and 8 + 4 operand fragments (two sets, alternating) in registers and issues the
// instructions the GEMM kernels use: v_mfma_f32_16x16x32 (16-bit), v_mfma_scale_f32_16x16x128_f8f6f4
// (fp8), v_mfma_f32_32x32x2 (f32).  WIDE: the 32x32x16 / 32x32x64 forms of the same products instead,
// which reach the same rate on zeros and a lower one on random operands.
template <int DT, bool WIDE>
__global__ void __launch_bounds__(512) mfma_rate_kernel(float* out, const u32x4* frag, int iters) {
  u32x4 fa[8], fb[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    fa[i] = frag[i * 512 + threadIdx.x];
    fb[i] = frag[(8 + i) * 512 + threadIdx.x];
  }
  if constexpr (DT == LH_F32 || WIDE) {
    f32x16 c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) c[i][e] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x4 b0 = fb[i + 2 * (it & 1)], a0 = fa[j];
          if constexpr (DT == LH_BF16) {
            c[4 * i + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b0),
                                                                   __builtin_bit_cast(bf16x8, a0), c[4 * i + j], 0, 0, 0);
          } else if constexpr (DT == LH_F8E4M3) {
            const u32x4 a1 = fa[(j + 1) & 3], b1 = fb[(i + 1 + 2 * (it & 1)) & 3];
            i32x8 a = {(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
            i32x8 b = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
            c[4 * i + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c[4 * i + j], 0, 0, 0, 0, 0, 0);
          } else {
            c[4 * i + j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, b0[it & 3]),
                                                                __builtin_bit_cast(float, a0[it & 3]), c[4 * i + j], 0,
                                                                0, 0);
          }
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) s += c[i][e];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  } else {
    // 4 column fragments x 8 row fragments of 16: the same 128 x 64 sub-tile, twice the k per instruction
    f32x4 c[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) c[i][j][e] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const u32x4 b0 = fb[i + 4 * (it & 1)], a0 = fa[j];
          if constexpr (DT == LH_BF16) {
            c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b0),
                                                              __builtin_bit_cast(bf16x8, a0), c[i][j], 0, 0, 0);
          } else {
            const u32x4 a1 = fa[(j + 1) & 7], b1 = fb[(i + 1 + 4 * (it & 1)) & 7];
            i32x8 a = {(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
            i32x8 b = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
            c[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b, a, c[i][j], 0, 0, 0, 0, 0, 0);
          }
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) s += c[i][j][e];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  }
}

}  // namespace lh

using namespace lh;

// Self-contained error handling: this file links against nothing of the main library.
#define PROBE_CHECK(expr)                  \
  do {                                     \
    if ((expr) != hipSuccess) return -3;   \
  } while (0)

// Returns 0, -1 (bad arguments) or -3 (HIP runtime failure).
// random_operands: 0 = zeros, 1 = random; bit 1 set (2, 3) = the 32x32 instruction forms of the 16-bit / fp8 products.
extern "C" int lh_probe_mfma_rate(int32_t dtype, int32_t random_operands, int64_t iters, double* tflops) {
  const bool wide = (random_operands & 2) != 0 || dtype == LH_F32;
  random_operands &= 1;
  if (!(tflops && iters > 0 && iters < (1ll << 30))) return -1;
  if (!(dtype == LH_BF16 || dtype == LH_F8E4M3 || dtype == LH_F32)) return -1;
  int dev = 0, cus = 0;
  PROBE_CHECK(hipGetDevice(&dev));
  PROBE_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  const size_t nfrag = 16 * 512;
  std::vector<uint32_t> host(nfrag * 4, 0u);
  if (random_operands) {
    // Values of magnitude close to 1 with random signs and mantissas (what N(0,1) inputs look like
    // to the multiplier arrays), from a fixed linear congruential sequence.
    uint64_t state = 0x9E3779B97F4A7C15ull;
    auto next = [&]() {
      state = state * 6364136223846793005ull + 1442695040888963407ull;
      return (uint32_t)(state >> 33);
    };
    for (auto& w : host) {
      if (dtype == LH_BF16) {
        const uint32_t lo = (0x3f00u + (next() & 0x1ffu)) | ((next() & 1u) << 15);
        const uint32_t hi = (0x3f00u + (next() & 0x1ffu)) | ((next() & 1u) << 15);
        w = lo | (hi << 16);
      } else if (dtype == LH_F8E4M3) {
        w = 0;
        for (int b = 0; b < 4; ++b) w |= ((((next() & 1u) << 7) | ((4u + next() % 6u) << 3) | (next() & 7u)) & 0xffu) << (8 * b);
      } else {
        const float v = (float)(next() & 0xffffffu) / (float)0x800000 - 1.0f;
        w = __builtin_bit_cast(uint32_t, v);
      }
    }
  }
  u32x4* frag = nullptr;
  float* out = nullptr;
  PROBE_CHECK(hipMalloc(reinterpret_cast<void**>(&frag), nfrag * 16));
  PROBE_CHECK(hipMalloc(reinterpret_cast<void**>(&out), (size_t)cus * 512 * sizeof(float)));
  PROBE_CHECK(hipMemcpy(frag, host.data(), nfrag * 16, hipMemcpyHostToDevice));
  hipEvent_t e0, e1;
  PROBE_CHECK(hipEventCreate(&e0));
  PROBE_CHECK(hipEventCreate(&e1));
  auto launch = [&]() {
    if (dtype == LH_BF16 && wide) hipLaunchKernelGGL((mfma_rate_kernel<LH_BF16, true>), dim3(cus), dim3(512), 0, nullptr, out, frag, (int)iters);
    else if (dtype == LH_BF16) hipLaunchKernelGGL((mfma_rate_kernel<LH_BF16, false>), dim3(cus), dim3(512), 0, nullptr, out, frag, (int)iters);
    else if (dtype == LH_F8E4M3 && wide) hipLaunchKernelGGL((mfma_rate_kernel<LH_F8E4M3, true>), dim3(cus), dim3(512), 0, nullptr, out, frag, (int)iters);
    else if (dtype == LH_F8E4M3) hipLaunchKernelGGL((mfma_rate_kernel<LH_F8E4M3, false>), dim3(cus), dim3(512), 0, nullptr, out, frag, (int)iters);
    else hipLaunchKernelGGL((mfma_rate_kernel<LH_F32, true>), dim3(cus), dim3(512), 0, nullptr, out, frag, (int)iters);
  };
  launch();  // warm-up
  PROBE_CHECK(hipEventRecord(e0, nullptr));
  launch();
  PROBE_CHECK(hipEventRecord(e1, nullptr));
  PROBE_CHECK(hipEventSynchronize(e1));
  const int rc = hipGetLastError() == hipSuccess ? 0 : -3;
  float ms = 0.0f;
  PROBE_CHECK(hipEventElapsedTime(&ms, e0, e1));
  PROBE_CHECK(hipEventDestroy(e0));
  PROBE_CHECK(hipEventDestroy(e1));
  PROBE_CHECK(hipFree(frag));
  PROBE_CHECK(hipFree(out));
  if (rc) return rc;
  // flop per wave and iteration: 8 (wide) or 32 instructions on the 128 x 64 sub-tile
  const double flop_per_iter = wide ? 8.0 * (dtype == LH_BF16 ? 32768.0 : dtype == LH_F8E4M3 ? 131072.0 : 4096.0)
                                    : 32.0 * (dtype == LH_BF16 ? 16384.0 : 65536.0);
  *tflops = (double)iters * flop_per_iter * 8.0 * cus / ((double)ms * 1e-3) / 1e12;
  return 0;
}
