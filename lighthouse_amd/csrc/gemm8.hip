// fp8 (OCP e4m3fn) GEMM with per-tensor scales on the gfx950 matrix cores:
// out = out_dtype((Aq . Bq)_f32 * (scale_a * scale_b)).  The benchmark's quantised
// configuration; the reference has no fp8 payload.
//
// Direct kernel (M and N multiples of 256, the benchmark shape): described at gemm8_direct below;
// v_mfma_f32_16x16x128_f8f6f4 on panels that go global -> LDS without passing through registers.
//
// Register-staged kernel (other row counts): workgroup tile 256 x 256 x 128, 8 waves, v_mfma_f32_32x32x64_f8f6f4, A and B
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

// EDGE_M: M need not be a multiple of the tile: rows past the end are loaded from the last row
// (their products land in accumulators that are never stored) and the epilogue skips them.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool EDGE_M>
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
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = g.N / BN;
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
      const int arow = EDGE_M ? min(m0 + row, g.M - 1) : m0 + row;
      ra[i] = *reinterpret_cast<const u32x4*>(A + (int64_t)arow * g.lda + k0 + kc * 16);
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
        if (!EDGE_M || m_base + 32 * j < g.M)
          epilogue4<LH_BF16>(g, m_base + 32 * j, n_base + 32 * i + 8 * q, acc[i][j][4 * q], acc[i][j][4 * q + 1],
                             acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
}

// ---- direct-to-LDS kernel ---------------------------------------------------------------
// Same structure as the 16-bit direct kernel: 256 x 256 workgroup tile, 8 waves (2 x 4, 128 x 64
// per wave), panels global -> LDS with buffer_load_dwordx4 ... lds in their global orientation, A ring
// 2 stages x 128 k (256 rows x 128 bytes), B ring 4 stages x 64 k (64 rows x 256 bytes), used as
// two pairs of 128 k.  The matrix instruction is v_mfma_f32_16x16x128_f8f6f4: on random operands
// the matrix cores hold a higher clock with it than with 32x32x64 (register-only loops: 4.43 against
// 4.04 PFLOP/s; both reach the published peak on zeros).  A main-loop step is 128 k: 8 A fragments
// of 16 rows and 4 B fragments of 16 columns per wave, in two phases (the MFMAs of the lower four
// A fragments, then of the upper four), with one barrier per step between the phases.
// The k-contiguous A fragment (32 bytes per lane) is two 16-byte LDS reads; the n-contiguous B
// panel is read with ds_read_b64_tr_b8, which hands a lane 8 k-values of one column (16 lanes
// cover 8 k-rows x 16 columns), four reads per fragment.  Swizzles: A chunk ^ ((row / 2) % 8),
// B chunk ^ 2 (k % 8) ^ ((k / 16) % 2).
constexpr int kD8ABytes = 256 * 128;   // one A stage (128 k): 32 KiB
constexpr int kD8BBytes = 64 * 256;    // one B stage (64 k): 16 KiB
constexpr int kD8BBase = 2 * kD8ABytes;
constexpr int kD8RingBytes = kD8BBase + 4 * kD8BBytes;  // 128 KiB
constexpr int kD8LdsBytes = kD8RingBytes + 8 * 32 * 128;  // + bf16 output staging, 32 rows per wave at a time

typedef __attribute__((address_space(3))) void lds8_void_t;
typedef int i32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void async8_copy16(const void* gsrc, uint8_t* lds_wave_base) {
  __builtin_amdgcn_global_load_lds(gsrc, (lds8_void_t*)lds_wave_base, 16, 0, 0);
}
// The buffer form of the same load (base + per-lane + scalar byte offsets).  The direct kernel uses
// it: with the global (flat-encoded) form in flight the compiler must assume LDS operations complete
// out of order and waits for all of a wave's LDS reads before the first use of any; with the buffer
// form it counts them, and an MFMA waits for its own fragments only.
__device__ __forceinline__ void dma8_16(const void* base, uint32_t lane_bytes, uint32_t scalar_bytes,
                                        uint8_t* lds_wave_base) {
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds8_void_t*)lds_wave_base, 16, (int)lane_bytes, (int)scalar_bytes, 0, 0);
}

struct D8Ctx {
  // Sources of the lane's loads at k = 0: a wave-uniform base (the tile's first A row / B column)
  // plus a 32-bit byte offset per load (at most 255 lda, 63 ldb + 255).
  const uint8_t* a_base;
  const uint8_t* b_base;
  uint32_t a_voff[4];
  uint32_t b_voff[2];
  int a_rd;  // byte offset of the lane's first 16 bytes of A fragment 0 in a stage (row wm0 + lane % 16, chunk
             // lane / 16, swizzled); its second 16 bytes (chunk + 4) are at a_rd ^ 64, fragment jj 2048 jj further on
  int64_t ldb;
  int wave, b_off, b_chunk, b_swz;
};

// Fragments in registers: the A fragments of the lower (a[0]) and upper (a[1]) half of the wave's
// rows, four of 16 rows each, and the step's four B fragments of 16 columns.
struct D8Frags {
  i32x8 a[2][4];
  i32x8 b[4];
};

__device__ __forceinline__ void d8_load_a(const D8Ctx& c, int sa, uint8_t* __restrict__ abuf) {
#pragma unroll
  for (int i = 0; i < 4; ++i) dma8_16(c.a_base, c.a_voff[i], (uint32_t)(sa * 128), abuf + (8 * i + c.wave) * 1024);
}
__device__ __forceinline__ void d8_load_b(const D8Ctx& c, int sb, uint8_t* __restrict__ bbuf) {
  // (the resource starts at the stage's first k row: lane offsets stay within 64 rows)
  const uint8_t* stage_base = c.b_base + (int64_t)(sb * 64) * c.ldb;
#pragma unroll
  for (int i = 0; i < 2; ++i) dma8_16(stage_base, c.b_voff[i], 0u, bbuf + (8 * i + c.wave) * 1024);
}

// A fragments HALF * 4 .. + 4 (16 rows each) of the 128-k stage `as`.
template <int HALF>
__device__ __forceinline__ void d8_read_a(const D8Ctx& c, const uint8_t* __restrict__ as, i32x8 (&a)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    i32x4 lo = *reinterpret_cast<const i32x4*>(as + c.a_rd + 2048 * (4 * HALF + j));
    i32x4 hi = *reinterpret_cast<const i32x4*>(as + (c.a_rd ^ 64) + 2048 * (4 * HALF + j));
    a[j] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }
}
// B fragment i (16 columns) of the 128 k held by the stage pair `bs` (two consecutive 64-k stages).
__device__ __forceinline__ i32x8 d8_read_b(const D8Ctx& c, const uint8_t* __restrict__ bs, int i) {
  const uint8_t* p0 = bs + c.b_off + (((c.b_chunk + i) ^ c.b_swz) << 4);
  i32x2 r[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)  // k rows 16 g4 + 8 (q % 2) + 64 (q / 2) + ...: the k order of the A fragment
    r[q] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
        (__attribute__((address_space(3))) i32x2*)(p0 + (q & 1) * 8 * 256 + (q >> 1) * 64 * 256));
  return i32x8{r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]};
}

// NR LDS reads spread over the 16 MFMAs of a phase.
template <int NR, int I = 0>
__device__ __forceinline__ void d8_interleave_hint() {
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  __builtin_amdgcn_sched_group_barrier(0x100, (I + 1) * NR / 16 - I * NR / 16, 0);
  if constexpr (I + 1 < 16) d8_interleave_hint<NR, I + 1>();
}

// All loads of this wave have landed and all its LDS reads have returned, then barrier.  One asm
// block: a __syncthreads() would add a release fence.
__device__ __forceinline__ void d8_wait_barrier() {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// First phase of a step: the MFMAs of the lower row fragments under the reads of the step's upper ones.
__device__ __forceinline__ void d8_phase_lo(const D8Ctx& c, f32x4 (&acc)[4][8], D8Frags& f,
                                            const uint8_t* __restrict__ as) {
  d8_read_a<1>(c, as, f.a[1]);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = mfma_f8_16(f.b[i], f.a[0][j], acc[i][j]);
  d8_interleave_hint<8>();
}
// Second phase: the MFMAs of the upper row fragments under the reads of the NEXT step's lower row
// fragments (A stage `as_n`) and B fragments (stage pair `bs_n`), each B fragment requested behind
// the last MFMA that uses the one it replaces.  LOAD false: a tile's last step.
template <bool LOAD = true>
__device__ __forceinline__ void d8_phase_hi(const D8Ctx& c, f32x4 (&acc)[4][8], D8Frags& f,
                                            const uint8_t* __restrict__ as_n, const uint8_t* __restrict__ bs_n) {
  if constexpr (LOAD) d8_read_a<0>(c, as_n, f.a[0]);
  i32x8 bn[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][4 + j] = mfma_f8_16(f.b[i], f.a[1][j], acc[i][4 + j]);
    if constexpr (LOAD) bn[i] = d8_read_b(c, bs_n, i);
  }
  if constexpr (LOAD) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f.b[i] = bn[i];
    d8_interleave_hint<24>();
  }
}

// Step kt / 2 of 128 k (B stages kt and kt + 1).  f holds the step's lower A fragments and its B
// fragments on entry and the next step's on exit.  ONE barrier, between the two phases: at the
// barrier every fragment of this step's stages has been read and the next step's stages
// (requested at the previous barrier, 128 k ago) are awaited in full; the step after that is then
// requested into this step's buffers.  (Two barriers per 128 k with B requested three stages ahead,
// as in the small tiles of the 16-bit kernel, measured 2-2.5 % slower: 8192^3 426 -> 416 us.)
__device__ __forceinline__ void d8_step(const D8Ctx& c, f32x4 (&acc)[4][8], D8Frags& f,
                                        const uint8_t* __restrict__ a_cur, const uint8_t* __restrict__ a_nxt,
                                        const uint8_t* __restrict__ b_nxt, uint8_t* __restrict__ a_refill,
                                        uint8_t* __restrict__ b_refill0, uint8_t* __restrict__ b_refill1, int kt,
                                        int nk) {
  d8_phase_lo(c, acc, f, a_cur);
  d8_wait_barrier();
  if (kt + 4 < nk) {
    d8_load_a(c, kt / 2 + 2, a_refill);
    d8_load_b(c, kt + 4, b_refill0);
    d8_load_b(c, kt + 5, b_refill1);
  }
  d8_phase_hi(c, acc, f, a_nxt, b_nxt);
}

// Source pointers of tile `id` (its position in the XCD-grouped order) and the tile's origin.
__device__ __forceinline__ void d8_place(const GemmArgs& g, int id, D8Ctx& c, int& m0, int& n0) {
  constexpr int BM = 256, BN = 256;
  const int lane = lane_now();  // the lane's offsets are recomputed per tile rather than kept in registers
  const int tiles_m = g.M / BM, tiles_n = g.N / BN;
  constexpr int GROUP_M = 4;
  const int group_size = GROUP_M * tiles_n;
  const int first_m = (id / group_size) * GROUP_M;
  const int gm = min(tiles_m - first_m, GROUP_M);
  m0 = (first_m + (id % group_size) % gm) * BM;
  n0 = ((id % group_size) / gm) * BN;
  c.a_base = reinterpret_cast<const uint8_t*>(g.a) + (int64_t)m0 * g.lda;
  c.b_base = reinterpret_cast<const uint8_t*>(g.b) + n0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ar = (8 * i + c.wave) * 8 + (lane >> 3);
    const int ac = (lane & 7) ^ ((ar >> 1) & 7);
    c.a_voff[i] = (uint32_t)ar * (uint32_t)g.lda + ac * 16;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int bk = (8 * i + c.wave) * 4 + (lane >> 4);
    const int bc = (lane & 15) ^ (2 * (bk & 7)) ^ ((bk >> 4) & 1);
    c.b_voff[i] = (uint32_t)bk * (uint32_t)g.ldb + bc * 16;
  }
}

// First loads of a tile: A stages 0, 1 and B stages 0 .. 3 (nk = K / 64 >= 2).
__device__ __forceinline__ void d8_prologue(const D8Ctx& c, int nk, uint8_t* __restrict__ ring) {
  d8_load_a(c, 0, ring);
  if (nk > 2) d8_load_a(c, 1, ring + kD8ABytes);
#pragma unroll
  for (int st = 0; st < 4; ++st)
    if (st < nk) d8_load_b(c, st, ring + kD8BBase + st * kD8BBytes);
}

// Main loop of one tile, whose first loads have been issued.
__device__ __forceinline__ void d8_mainloop(const D8Ctx& c, f32x4 (&acc)[4][8], uint8_t* smem_8, int nk) {
  uint8_t* const abuf = smem_8;
  uint8_t* const bbuf = smem_8 + kD8BBase;
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  D8Frags f;
  d8_read_a<0>(c, abuf, f.a[0]);
#pragma unroll
  for (int i = 0; i < 4; ++i) f.b[i] = d8_read_b(c, bbuf, i);
  int kt = 0;
  for (; kt + 2 < nk; kt += 2) {
    uint8_t* a_cur = abuf + ((kt >> 1) & 1) * kD8ABytes;
    uint8_t* a_nxt = abuf + (((kt >> 1) + 1) & 1) * kD8ABytes;
    uint8_t* b0 = bbuf + (kt & 3) * kD8BBytes;         // kt is even: stages kt and kt + 1 are adjacent
    uint8_t* b2 = bbuf + ((kt + 2) & 3) * kD8BBytes;
    d8_step(c, acc, f, a_cur, a_nxt, b2, a_cur, b0, b0 + kD8BBytes, kt, nk);
  }
  {
    // (the last step's stages were awaited at the barrier of the step before, or at the start)
    const uint8_t* a_cur = abuf + ((kt >> 1) & 1) * kD8ABytes;
    d8_phase_lo(c, acc, f, a_cur);
    d8_phase_hi<false>(c, acc, f, a_cur, a_cur);
  }
}

// End of a tile: once every wave has left the rings, the first loads of the workgroup's next tile
// are issued into them, then the accumulators are written out.  bf16 outputs are staged through
// `stage`, an LDS area of its own (32 rows of the wave's 128 x 64 sub-tile at a time, 16-byte
// chunk ^ ((row / 2) % 8) against bank conflicts); the last tile of a workgroup stages its whole
// sub-tile in the idle rings at once.  `ring` and `stage` are separate restrict parameters so
// that the staging traffic does not wait for the asynchronous ring writes.
template <bool HAS_NEXT>
__device__ __forceinline__ void d8_finish(const GemmArgs& g, const D8Ctx& next, int nk, uint8_t* __restrict__ ring,
                                          uint8_t* __restrict__ stage, const f32x4 (&acc)[4][8], int m0, int n0, int wm0,
                                          int wn0) {
  constexpr int TM = 4, RB = 128, chunks = 8, rows_per_pass = 8;
  // Accumulator acc[i][j][e] of a lane: row wm0 + 16 j + lane % 16, column wn0 + 16 i + 4 (lane / 16) + e.
  const int lane = lane_now();  // keeps the addresses below out of registers during the main loop
  const int l16 = lane & 15, g4 = lane >> 4;
  const int m_base = m0 + wm0 + l16;
  const int n_base = n0 + wn0 + 4 * g4;
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the rings
  if constexpr (HAS_NEXT) d8_prologue(next, nk, ring);
  if (g.out_dt != LH_F32) {
    constexpr int JB = HAS_NEXT ? 1 : TM;
    uint8_t* cw = HAS_NEXT ? stage + next.wave * (32 * RB) : ring + next.wave * (TM * 32 * RB);
    uint16_t* outp = reinterpret_cast<uint16_t*>(g.out);
    // One variant of the scale / bias / activation code per tile (epi_dispatch), not a test of the
    // call's flags per element group.
    epi_dispatch(g, [&](auto variant) {
      using E = decltype(variant);
      f32x4 b4[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) b4[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (epi_has_bias<E>(g)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) b4[i] = bias4<LH_BF16>(g, n_base + 16 * i);
      }
#pragma unroll
      for (int j0 = 0; j0 < TM; j0 += JB) {
#pragma unroll
        for (int jj = 0; jj < 2 * JB; ++jj)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int j = 2 * j0 + jj;
            const u32x2 w = epi_pack4<LH_BF16, E>(g, b4[i], acc[i][j]);
            const int row = 16 * jj + l16;
            *reinterpret_cast<u32x2*>(cw + row * RB + (((2 * i + (g4 >> 1)) ^ ((row >> 1) & (chunks - 1))) << 4) +
                                      8 * (g4 & 1)) = w;
          }
#pragma unroll
        for (int t = 0; t < JB * 32 / rows_per_pass; ++t) {
          const int row = rows_per_pass * t + lane / chunks, ch = lane % chunks;
          u32x4 w = *reinterpret_cast<const u32x4*>(cw + row * RB + ((ch ^ ((row >> 1) & (chunks - 1))) << 4));
          *reinterpret_cast<u32x4*>(outp + (int64_t)(m0 + wm0 + 32 * j0 + row) * g.ldc + n0 + wn0 + ch * 8) = w;
        }
      }
    });
    return;
  }
  // f32 output (the blocks of a cut along K among them): no accumulator input in this kernel
  epi_dispatch_linear(g, [&](auto variant) {
    using E = decltype(variant);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f32x4 b4 = {0.0f, 0.0f, 0.0f, 0.0f};
      if (epi_has_bias<E>(g)) b4 = bias4<LH_BF16>(g, n_base + 16 * i);
#pragma unroll
      for (int j = 0; j < 8; ++j) epi_store4<LH_BF16, E, true, false>(g, m_base + 16 * j, n_base + 16 * i, b4, acc[i][j]);
    }
  });
}

// Persistent workgroups, one per CU, each walking the tile list with the grid as stride (tile
// ids congruent modulo 8 stay on one XCD, which is what xcd_remap assumes).
// SPLITK: the tile list is g.splits copies of the problem's tiles, copy sp working on its own K
// columns of A / rows of B and its own f32 block of the output; a second kernel adds the blocks,
// scales and converts.  For problems with too few tiles for the CUs and a long K.
template <bool SPLITK>
__global__ void __launch_bounds__(512) gemm8_direct(GemmArgs g) {
  constexpr int TM = 4, TN = 2, WN = 4, WTN = 64;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_8[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WN) * 128, wn0 = (wave % WN) * WTN;
  const int tiles1 = (g.M / 256) * (g.N / 256);
  const int ntiles = SPLITK ? tiles1 * g.splits : tiles1;
  GemmArgs g_cur = g, g_nxt = g;  // (SPLITK) the problem copy of the current / next tile
  auto select = [&](int t, GemmArgs& ga) -> int {
    if constexpr (SPLITK) {
      const int sp = t / tiles1;
      ga.a = reinterpret_cast<const uint8_t*>(g.a) + (int64_t)sp * g.K;
      ga.b = reinterpret_cast<const uint8_t*>(g.b) + (int64_t)sp * g.K * g.ldb;
      ga.out = reinterpret_cast<float*>(g.out) + (int64_t)sp * g.M * g.ldc;
      ga.c = ga.out;
      return t - sp * tiles1;
    }
    return t;
  };

  D8Ctx c;
  c.ldb = g.ldb;
  c.wave = wave;
  const int l16 = lane & 15, g4 = lane >> 4;
  {
    // A fragment jj: row wm0 + 16 jj + l16.  The lane's 32 k values are the 16-byte chunks g4 and g4 + 4
    // of the row's eight (k = 16 g4 .. +16 and 64 + 16 g4 .. +16), not two neighbouring chunks: the matrix
    // instruction only needs A and B to agree on which k a lane holds, and with the four lane groups
    // on four neighbouring chunks a 16-byte read is free of bank conflicts (on chunks 2 g4 and 2 g4 + 1
    // every such read took twice as long: SQ_LDS_BANK_CONFLICT 3.5e7 per 8192^3 launch against 1e6).
    // Swizzled with (row / 2) % 8 (the same for every jj: wm0 and 16 jj are multiples of 16).
    const int r = wm0 + l16;
    c.a_rd = r * 128 + ((g4 ^ ((r >> 1) & 7)) << 4);
  }
  {
    // B fragment i: the 16 lanes of group g4 address k rows 16 g4 + 8 (q % 2) + 64 (q / 2) + l16 / 2
    // (q = 0..3) of the stage pair, the k values of the lane's A chunks, columns
    // wn0 + 16 i + 8 (l16 % 2) .. +8; each lane receives the 8 k-values per q of column wn0 + 16 i + l16.
    const int krow = 16 * g4 + (l16 >> 1);
    const int col = wn0 + 8 * (l16 & 1);
    c.b_chunk = col >> 4;
    c.b_swz = (2 * (krow & 7)) ^ (g4 & 1);
    c.b_off = krow * 256 + (col & 8);
  }

  const int nk = g.K / 64;  // even: K is a multiple of 128
  int t = blockIdx.x;       // < ntiles: the grid is never larger than the tile list
  int m0, n0;
  {
    const int id = select(t, g_cur);
    d8_place(SPLITK ? g_cur : g, xcd_remap(id, tiles1), c, m0, n0);
  }
  d8_prologue(c, nk, smem_8);
  for (;;) {
    f32x4 acc[4][8];  // [16-column fragment][16-row fragment]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0f;
    d8_mainloop(c, acc, smem_8, nk);
    const int tn = t + (int)gridDim.x;
    const bool more = tn < ntiles;
    D8Ctx cn = c;
    int m1 = 0, n1 = 0;
    uint8_t* const stage = smem_8 + kD8RingBytes;
    const GemmArgs& ga = SPLITK ? g_cur : g;
    if (more) {
      const int idn = select(tn, g_nxt);
      d8_place(SPLITK ? g_nxt : g, xcd_remap(idn, tiles1), cn, m1, n1);
      d8_finish<true>(ga, cn, nk, smem_8, stage, acc, m0, n0, wm0, wn0);
    } else {
      d8_finish<false>(ga, cn, nk, smem_8, stage, acc, m0, n0, wm0, wn0);
    }
    if (!more) break;
    if constexpr (SPLITK) g_cur = g_nxt;
    c = cn;
    m0 = m1;
    n0 = n1;
    t = tn;
  }
}

static int launch_direct8(const GemmArgs& g, hipStream_t s) {
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_direct<false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kD8LdsBytes));
    configured = true;
  }
  const int ntiles = (g.M / 256) * (g.N / 256), cus = num_cus();
  LH_LAUNCH(gemm8_direct<false>, dim3(ntiles < cus ? ntiles : cus), dim3(512), kD8LdsBytes, s, g);
  return check_launch("gemm8_direct");
}

// Sum of the split-K blocks ([splits][M][N] f32), scale, conversion: 4 columns per thread.
__global__ void __launch_bounds__(256) gemm8_splitk_reduce(GemmArgs g, const float* partial, int splits) {
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= (int64_t)g.M * g.N) return;
  const int m = (int)(idx / g.N), n = (int)(idx % g.N);
  const f32x4 v = splitk_sum4(partial + (int64_t)m * g.N + n, (int64_t)g.M * g.N, splits, blockDim.x == 64);
  epilogue4<LH_BF16>(g, m, n, v[0], v[1], v[2], v[3]);
}

// Too few 256 x 256 tiles for the CUs and a K long enough to cut.  Returns 1 when the problem does
// not qualify.
static int gemm8_splitk(const GemmArgs& g, hipStream_t s) {
  const int cus = num_cus();
  const int64_t tiles = (int64_t)(g.M / 256) * (g.N / 256);
  // Measured against the uncut kernel (M 256 ... 4096, N 1024 ... 8192): cutting pays from K = 8192 on,
  // and at K = 4096 only when the tiles cover at most an eighth of the CUs (four cuts); below
  // that the partial blocks and the second kernel cost more than the shorter main loop saves
  // (512 x 8192 x 2048: 30.3 us cut, 20.9 us whole; 256 x 1024 x 8192: 26 us cut, 62 us whole).
  if (tiles * 2 > cus || g.K < 4096) return 1;
  if (g.K < 8192 && tiles * 8 > cus) return 1;
  int splits = 1;
  while (splits < 8 && tiles * splits * 2 <= cus && (g.K / (splits * 2)) % kBK8 == 0 && g.K / (splits * 2) >= 1024)
    splits *= 2;
  if (splits == 1) return 1;
  void* taken = nullptr;
  if (int rc = scratch_take(g.ws, s, kScratchSplitK, (size_t)splits * g.M * g.N * sizeof(float), "fp8 gemm (split K)", &taken))
    return rc;
  float* partial = static_cast<float*>(taken);
  GemmArgs p = g;
  p.K = g.K / splits;
  p.splits = splits;
  p.out = partial;
  p.c = partial;
  p.ldc = g.N;
  p.out_dt = LH_F32;
  p.alpha = 1.0f;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_direct<true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kD8LdsBytes));
    configured = true;
  }
  const int64_t total = tiles * splits;
  LH_LAUNCH(gemm8_direct<true>, dim3((unsigned)(total < cus ? total : cus)), dim3(512), kD8LdsBytes, s, p);
  int rc = check_launch("gemm8_direct (split K)");
  if (rc) return rc;
  const int64_t groups = (int64_t)g.M * g.N / 4;
  const int rb = reduce_block(groups);
  LH_LAUNCH(gemm8_splitk_reduce, dim3((unsigned)((groups + rb - 1) / rb)), dim3(rb), 0, s, g, partial, splits);
  return check_launch("gemm8_splitk_reduce");
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
// M <= 16: the job is streaming B once from HBM.  Grid (N / 256, splits); a workgroup of 4 waves
// owns 256 columns and a K chunk, wave w the columns 64 w .. 64 w + 63 (four 16-wide MFMA tiles,
// v_mfma_scale_f32_16x16x128_f8f6f4 with M padded to 16).  B goes global -> LDS with
// global_load_lds_dwordx4 in its global orientation (k rows of 256 contiguous bytes) through a
// ring of 4 stages of 128 k, three of them in flight (96 KiB per CU, what the HBM
// latency-bandwidth product needs); fragments come from ds_read_b64_tr_b8.  The A chunk (16 rows)
// is staged once, as one 16 x 128-byte block per k-step.  Rows cannot be padded (a wave-wide load
// writes 1 KiB contiguously): the 16-byte chunk a lane fetches is XOR-swizzled, B chunk ^
// (k % 8 + 8 ((k / 32) % 2)), A chunk ^ ((m / 2) % 8).
// Partial sums go to partial[split][16][N] (f32); gemm8_skinny_reduce adds them and runs the
// epilogue.
constexpr int kSkinnyBN = 256;
constexpr int kSkinnyStages = 4;
constexpr int kSkinnyStageBytes = kBK8 * kSkinnyBN;  // 32 KiB
constexpr int kSkinnyMaxChunk = 1024;                // K chunk whose A block fits the 16 KiB A area
constexpr int kSkinnyLdsBytes = kSkinnyStages * kSkinnyStageBytes + 16 * kSkinnyMaxChunk;

__device__ __forceinline__ void skinny_issue_b(const uint8_t* const (&b_src)[8], int64_t ldb, int kt, int wave,
                                               uint8_t* __restrict__ stage) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    async8_copy16(b_src[i] + (int64_t)(kt * kBK8) * ldb, stage + (4 * i + wave) * 1024);
}

// One k-step: refill `wr` (if `prefetch`) and multiply the stage in `bs`.  The LDS reads and the
// asynchronous LDS writes go through separate restrict pointers of one function, otherwise the
// compiler makes every LDS read wait for all outstanding loads.
__device__ __forceinline__ void skinny_step(f32x4 (&acc)[4], const uint8_t* __restrict__ bs,
                                            const uint8_t* __restrict__ as, uint8_t* __restrict__ wr,
                                            const uint8_t* const (&b_src)[8], int64_t ldb, int next_kt, bool prefetch,
                                            int wave, int a_off, int a_swz, int qd, int b_off, int b_chunk, int b_swz) {
  if (prefetch) skinny_issue_b(b_src, ldb, next_kt, wave, wr);
  const int c0 = 2 * qd;
  i32x4 alo = *reinterpret_cast<const i32x4*>(as + a_off + ((c0 ^ a_swz) << 4));
  i32x4 ahi = *reinterpret_cast<const i32x4*>(as + a_off + (((c0 + 1) ^ a_swz) << 4));
  i32x8 fa = {alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint8_t* p0 = bs + b_off + (((b_chunk + i) ^ b_swz) << 4);
    i32x2 r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      r[q] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(p0 + q * 8 * kSkinnyBN));
    i32x8 fb = {r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]};
    // First operand = B panel: the accumulator of lane (m = r16, quarter qd) holds columns
    // n = 4 qd + v of row m.
    acc[i] = mfma_f8_16(fb, fa, acc[i]);
  }
}

template <int N>
__device__ __forceinline__ void skinny_wait_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

__global__ void __launch_bounds__(256) gemm8_skinny(GemmArgs g, float* partial, int k_chunk) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_sk[];
  uint8_t* const ring = smem_sk;
  uint8_t* const a_lds = smem_sk + kSkinnyStages * kSkinnyStageBytes;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * kSkinnyBN;
  const int kbeg = blockIdx.y * k_chunk;
  const int nk = k_chunk / kBK8;
  const uint8_t* A = reinterpret_cast<const uint8_t*>(g.a);
  const uint8_t* B = reinterpret_cast<const uint8_t*>(g.b);
  const int r16 = lane & 15, qd = lane >> 4;

  // A: k-step t is a 16 x 128-byte block (2 KiB = 2 wave-wide loads); wave w loads the halves
  // u = w, w + 4, ... of the 2 nk halves.  Rows >= M repeat row M - 1 (their results are unused).
  for (int u = wave; u < 2 * nk; u += 4) {
    const int m = 8 * (u & 1) + (lane >> 3);
    const int gc = (lane & 7) ^ ((m >> 1) & 7);
    const int row = m < g.M ? m : g.M - 1;
    async8_copy16(A + (int64_t)row * g.lda + kbeg + (u >> 1) * kBK8 + gc * 16, a_lds + u * 1024);
  }
  // B: load i of wave w fills k rows (4 i + w) 4 .. +4 of a stage; lane -> row += lane / 16, LDS
  // chunk lane % 16.
  const uint8_t* b_src[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int k = (4 * i + wave) * 4 + (lane >> 4);
    const int gc = (lane & 15) ^ ((k & 7) | (((k >> 5) & 1) << 3));
    b_src[i] = B + (int64_t)(kbeg + k) * g.ldb + n0 + gc * 16;
  }
#pragma unroll
  for (int st = 0; st < kSkinnyStages - 1; ++st)
    if (st < nk) skinny_issue_b(b_src, g.ldb, st, wave, ring + st * kSkinnyStageBytes);

  // Fragment addressing.  A: row r16 of the step's block, logical chunks 2 qd, 2 qd + 1.  B
  // through the transposing read: lane (j = lane % 16, quarter qd) addresses k row
  // 32 qd + 8 q + j / 2, bytes 16 (4 w + i) + 8 (j % 2) .. +8 of it.
  const int a_off = r16 * 128, a_swz = (r16 >> 1) & 7;
  const int b_off = (32 * qd + (r16 >> 1)) * kSkinnyBN + 8 * (r16 & 1);
  const int b_chunk = 4 * wave;
  const int b_swz = (r16 >> 1) | ((qd & 1) << 3);

  f32x4 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[i][v] = 0.0f;

  for (int kt = 0; kt < nk; ++kt) {
    // Stages kt + 1, kt + 2 may stay in flight (8 loads per lane each); the A loads were issued
    // first and are older than every B stage.
    const int younger = min(nk - 1 - kt, kSkinnyStages - 2);
    if (younger >= 2) skinny_wait_barrier<16>();
    else if (younger == 1) skinny_wait_barrier<8>();
    else skinny_wait_barrier<0>();
    const int nxt = kt + kSkinnyStages - 1;
    skinny_step(acc, ring + (kt % kSkinnyStages) * kSkinnyStageBytes, a_lds + kt * 2048,
                ring + (nxt % kSkinnyStages) * kSkinnyStageBytes, b_src, g.ldb, nxt, nxt < nk, wave, a_off, a_swz, qd,
                b_off, b_chunk, b_swz);
  }
  float* dst = partial + ((int64_t)blockIdx.y * 16 + r16) * g.N + n0 + wave * 64 + 4 * qd;
#pragma unroll
  for (int i = 0; i < 4; ++i) *reinterpret_cast<f32x4*>(dst + 16 * i) = acc[i];
}

// 16 < M <= 128 (decode batches): the same streaming scheme with MT = 2, 4 or 8 row groups of 16, so
// that B is still read once.  The A block of a k-step (16 MT rows x 128 bytes; rows >= M repeat the
// last row) travels through the ring next to the B stage it belongs to, so the K chunk of a
// workgroup is not limited by an A area and the waits count A and B loads alike.  A stage is
// 32 + 2 MT KiB; MT <= 4: a ring of 4 stages (the whole 160 KiB of a CU with MT = 4), MT = 8: 3
// stages of 48 KiB.  Partial sums: partial[split][16 MT][N].
template <int MT>
struct SkinnyMt {
  static constexpr int kStages = MT == 8 ? 3 : 4;
  static constexpr int kStageBytes = kSkinnyStageBytes + (MT < 4 ? 4 : MT) * 16 * kBK8;
  static constexpr int kLdsBytes = kStages * kStageBytes;
};

template <int MT>
__device__ __forceinline__ void skinny_mt_issue(const uint8_t* const (&b_src)[8], const uint8_t* const (&a_src)[MT / 2],
                                                int64_t ldb, int kt, int wave, uint8_t* __restrict__ stage) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    async8_copy16(b_src[i] + (int64_t)(kt * kBK8) * ldb, stage + (4 * i + wave) * 1024);
#pragma unroll
  for (int i = 0; i < MT / 2; ++i)
    async8_copy16(a_src[i] + kt * kBK8, stage + kSkinnyStageBytes + (4 * i + wave) * 1024);
}

template <int MT>
__device__ __forceinline__ void skinny_mt_step(f32x4 (&acc)[MT][4], const uint8_t* __restrict__ st,
                                               uint8_t* __restrict__ wr, const uint8_t* const (&b_src)[8],
                                               const uint8_t* const (&a_src)[MT / 2], int64_t ldb, int next_kt,
                                               bool prefetch, int wave, int a_off, int a_swz, int qd, int b_off,
                                               int b_chunk, int b_swz) {
  if (prefetch) skinny_mt_issue<MT>(b_src, a_src, ldb, next_kt, wave, wr);
  const uint8_t* as = st + kSkinnyStageBytes;
  const int c0 = 2 * qd;
  i32x8 fa[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    i32x4 alo = *reinterpret_cast<const i32x4*>(as + mt * 2048 + a_off + ((c0 ^ a_swz) << 4));
    i32x4 ahi = *reinterpret_cast<const i32x4*>(as + mt * 2048 + a_off + (((c0 + 1) ^ a_swz) << 4));
    fa[mt] = i32x8{alo[0], alo[1], alo[2], alo[3], ahi[0], ahi[1], ahi[2], ahi[3]};
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint8_t* p0 = st + b_off + (((b_chunk + i) ^ b_swz) << 4);
    i32x2 r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      r[q] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(p0 + q * 8 * kSkinnyBN));
    i32x8 fb = {r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt][i] = mfma_f8_16(fb, fa[mt], acc[mt][i]);
  }
}

template <int MT>
__global__ void __launch_bounds__(256) gemm8_skinny_mt(GemmArgs g, float* partial, int k_chunk) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_sk[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * kSkinnyBN;
  const int kbeg = blockIdx.y * k_chunk;
  const int nk = k_chunk / kBK8;
  const uint8_t* A = reinterpret_cast<const uint8_t*>(g.a);
  const uint8_t* B = reinterpret_cast<const uint8_t*>(g.b);
  const int r16 = lane & 15, qd = lane >> 4;

  // A: load i of wave w fills rows (4 i + w) 8 .. +8 of the step's block; lane -> row += lane / 8,
  // LDS chunk lane % 8 holds global chunk (lane % 8) ^ ((row / 2) % 8).
  const uint8_t* a_src[MT / 2];
#pragma unroll
  for (int i = 0; i < MT / 2; ++i) {
    const int m = (4 * i + wave) * 8 + (lane >> 3);
    const int gc = (lane & 7) ^ ((m >> 1) & 7);
    a_src[i] = A + (int64_t)min(m, g.M - 1) * g.lda + kbeg + gc * 16;
  }
  const uint8_t* b_src[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int k = (4 * i + wave) * 4 + (lane >> 4);
    const int gc = (lane & 15) ^ ((k & 7) | (((k >> 5) & 1) << 3));
    b_src[i] = B + (int64_t)(kbeg + k) * g.ldb + n0 + gc * 16;
  }
#pragma unroll
  for (int st = 0; st < SkinnyMt<MT>::kStages - 1; ++st)
    if (st < nk) skinny_mt_issue<MT>(b_src, a_src, g.ldb, st, wave, smem_sk + st * SkinnyMt<MT>::kStageBytes);

  const int a_off = r16 * 128, a_swz = (r16 >> 1) & 7;
  const int b_off = (32 * qd + (r16 >> 1)) * kSkinnyBN + 8 * (r16 & 1);
  const int b_chunk = 4 * wave;
  const int b_swz = (r16 >> 1) | ((qd & 1) << 3);

  f32x4 acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[mt][i][v] = 0.0f;

  constexpr int L = 8 + MT / 2;  // loads per lane and stage
  for (int kt = 0; kt < nk; ++kt) {
    const int younger = min(nk - 1 - kt, SkinnyMt<MT>::kStages - 2);
    if (younger >= 2) skinny_wait_barrier<2 * L>();
    else if (younger == 1) skinny_wait_barrier<L>();
    else skinny_wait_barrier<0>();
    const int nxt = kt + SkinnyMt<MT>::kStages - 1;
    skinny_mt_step<MT>(acc, smem_sk + (kt % SkinnyMt<MT>::kStages) * SkinnyMt<MT>::kStageBytes,
                       smem_sk + (nxt % SkinnyMt<MT>::kStages) * SkinnyMt<MT>::kStageBytes, b_src, a_src, g.ldb, nxt, nxt < nk, wave,
                       a_off, a_swz, qd, b_off, b_chunk, b_swz);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float* dst = partial + ((int64_t)blockIdx.y * (16 * MT) + 16 * mt + r16) * g.N + n0 + wave * 64 + 4 * qd;
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<f32x4*>(dst + 16 * i) = acc[mt][i];
  }
}

// Sum of the split-K blocks partial[split][rows][N] and the epilogue, 4 columns per thread.
__global__ void __launch_bounds__(256) gemm8_skinny_reduce(GemmArgs g, const float* partial, int splits, int rows) {
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= (int64_t)g.M * g.N) return;
  const int m = (int)(idx / g.N), n = (int)(idx % g.N);
  const f32x4 v = splitk_sum4(partial + (int64_t)m * g.N + n, (int64_t)rows * g.N, splits, blockDim.x == 64);
  epilogue4<LH_BF16>(g, m, n, v[0], v[1], v[2], v[3]);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool EDGE_M = false>
static int launch_fast8(const GemmArgs& g, hipStream_t s) {
  auto kern = gemm8_fast<BM, BN, WAVES_M, WAVES_N, EDGE_M>;
  constexpr size_t lds = (size_t)2 * (BM + BN) * kStride8;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  LH_LAUNCH(kern, dim3(((g.M + BM - 1) / BM) * (g.N / BN)), dim3(WAVES_M * WAVES_N * 64), lds, s, g);
  return check_launch("gemm8_fast");
}

// f32 partial blocks of the decode kernels, [splits][rows][N].
static int skinny_partial_buffer(const GemmArgs& g, hipStream_t s, size_t need, float** partial) {
  void* taken = nullptr;
  if (int rc = scratch_take(g.ws, s, kScratchSkinny, need, "fp8 gemm (decode partial sums)", &taken)) return rc;
  *partial = static_cast<float*>(taken);
  return LH_OK;
}

template <int MT>
static int launch_skinny_mt(const GemmArgs& g, hipStream_t s) {
  // Split K until about one workgroup per CU streams B.
  const int nblk = g.N / kSkinnyBN;
  int splits = 1;
  while (nblk * splits < num_cus() && (g.K / kBK8) % (splits * 2) == 0) splits *= 2;
  float* g_partial = nullptr;
  int rc = skinny_partial_buffer(g, s, (size_t)splits * 16 * MT * g.N * sizeof(float), &g_partial);
  if (rc) return rc;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_skinny_mt<MT>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, SkinnyMt<MT>::kLdsBytes));
    configured = true;
  }
  LH_LAUNCH(gemm8_skinny_mt<MT>, dim3(nblk, splits), dim3(256), SkinnyMt<MT>::kLdsBytes, s, g, g_partial,
                     g.K / splits);
  rc = check_launch("gemm8_skinny_mt");
  if (rc) return rc;
  const int64_t groups = (int64_t)g.M * g.N / 4;
  const int rb = reduce_block(groups);
  LH_LAUNCH(gemm8_skinny_reduce, dim3((unsigned)((groups + rb - 1) / rb)), dim3(rb), 0, s, g, g_partial, splits,
                     16 * MT);
  return check_launch("gemm8_skinny_reduce");
}

int gemm8(const GemmArgs& g, hipStream_t s) {
  const bool vec_ok = g.K % kBK8 == 0 && g.lda % 16 == 0 && g.ldb % 4 == 0 && g.ldc % 4 == 0 && aligned16(g.a) &&
                      aligned16(g.b) && aligned16(g.out);
  if (!(vec_ok && g.N % 128 == 0) && (int64_t)g.M * g.N * g.K >= (1 << 22)) {
    // K that is no multiple of the k-step, N of no tile, unaligned rows: zero-padded copies (code 0 is +0)
    const int rc = gemm_padded<1>(g, kBK8, 128, s, [&](const GemmArgs& p) { return gemm8(p, s); });
    if (rc <= 0) return rc;
  }
  if (vec_ok && g.M <= 16 && g.N % kSkinnyBN == 0 && g.ldb % 16 == 0) {
    // Split K so that about one workgroup per CU streams B (its ring alone keeps 96 KiB in
    // flight) and the A chunk fits its LDS area.
    const int nblk = g.N / kSkinnyBN;
    int splits = 1;
    while ((nblk * splits < num_cus() || g.K / splits > kSkinnyMaxChunk) && (g.K / kBK8) % (splits * 2) == 0) splits *= 2;
    if (g.K / splits <= kSkinnyMaxChunk) {
      float* g_partial = nullptr;
      int prc = skinny_partial_buffer(g, s, (size_t)splits * 16 * g.N * sizeof(float), &g_partial);
      if (prc) return prc;
      static bool configured = false;
      if (!configured && !planning()) {
        LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_skinny),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kSkinnyLdsBytes));
        configured = true;
      }
      LH_LAUNCH(gemm8_skinny, dim3(nblk, splits), dim3(256), kSkinnyLdsBytes, s, g, g_partial, g.K / splits);
      int rc = check_launch("gemm8_skinny");
      if (rc) return rc;
      const int64_t groups = (int64_t)g.M * g.N / 4;
      const int rb = reduce_block(groups);
      LH_LAUNCH(gemm8_skinny_reduce, dim3((unsigned)((groups + rb - 1) / rb)), dim3(rb), 0, s, g, g_partial,
                         splits, 16);
      return check_launch("gemm8_skinny_reduce");
    }
  }
  if (vec_ok && g.M > 16 && g.M <= 128 && g.N % kSkinnyBN == 0 && g.ldb % 16 == 0) {
    if (g.M <= 32) return launch_skinny_mt<2>(g, s);
    if (g.M <= 64) return launch_skinny_mt<4>(g, s);
    return launch_skinny_mt<8>(g, s);
  }
  if (vec_ok && g.M % 256 == 0 && g.N % 256 == 0 && g.ldb % 16 == 0 && g.ldc % 8 == 0 && g.lda < (1 << 24) &&
      g.ldb < (1 << 24)) {
    const int rc = gemm8_splitk(g, s);
    if (rc <= 0) return rc;
  }
  if (vec_ok && g.M % 256 == 0 && g.N % 256 == 0 && (int64_t)(g.M / 256) * (g.N / 256) >= 128) {
    // the direct kernel addresses a tile's rows with 32-bit byte offsets from the tile's origin
    if (g.ldb % 16 == 0 && g.ldc % 8 == 0 && g.lda < (1 << 24) && g.ldb < (1 << 24)) return launch_direct8(g, s);
    return launch_fast8<256, 256, 2, 4>(g, s);
  }
  if (vec_ok && g.M % 128 == 0 && g.N % 128 == 0) return launch_fast8<128, 128, 2, 2>(g, s);
  if (vec_ok && g.N % 128 == 0) return launch_fast8<128, 128, 2, 2, true>(g, s);  // any M
  dim3 grid((g.N + 31) / 32, (g.M + 31) / 32);
  LH_LAUNCH(gemm8_generic, grid, dim3(64), 0, s, g);
  return check_launch("gemm8_generic");
}

}  // namespace lh
