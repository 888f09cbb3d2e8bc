// f32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32, full f32 products and
// accumulation) with the fused epilogue of the matmul payload
// (emit_mlp_layer, lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:110-156; the f32
// generic-form fixture test/opt/pipeline-check.mlir:27-46).
//
// Fast kernel: A panel [m][k] and B panel [k][n] in LDS in their global orientation.  The MFMA
// takes one f32 per lane and operand; a lane reads 4 consecutive k of its A row with one 16-byte
// LDS read and issues 4 MFMAs, and reads the 4 matching B rows with 4-byte reads that are
// contiguous across the lanes of a half wave.  As in the 16-bit kernel the B panel is the first
// MFMA operand, so a lane's accumulator holds 4 consecutive columns of one row.
#include "gemm_common.h"

namespace lh {

constexpr int kBK32 = 32;

// ---- direct-to-LDS kernel ---------------------------------------------------------------
// Workgroup tile (64 TM) x (64 TN) x 32 with NW = 4 waves (2 x 2) or 8 waves (4 x 2, two per
// SIMD: one wave's waits and barriers are covered by the other's MFMAs).  Both panels go global -> LDS with
// buffer_load_dwordx4 ... lds in their global orientation through a ring of NS stages, NS - 1 of
// them in flight: at f32 rates a k-step lasts about as long as a global load takes, so a
// register-staged double buffer stalls on every step.  A wave-wide load writes 1 KiB
// contiguously, so rows cannot be padded; which 16-byte chunk of a row a lane fetches is
// XOR-swizzled instead (A rows of 128 bytes: chunk ^ ((row / 2) % 8); B rows: chunk ^ 8 for the
// k rows with (k / 4) odd, which are the rows the upper half wave reads).
typedef __attribute__((address_space(3))) void lds32_void_t;

// 16 bytes per lane from a buffer resource over [base, base + 4 GiB) (+ per-lane and scalar byte
// offsets) straight into LDS, 1 KiB per wave.  The buffer form of the LDS-DMA load: with the global
// (flat-encoded) form in flight the compiler must assume LDS operations complete out of order and
// waits for all of a wave's LDS reads before the first use of any; with this form it counts them.
__device__ __forceinline__ void dma16_f32(const float* base, int lane_bytes, int scalar_bytes, uint8_t* lds_wave_base) {
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, 0xffffffff, 0x00020000);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds32_void_t*)lds_wave_base, 16, lane_bytes, scalar_bytes, 0, 0);
}
// The tile's operand panels (64 TM rows of A, K rows of B) are addressed with 32-bit byte offsets.
static inline bool direct32_offsets_fit(const GemmArgs& g) {
  return g.lda < (1ll << 21) && (int64_t)g.K * g.ldb < (1ll << 29);
}

template <int TM, int TN, int NW_>
struct Direct32Ctx {
  static constexpr int NW = NW_;               // waves, as (NW / 2) x 2
  static constexpr int WTM = 4 * TM / NW;      // 32-row sub-tiles per wave (a wave spans 32 TN columns)
  static constexpr int LA = 8 * TM / NW;       // A loads per lane and stage
  static constexpr int LB = 8 * TN / NW;       // B loads per lane and stage
  static_assert(WTM >= 1 && LA >= 1 && LB >= 1, "tile too small for the wave count");
  const float* a_base;  // the tile's first A row and first B column (uniform)
  const float* b_base;
  int a_src[LA];        // the lane's byte offsets within the panels at k = 0
  int b_src[LB];
  int b_step;           // bytes between B stages (32 k rows)
  int wave, h;
  int a_off[WTM], a_swz[WTM];  // byte offset of the lane's A row, its swizzle
  int b_off[TN];               // byte offset of the lane's B column inside a k row (swizzle applied)
};

template <int TM, int TN, int NW>
__device__ __forceinline__ void direct32_issue(const Direct32Ctx<TM, TN, NW>& c, int kt, uint8_t* __restrict__ stage) {
  using C = Direct32Ctx<TM, TN, NW>;
  constexpr int a_bytes = 64 * TM * 128;
#pragma unroll
  for (int i = 0; i < C::LA; ++i) dma16_f32(c.a_base, c.a_src[i], kt * 128, stage + (C::NW * i + c.wave) * 1024);
#pragma unroll
  for (int i = 0; i < C::LB; ++i)
    dma16_f32(c.b_base, c.b_src[i], kt * c.b_step, stage + a_bytes + (C::NW * i + c.wave) * 1024);
}

// One k-step: refill `wr` (if `prefetch`) and multiply the stage in `rd`.
// Separate restrict pointers keep the compiler from making the LDS reads wait for the
// asynchronous writes.
template <int TM, int TN, int NW>
__device__ __forceinline__ void direct32_step(const Direct32Ctx<TM, TN, NW>& c,
                                              f32x16 (&acc)[TN][Direct32Ctx<TM, TN, NW>::WTM],
                                              const uint8_t* __restrict__ rd, uint8_t* __restrict__ wr, int next_kt,
                                              bool prefetch) {
  constexpr int a_bytes = 64 * TM * 128, b_row = 64 * TN * 4, WTM = Direct32Ctx<TM, TN, NW>::WTM;
  constexpr int NKK = 4;  // groups of 8 k per stage
  if (prefetch) direct32_issue(c, next_kt, wr);
  const uint8_t* as = rd;
  const uint8_t* bs = rd + a_bytes;
  // Fragments of k-group kk (k = 8 kk + 4 h + t, t = 0..3) are read while the MFMAs of group
  // kk - 1 run.
  f32x4 fa[2][WTM];
  float fb[2][TN][4];
  auto read = [&](int kk, int buf) {
#pragma unroll
    for (int j = 0; j < WTM; ++j)
      fa[buf][j] = *reinterpret_cast<const f32x4*>(as + c.a_off[j] + (((2 * kk + c.h) ^ c.a_swz[j]) << 4));
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        fb[buf][i][t] = *reinterpret_cast<const float*>(bs + (8 * kk + 4 * c.h + t) * b_row + c.b_off[i]);
  };
  read(0, 0);
#pragma unroll
  for (int q = 0; q < NKK; ++q) {
    const int cur = q & 1;
    if (q + 1 < NKK) read(q + 1, cur ^ 1);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < WTM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cur][i][t], fa[cur][j][t], acc[i][j], 0, 0, 0);
    if (q + 1 < NKK) {
      // keep the reads of the next group ahead of this group's MFMAs in the issue order
      __builtin_amdgcn_sched_group_barrier(0x100, WTM + 4 * TN, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * WTM * TN, 0);
    }
  }
}

template <int N>
__device__ __forceinline__ void direct32_wait_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Source pointers of tile `id` (row-major over the tile grid) and the tile's origin.  EDGE: M and
// N need not be multiples of the tile (N still a multiple of 4): loads of rows / column chunks
// past the end are redirected to the last valid row / chunk (their products land in accumulators
// that are never stored) and the epilogue skips what lies outside the matrix.
template <bool EDGE, int TM, int TN, int NW>
__device__ __forceinline__ void direct32_place(const GemmArgs& g, int id, Direct32Ctx<TM, TN, NW>& c, int& m0, int& n0) {
  using C = Direct32Ctx<TM, TN, NW>;
  constexpr int BM = 64 * TM, BN = 64 * TN;
  const int lane = lane_now();  // the lane's offsets are recomputed per tile rather than kept in registers
  const int tiles_n = (g.N + BN - 1) / BN;
  m0 = (id / tiles_n) * BM;
  n0 = (id % tiles_n) * BN;
  const float* A = reinterpret_cast<const float*>(g.a);
  const float* B = reinterpret_cast<const float*>(g.b);
  const int lda = (int)g.lda, ldb = (int)g.ldb;
  c.a_base = A + (int64_t)m0 * g.lda;
  c.b_base = B + n0;
  c.b_step = 128 * ldb;
  // A: load i of wave w fills rows (NW i + w) 8 .. +8; lane -> row += lane / 8, LDS chunk lane % 8.
#pragma unroll
  for (int i = 0; i < C::LA; ++i) {
    const int row = (C::NW * i + c.wave) * 8 + (lane >> 3);
    const int gc = (lane & 7) ^ ((row >> 1) & 7);
    c.a_src[i] = ((EDGE ? min(row, g.M - 1 - m0) : row) * lda + gc * 4) * 4;
  }
  // B: a k row is 16 TN chunks; load i of wave w fills k rows (NW i + w) (4 / TN) .. ; lane ->
  // row += lane / (16 TN), LDS chunk lane % (16 TN).
#pragma unroll
  for (int i = 0; i < C::LB; ++i) {
    constexpr int chunks = 16 * TN;
    const int k = (C::NW * i + c.wave) * (64 / chunks) + lane / chunks;
    const int gc = (lane % chunks) ^ (8 * ((k >> 2) & 1));
    c.b_src[i] = (k * ldb + (EDGE ? min(gc * 4, g.N - 4 - n0) : gc * 4)) * 4;
  }
}

// Persistent workgroups, each walking the tile list with the grid as stride (tile ids congruent
// modulo 8 stay on one XCD, which is what xcd_remap assumes).  At the end of a tile, once every
// wave has left the ring, the first NS - 1 stages of the workgroup's next tile are issued before
// the epilogue, so their latency and the cold start of the pipeline hide behind its stores.
template <int TM, int TN, int NS, int NW, bool EDGE>
__global__ void __launch_bounds__(NW * 64) gemm32_direct(GemmArgs g) {
  using C = Direct32Ctx<TM, TN, NW>;
  constexpr int WTM = C::WTM;
  constexpr int BM = 64 * TM, BN = 64 * TN;
  constexpr int a_bytes = BM * 128, b_row = BN * 4, stage_bytes = a_bytes + 32 * b_row;
  constexpr int L = C::LA + C::LB;  // loads a lane has in flight per stage
  static_assert(NS >= 3 && NS <= 8, "ring shape");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem32d[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * 32 * WTM, wn0 = (wave & 1) * 32 * TN;
  const int ntiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
  const int r32 = lane & 31, h = lane >> 5;

  C c;
    c.wave = wave;
  c.h = h;
#pragma unroll
  for (int j = 0; j < WTM; ++j) {
    const int row = wm0 + 32 * j + r32;
    c.a_off[j] = row * 128;
    c.a_swz[j] = (row >> 1) & 7;
  }
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int n = wn0 + 32 * i + r32;
    c.b_off[i] = (((n >> 2) ^ (8 * h)) << 4) + (n & 3) * 4;  // rows 8 kk + 4 h + t have (k / 4) % 2 == h
  }

  const int nk = g.K / 32;
  // G k-steps per barrier.  The 64 x 64 tile runs one wave per SIMD: nobody covers its barrier
  // wait and the LDS latency of a step's first fragments, so it takes G > 1 steps behind one
  // barrier (fewer waits, and the next step's first reads are issued under this step's MFMAs).
  // Loads then run NS - G stages ahead.
  constexpr int G = (TM == 1 && TN == 1 && NW == 4) ? (NS == 8 ? 4 : NS == 6 ? 2 : 1) : 1;
  constexpr int kAhead = NS - G;
  static_assert(NS >= 2 * G && L * (NS - 2 * G) < 64, "ring shape");
  int t = blockIdx.x;  // < ntiles: the grid is never larger than the tile list
  int m0, n0;
  direct32_place<EDGE>(g, xcd_remap(t, ntiles), c, m0, n0);
#pragma unroll
  for (int st = 0; st < kAhead; ++st)
    if (st < nk) direct32_issue(c, st, smem32d + st * stage_bytes);
  for (;;) {
    f32x16 acc[TN][WTM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < WTM; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    int kt = 0;
    for (; kt + G <= nk; kt += G) {
      // Stages kt + G .. kt + NS - G - 1 may stay in flight (anything issued after them, such as
      // the previous tile's stores, only makes the wait longer); one asm block per case because a
      // __syncthreads() would add a fence that waits for every outstanding load.
      const int younger = min(nk - G - kt, NS - 2 * G);
      if (younger >= 4) direct32_wait_barrier<L * 4>();
      else if (younger == 3) direct32_wait_barrier<L * 3>();
      else if (younger == 2) direct32_wait_barrier<L * 2>();
      else if (younger == 1) direct32_wait_barrier<L>();
      else direct32_wait_barrier<0>();
#pragma unroll
      for (int sg = 0; sg < G; ++sg) {
        const int nxt = kt + kAhead + sg;
        direct32_step(c, acc, smem32d + ((kt + sg) % NS) * stage_bytes, smem32d + (nxt % NS) * stage_bytes, nxt,
                      nxt < nk);
      }
    }
    for (; kt < nk; ++kt) {  // G > 1: the steps left over at the end of a tile, every stage issued already
      direct32_wait_barrier<0>();
      direct32_step(c, acc, smem32d + (kt % NS) * stage_bytes, smem32d, 0, false);
    }
    const int tn = t + (int)gridDim.x;
    const bool more = tn < ntiles;
    const int em0 = m0, en0 = n0;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the ring
    if (more) {
      direct32_place<EDGE>(g, xcd_remap(tn, ntiles), c, m0, n0);
#pragma unroll
      for (int st = 0; st < kAhead; ++st)
        if (st < nk) direct32_issue(c, st, smem32d + st * stage_bytes);
    }
    const int elane = lane_now();  // as in direct32_place
    const int m_base = em0 + wm0 + (elane & 31);
    const int n_base = en0 + wn0 + 4 * (elane >> 5);
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < WTM; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (!EDGE || (m_base + 32 * j < g.M && n_base + 32 * i + 8 * q < g.N))
            epilogue4<LH_F32>(g, m_base + 32 * j, n_base + 32 * i + 8 * q, acc[i][j][4 * q], acc[i][j][4 * q + 1],
                              acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
    if (!more) break;
    t = tn;
  }
}

template <int TM, int TN, int NS, int NW, bool EDGE>
static int launch_direct32_edge(const GemmArgs& g, hipStream_t s) {
  auto kern = gemm32_direct<TM, TN, NS, NW, EDGE>;
  constexpr size_t lds = (size_t)NS * (64 * TM * 128 + 32 * 64 * TN * 4);
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int ntiles = ((g.M + 64 * TM - 1) / (64 * TM)) * ((g.N + 64 * TN - 1) / (64 * TN));
  const int resident = num_cus() * (int)((160 * 1024) / lds);  // workgroups that fit the CUs' LDS together
  LH_LAUNCH(kern, dim3(ntiles < resident ? ntiles : resident), dim3(NW * 64), lds, s, g);
  return check_launch("gemm32_direct");
}

template <int TM, int TN, int NS, int NW = 4>
static int launch_direct32(const GemmArgs& g, hipStream_t s) {
  if (g.M % (64 * TM) == 0 && g.N % (64 * TN) == 0) return launch_direct32_edge<TM, TN, NS, NW, false>(g, s);
  return launch_direct32_edge<TM, TN, NS, NW, true>(g, s);
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

int gemm32(const GemmArgs& g_in, hipStream_t s) {
  GemmArgs g = g_in;
  const uint32_t tile = g.flags & LH_GEMM_TILE_MASK;
  if (tile == LH_GEMM_TILE_AUTO && g.ldc % 4 == 0 && aligned16(g.out) && (!(g.flags & LH_GEMM_HAS_BIAS) || aligned16(g.bias))) {
    const int rc = untranspose_operands<4>(g, kBK32, 4, s);
    if (rc < 0) return rc;
  }
  const bool trans = g.flags & (LH_GEMM_TRANSPOSE_A | LH_GEMM_TRANSPOSE_B);
  const bool vec_ok = !trans && g.K % kBK32 == 0 && g.lda % 4 == 0 && g.ldb % 4 == 0 && g.ldc % 4 == 0 &&
                      aligned16(g.a) && aligned16(g.b) && aligned16(g.out) &&
                      (!(g.flags & LH_GEMM_HAS_BIAS) || aligned16(g.bias));
  if (tile != LH_GEMM_TILE_AUTO) {
    LH_REQUIRE(vec_ok && g.N % 4 == 0 && direct32_offsets_fit(g),
               "gemm: a tile request on f32 inputs needs untransposed operands, K %% 32 == 0, N %% 4 == 0 and 16-byte "
               "aligned rows (M=%d N=%d K=%d)", g.M, g.N, g.K);
    if (tile == LH_GEMM_TILE_128x128) return launch_direct32<2, 2, 4, 8>(g, s);
    if (tile == LH_GEMM_TILE_128x64) return launch_direct32<2, 1, 4, 8>(g, s);
    if ((int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64) <= 512) return launch_direct32<1, 1, 8>(g, s);
    return launch_direct32<1, 1, 3>(g, s);
  }
  if (!(vec_ok && g.N % 4 == 0) && (int64_t)g.M * g.N * g.K >= (1 << 22)) {
    // not a shape for the direct kernels as it stands: run it on padded copies of the operands
    const int rc = gemm_padded<4>(g, kBK32, 4, s, [&](const GemmArgs& p) { return gemm32(p, s); });
    if (rc <= 0) return rc;
  }
  if (vec_ok && g.N % 4 == 0 && direct32_offsets_fit(g)) {
    // Tiles are counted with edge tiles in full (M, N need not be multiples of a tile).
    const int cus = num_cus();
    const int64_t t128 = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
    if (t128 >= 256) {
      // 128 x 128 or 128 x 64 tiles, one workgroup per CU, or 64 x 64 tiles, three per CU: whichever
      // needs less time in whole rounds of tiles (per flop the narrow tile costs about 8 % more,
      // three resident small ones 3 %: 4096^3 1058 / 1101 / 1079 us; 3072 x 3072 x 1024, 2.25 rounds of
      // wide tiles but exactly 3 of small ones, 206 / 181 / 164 us).
      const int64_t t64n = (int64_t)((g.M + 127) / 128) * ((g.N + 63) / 64);
      const int64_t t64 = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64);
      const double wide = (double)((t128 + cus - 1) / cus), narrow = (double)((t64n + cus - 1) / cus) * 0.54;
      const double small = (double)((t64 + 3 * cus - 1) / (3 * cus)) * 0.7725;
      if (small < wide && small < narrow) return launch_direct32<1, 1, 3>(g, s);
      if (narrow < wide) return launch_direct32<2, 1, 4, 8>(g, s);
      return launch_direct32<2, 2, 4, 8>(g, s);
    }
    // Up to two rounds of one workgroup per CU: a deep ring, four k-steps per barrier (1024^3: 26.7 ->
    // 24.3 us); more tiles: a shallow ring so that three workgroups share a CU.
    if ((int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64) <= 512) return launch_direct32<1, 1, 8>(g, s);
    return launch_direct32<1, 1, 3>(g, s);
  }
  dim3 grid((g.N + 63) / 64, (g.M + 63) / 64);
  LH_LAUNCH(gemm32_generic, grid, dim3(256), 0, s, g);
  return check_launch("gemm32_generic");
}

}  // namespace lh
