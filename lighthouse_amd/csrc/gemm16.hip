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
#include <type_traits>

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
  __device__ static __forceinline__ f32x4 mma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  }
};
template <>
struct Mfma16<LH_F16> {
  __device__ static __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
  }
  __device__ static __forceinline__ f32x4 mma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
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


// ---- direct-to-LDS kernels --------------------------------------------------------------
// Workgroup tile (64 TM) x (128 TN), 8 waves as 2 x 4, (32 TM) x (32 TN) per wave; TM x TN is
// 4 x 2 (256 x 256), 4 x 1 (256 x 128), 2 x 2 (128 x 256) or 2 x 1 (128 x 128).  Both panels go
// global -> LDS with buffer_load_dwordx4 ... lds (no register staging, no LDS store instructions) in
// their GLOBAL orientation.  The k-contiguous A fragment is one 16-byte LDS read; the
// n-contiguous B panel is read with ds_read_b64_tr_b16, which hands each lane 4 k-values of one
// column, i.e. the MFMA operand layout, transposing in the LDS crossbar.
//
// The matrix instruction is v_mfma_f32_16x16x32 (16 rows x 16 columns x 32 k), not 32x32x16: for
// the same products it keeps the matrix cores' clock higher on random operands (a register-only
// loop of either runs at the published peak on zeros, but at 2.02 against 1.74 PFLOP/s on N(0,1)
// data).  A wave's sub-tile is 2 TM fragments of 16 rows by 2 TN fragments of 16 columns per 32 k.
//
// LDS rings: A in 2 stages of 64 k (rows of 128 bytes: every global request is a full 128-byte
// line), B in 4 stages of 32 k.  The main loop advances 32 k per step, each step in two phases:
// the MFMAs of the wave's lower TM row fragments, then of its upper ones, all against the step's
// 2 TN column fragments.  The LDS reads of a phase fetch what the next phase needs (the other
// half of the A fragments; in the second phase also the next step's B fragments, each after the
// last MFMA that uses its predecessor), so reads always overlap MFMAs.  The barrier sits between
// the two phases of a step and the buffers a step has finished reading are refilled right
// behind it (B: 3 stages ahead, A: on odd steps, one 64-k stage ahead).
// The large tiles (and the 128 x 128 tile when workgroups share a compute unit) run a second form
// with one barrier per 64 k, the rings as two halves: direct_step_pair_1b.
//
// A wave-wide load into LDS writes 64 x 16 contiguous LDS bytes, so rows cannot be padded;
// bank conflicts are avoided by XOR-swizzling which 16-byte chunk of a row each lane fetches
// (A: chunk ^ ((row / 2) % 8); B: chunk ^ 4 (k % 4) ^ 2 ((k / 8) % 2)).
template <int TM, int TN>
struct DirectCfg {
  static constexpr int BM = 64 * TM, BN = 128 * TN;
  static constexpr int WTM = 32 * TM, WTN = 32 * TN;      // per-wave sub-tile
  static constexpr int kABytes = BM * 64 * 2;             // one A stage (64 k)
  static constexpr int kBRow = BN * 2;                    // bytes of one k row of a B stage
  static constexpr int kBBytes = 32 * kBRow;              // one B stage (32 k)
  static constexpr int kBtBytes = BN * 64 * 2;            // one stage (64 k) of a transposed B: rows n, like A
  static constexpr int kBBase = 2 * kABytes;
  static constexpr int kRingBytes = kBBase + 4 * kBBytes;
  static constexpr int kStageBytes = 8 * 32 * WTN * 2;    // output staging: 32 rows of each wave's sub-tile
  static constexpr int kStagedStores = 2 * TM * TN;       // 16-byte stores per lane of a staged epilogue
  static constexpr int kLdsBytes = kRingBytes + kStageBytes;
  static constexpr int kBChunks = kBRow / 16;             // 16-byte chunks per B row
  static constexpr int kBRowsPerLoad = 1024 / kBRow;      // k rows one wave-wide load covers
  // Loads a lane has in flight per stage, hence the s_waitcnt immediates of the main loop.
  static constexpr int kWaitEven = TM + 2 * TN;
  static constexpr int kWaitOdd = 2 * TN;
};

typedef __attribute__((address_space(3))) void lds_void_t;
typedef short s16x4 __attribute__((ext_vector_type(4)));

// 16 bytes per lane from a buffer resource (base + per-lane byte offset + scalar byte offset)
// straight into LDS, 1 KiB per wave starting at lds_wave_base.  The buffer form of the LDS-DMA
// load, not the global (flat-encoded) one: with a flat-encoded LDS access in flight the compiler
// must assume that LDS operations complete out of order and turns every s_waitcnt on an LDS read
// into lgkmcnt(0); with the buffer form it counts, so a fragment read issued a few MFMAs ago is
// not waited for behind the ones issued last.
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t rsrc, int lane_bytes, int scalar_bytes,
                                      uint8_t* lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_t*)lds_wave_base, 16, lane_bytes, scalar_bytes, 0, 0);
}
// A resource over [base, base + 4 GiB): raw (unstructured) addressing, offsets in bytes.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t panel_resource(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
}
// The direct kernels address a tile's operand panels with 32-bit byte offsets from the panel's
// first element: 256 rows of A, K rows of B.
static inline bool direct_offsets_fit(const GemmArgs& g) {
  if (g.flags & LH_GEMM_TRANSPOSE_B) return g.lda < (1ll << 22) && g.ldb < (1ll << 22);  // 256 rows of B^T
  return g.lda < (1ll << 22) && (int64_t)g.K * g.ldb < (1ll << 30);
}

template <int TM, int TN>
struct DirectCtx {
  const uint16_t* a_base;     // the tile's A row panel and B column panel (uniform; the buffer
  const uint16_t* b_base;     // resources are made from them at each load: four scalar moves)
  int a_src[TM];              // lane's byte offset in the A panel for load i at k = 0
  int b_src[TN];
  int b_step;                 // bytes between B stages (32 k rows)
  // Fragment reads.  A: the lane's first row (wm0 + lane % 16) of a stage, its 16-byte chunk for the
  // first / second 32 k of the stage's 64 (fragment jj, 16 rows further on, adds 2048 jj: the
  // swizzle term (row / 2) % 8 does not change with 16 rows).
  int a_rd[2];
  int wave, b_off, b_chunk, b_swz;
  // B stored transposed ([N, K], k contiguous): its panel is laid out, loaded and read like A's
  int bt_src[2 * TN];         // lane's byte offset in the B^T panel for load i at k = 0
  int bt_rd[2];               // like a_rd, for row wn0 + lane % 16 of a B^T stage
};

// Fragments in registers: the A fragments of the lower (a[0]) and upper (a[1]) half of the wave's
// rows, TM of 16 rows each, and the step's 2 TN B fragments of 16 columns.
template <int TM, int TN>
struct DirectFrags {
  u32x4 a[2][TM];
  u32x4 b[2 * TN];
};

// A stage `sa` (k = 64 sa .. +64): TM loads per lane.
template <int TM, int TN>
__device__ __forceinline__ void direct_load_a(const DirectCtx<TM, TN>& c, int sa, uint8_t* __restrict__ abuf) {
  const __amdgpu_buffer_rsrc_t rsrc = panel_resource(c.a_base);
#pragma unroll
  for (int i = 0; i < TM; ++i) dma16(rsrc, c.a_src[i], sa * 128, abuf + (8 * i + c.wave) * 1024);
}
// B stage `sb` (k = 32 sb .. +32): TN loads per lane.  BT (B stored [N, K]): stage sb is k = 64 sb .. +64
// of the panel's rows, 2 TN loads per lane.
template <int TM, int TN, bool BT = false>
__device__ __forceinline__ void direct_load_b(const DirectCtx<TM, TN>& c, int sb, uint8_t* __restrict__ bbuf) {
  const __amdgpu_buffer_rsrc_t rsrc = panel_resource(c.b_base);
  if constexpr (BT) {
#pragma unroll
    for (int i = 0; i < 2 * TN; ++i) dma16(rsrc, c.bt_src[i], sb * 128, bbuf + (8 * i + c.wave) * 1024);
  } else {
#pragma unroll
    for (int i = 0; i < TN; ++i) dma16(rsrc, c.b_src[i], sb * c.b_step, bbuf + (8 * i + c.wave) * 1024);
  }
}

// A fragments of one half of the wave's rows (HALF 0: 16-row fragments 0 .. TM-1, 1: TM .. 2 TM-1)
// for the 32 k `kc` (0 / 1) of the 64-k stage `as`.
template <int TM, int TN, int HALF>
__device__ __forceinline__ void direct_read_a(const DirectCtx<TM, TN>& c, const uint8_t* __restrict__ as, int kc,
                                              u32x4 (&a)[TM]) {
#pragma unroll
  for (int j = 0; j < TM; ++j) a[j] = *reinterpret_cast<const u32x4*>(as + c.a_rd[kc] + 2048 * (HALF * TM + j));
}
// B fragment i (16 columns) of a 32-k step: from the 32-k stage `bs` of an n-contiguous B through two
// transposing reads, or (BT) from the 32 k `kc` of the 64-k stage `bs` of a transposed B like an A fragment.
template <int TM, int TN, bool BT>
__device__ __forceinline__ u32x4 direct_read_b(const DirectCtx<TM, TN>& c, const uint8_t* __restrict__ bs, int kc,
                                               int i) {
  if constexpr (BT) {
    return *reinterpret_cast<const u32x4*>(bs + c.bt_rd[kc] + 2048 * i);
  } else {
    constexpr int row = DirectCfg<TM, TN>::kBRow;
    const int p = (c.b_chunk + 2 * i) ^ c.b_swz;
    const uint8_t* p0 = bs + c.b_off + p * 16;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p0);
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p0 + 4 * row));
    u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return u32x4{l2[0], l2[1], h2[0], h2[1]};
  }
}

// Scheduling hint for one phase: spread its NR LDS reads evenly between its NM MFMAs.
template <int I, int NM, int NR>
__device__ __forceinline__ void direct_interleave_step() {
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                // MFMA
  __builtin_amdgcn_sched_group_barrier(0x100, (I + 1) * NR / NM - I * NR / NM, 0);  // DS reads
  if constexpr (I + 1 < NM) direct_interleave_step<I + 1, NM, NR>();
}

// First phase of a step: the MFMAs of the lower row fragments (f.a[0]) against the step's B
// fragments, under the reads of the same step's upper row fragments (32 k `kc` of stage `as`).
template <int DT, int TM, int TN>
__device__ __forceinline__ void direct_phase_lo(const DirectCtx<TM, TN>& c, f32x4 (&acc)[2 * TN][2 * TM],
                                                DirectFrags<TM, TN>& f, const uint8_t* __restrict__ as, int kc) {
  direct_read_a<TM, TN, 1>(c, as, kc, f.a[1]);
#pragma unroll
  for (int i = 0; i < 2 * TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = Mfma16<DT>::mma16(f.b[i], f.a[0][j], acc[i][j]);
  direct_interleave_step<0, 2 * TN * TM, TM>();
}
// Second phase: the MFMAs of the upper row fragments (f.a[1]) under the reads of the NEXT step's
// lower row fragments (32 k `kc_n` of A stage `as_n`) and B fragments (stage `bs_n`; BT: its 32 k
// `kc_n`), each B fragment requested behind the last MFMA that uses the one it replaces.
// LOAD false: the tile's last step, nothing left to read.
template <int DT, int TM, int TN, bool BT, bool LOAD = true>
__device__ __forceinline__ void direct_phase_hi(const DirectCtx<TM, TN>& c, f32x4 (&acc)[2 * TN][2 * TM],
                                                DirectFrags<TM, TN>& f, const uint8_t* __restrict__ as_n,
                                                const uint8_t* __restrict__ bs_n, int kc_n) {
  if constexpr (LOAD) direct_read_a<TM, TN, 0>(c, as_n, kc_n, f.a[0]);
  u32x4 bn[2 * TN];
#pragma unroll
  for (int i = 0; i < 2 * TN; ++i) {
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][TM + j] = Mfma16<DT>::mma16(f.b[i], f.a[1][j], acc[i][TM + j]);
    if constexpr (LOAD) bn[i] = direct_read_b<TM, TN, BT>(c, bs_n, kc_n, i);
  }
  if constexpr (LOAD) {
#pragma unroll
    for (int i = 0; i < 2 * TN; ++i) f.b[i] = bn[i];
    direct_interleave_step<0, 2 * TN * TM, TM + (BT ? 2 : 4) * TN>();
  }
}
// Wait until at most N of this wave's loads are still in flight and all its LDS reads have
// returned, then barrier.  One asm block: a __syncthreads() would add a release fence, i.e. a
// wait for ALL outstanding loads, and drain the rings.
template <int N>
__device__ __forceinline__ void direct_wait_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}


// Steps kt (even) and kt + 1 of the main loop; both have a successor step.  On entry f holds the
// lower row fragments and the B fragments of step kt.  a_cur = A stage kt / 2, a_nxt = the next A
// stage, b1 / b2 = B stages kt + 1, kt + 2.  The refill pointers alias a_cur and B stages kt and
// kt + 1: every read of a buffer precedes the barrier after which it is refilled.  They are
// separate restrict parameters so that the compiler does not make LDS reads wait for the
// asynchronous writes.
//
// In-flight loads, oldest first, when a barrier is reached (steady state):
//   even step: [A(kt/2) B(kt+1)] [B(kt+2)] [A(kt/2+1) B(kt+3)]  -> B(kt+1) needed: TM + 2 TN may remain
//   odd step : [B(kt+1)] [A((kt+1)/2) B(kt+2)] [B(kt+3)]        -> A needed: 2 TN may remain
// Near the end loads are no longer issued and the waits become full waits.
template <int DT, int TM, int TN>
__device__ __forceinline__ void direct_step_pair(const DirectCtx<TM, TN>& c, f32x4 (&acc)[2 * TN][2 * TM],
                                                 DirectFrags<TM, TN>& f, const uint8_t* __restrict__ a_cur,
                                                 const uint8_t* __restrict__ a_nxt, const uint8_t* __restrict__ b1,
                                                 const uint8_t* __restrict__ b2, uint8_t* __restrict__ a_refill,
                                                 uint8_t* __restrict__ b_refill0, uint8_t* __restrict__ b_refill1,
                                                 int kt, int nk) {
  using Cfg = DirectCfg<TM, TN>;
  const bool steady = kt + 6 < nk;  // all loads of both steps are real
  // ---- even step kt
  direct_phase_lo<DT>(c, acc, f, a_cur, 0);
  if (steady) direct_wait_barrier<Cfg::kWaitEven>();
  else direct_wait_barrier<0>();
  if (kt + 4 < nk) direct_load_b(c, kt + 4, b_refill0);
  direct_phase_hi<DT, TM, TN, false>(c, acc, f, a_cur, b1, 1);
  // ---- odd step kt + 1
  direct_phase_lo<DT>(c, acc, f, a_cur, 1);
  if (steady) direct_wait_barrier<Cfg::kWaitOdd>();
  else direct_wait_barrier<0>();
  if (kt + 4 < nk) direct_load_a(c, kt / 2 + 2, a_refill);
  if (kt + 5 < nk) direct_load_b(c, kt + 5, b_refill1);
  direct_phase_hi<DT, TM, TN, false>(c, acc, f, a_nxt, b2, 0);
}

// Source pointers of tile `id` (its position in the XCD-grouped order) and the tile's origin.
// EDGE: M and N need not be multiples of the tile (N still a multiple of 8, K of 64): loads of
// rows / column chunks past the end are redirected to the last valid row / chunk (their products
// land in accumulators that are never stored) and the epilogue skips what lies outside the matrix.
template <int TM, int TN, bool EDGE, bool BT = false>
__device__ __forceinline__ void direct_place(const GemmArgs& g, int id, DirectCtx<TM, TN>& c, int& m0, int& n0) {
  using Cfg = DirectCfg<TM, TN>;
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  const int lane = lane_now();
  const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
  // Tiles are walked in groups of GROUP_M tile rows: 1024 rows of A.  For the 128-row tiles that
  // is 8 up to K = 1536 (1-3 % faster than 4 there; 0.3-1.4 % slower from K = 3072 on).
  const int GROUP_M = (BM == 128 && g.K <= 1536) ? 8 : 4;
  const int group_size = GROUP_M * tiles_n;
  const int first_m = (id / group_size) * GROUP_M;
  const int gm = min(tiles_m - first_m, GROUP_M);
  m0 = (first_m + (id % group_size) % gm) * BM;
  n0 = ((id % group_size) / gm) * BN;
  const uint16_t* A = reinterpret_cast<const uint16_t*>(g.a);
  const uint16_t* B = reinterpret_cast<const uint16_t*>(g.b);
  const int lda = (int)g.lda, ldb = (int)g.ldb;
  c.a_base = A + (int64_t)m0 * g.lda;
  c.b_base = BT ? B + (int64_t)n0 * g.ldb : B + n0;
  c.b_step = 64 * ldb;
  // A: load i of wave w fills rows (8 i + w) 8 .. +8 (1024 bytes); lane -> row += lane / 8, LDS
  // chunk p = lane % 8 holds global chunk p ^ ((row / 2) % 8).
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int ar = (8 * i + c.wave) * 8 + (lane >> 3);
    const int ac = (lane & 7) ^ ((ar >> 1) & 7);
    const int arow = EDGE ? min(ar, g.M - 1 - m0) : ar;  // row within the panel
    c.a_src[i] = (arow * lda + ac * 8) * 2;
  }
  // B: load i of wave w fills k rows (8 i + w) R .. +R with R = 1024 / row bytes; lane ->
  // row += lane / chunks-per-row, LDS chunk p holds global chunk p ^ 4 (k % 4) ^ 2 ((k / 8) % 2): the
  // four k rows a 16-lane group reads at once land in different banks, and so do the rows (8 apart)
  // of the group next to it.
  if constexpr (BT) {
    // B^T: exactly A's scheme on the panel's BN rows (row n of B^T = column n of B)
#pragma unroll
    for (int i = 0; i < 2 * TN; ++i) {
      const int br = (8 * i + c.wave) * 8 + (lane >> 3);
      const int bc = (lane & 7) ^ ((br >> 1) & 7);
      const int brow = EDGE ? min(br, g.N - 1 - n0) : br;
      c.bt_src[i] = (brow * ldb + bc * 8) * 2;
    }
  } else {
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      const int bk = (8 * i + c.wave) * Cfg::kBRowsPerLoad + lane / Cfg::kBChunks;
      const int bc = (lane % Cfg::kBChunks) ^ (4 * (bk & 3)) ^ (2 * ((bk >> 3) & 1));
      const int bcol = EDGE ? min(bc * 8, g.N - 8 - n0) : bc * 8;  // column within the panel
      c.b_src[i] = (bk * ldb + bcol) * 2;
    }
  }
}

// The same two steps with ONE barrier, in the middle of the odd step: the rings work as two halves
// of 64 k.  At the barrier every read of this pair's stages has returned and the next pair's
// stages (issued at the previous barrier, 64 k ago) are awaited in full; the pair after that is
// then requested into this pair's buffers.  BT: b1 is the pair's one 64-k stage of B^T, b2 the next.
template <int DT, int TM, int TN, bool BT = false>
__device__ __forceinline__ void direct_step_pair_1b(const DirectCtx<TM, TN>& c, f32x4 (&acc)[2 * TN][2 * TM],
                                                    DirectFrags<TM, TN>& f, const uint8_t* __restrict__ a_cur,
                                                    const uint8_t* __restrict__ a_nxt, const uint8_t* __restrict__ b1,
                                                    const uint8_t* __restrict__ b2, uint8_t* __restrict__ a_refill,
                                                    uint8_t* __restrict__ b_refill0, uint8_t* __restrict__ b_refill1,
                                                    int kt, int nk, bool stores_behind) {
  using Cfg = DirectCfg<TM, TN>;
  direct_phase_lo<DT>(c, acc, f, a_cur, 0);
  direct_phase_hi<DT, TM, TN, BT>(c, acc, f, a_cur, b1, 1);
  direct_phase_lo<DT>(c, acc, f, a_cur, 1);
  // At a tile's first barrier the only operations in flight are the previous tile's stores (the
  // tile's first loads, older than they, were awaited when the main loop began): they may stay.
  // Matters for the 128 x 128 tile, whose first 64 k pass in 0.5 us (M = 8192, N = 2304, K = 768:
  // 35.15 -> 34.9 us); the large tiles' stores have long completed by then.
  if (TM * TN == 2 && stores_behind && kt == 0) direct_wait_barrier<Cfg::kStagedStores>();
  else direct_wait_barrier<0>();
  if (kt + 4 < nk) {
    direct_load_a(c, kt / 2 + 2, a_refill);
    if constexpr (BT) {
      direct_load_b<TM, TN, true>(c, kt / 2 + 2, b_refill0);
    } else {
      direct_load_b(c, kt + 4, b_refill0);
      direct_load_b(c, kt + 5, b_refill1);
    }
  }
  direct_phase_hi<DT, TM, TN, BT>(c, acc, f, a_nxt, b2, 0);
}

// First loads of a tile: A stages 0, 1 and B stages 0 .. 3 (nk = K / 32 >= 2); BT: both 64-k stages of B^T.
template <int TM, int TN, bool BT = false>
__device__ __forceinline__ void direct_prologue(const DirectCtx<TM, TN>& c, int nk, uint8_t* __restrict__ ring) {
  using Cfg = DirectCfg<TM, TN>;
  direct_load_a(c, 0, ring);
  if (nk > 2) direct_load_a(c, 1, ring + Cfg::kABytes);
  if constexpr (BT) {
    direct_load_b<TM, TN, true>(c, 0, ring + Cfg::kBBase);
    if (nk > 2) direct_load_b<TM, TN, true>(c, 1, ring + Cfg::kBBase + Cfg::kBtBytes);
  } else {
#pragma unroll
    for (int st = 0; st < 4; ++st)
      if (st < nk) direct_load_b(c, st, ring + Cfg::kBBase + st * Cfg::kBBytes);
  }
}

// The lane's 16-bit bias values for a staged epilogue, columns n_base + 16 i .. +4, as packed
// pairs; all loads are issued back to back.  (An f32 bias is read by the epilogue itself.)
template <int TN, bool EDGE>
__device__ __forceinline__ void direct_load_bias(const GemmArgs& g, int n_base, u32x2 (&bias)[2 * TN]) {
#pragma unroll
  for (int i = 0; i < 2 * TN; ++i) bias[i] = u32x2{0u, 0u};
  if (!(g.flags & LH_GEMM_HAS_BIAS) || g.bias_dt == LH_F32) return;
#pragma unroll
  for (int i = 0; i < 2 * TN; ++i) {
    const int n = n_base + 16 * i;
    bias[i] = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g.bias) + (EDGE ? min(n, g.N - 4) : n));
  }
}

// Main loop of one tile, whose first loads have been issued.
// `stores_behind`: the previous tile's staged epilogue issued exactly Cfg::kStagedStores stores
// per lane AFTER this tile's first loads; vector memory operations complete in issue order, so
// those stores may stay in flight.
// `staged`: the epilogue will want `bias` (for columns from n_base); it is loaded ahead of the
// last two steps, whose full wait covers it.
template <int DT, int TM, int TN, bool EDGE, bool BT = false>
__device__ __forceinline__ void direct_mainloop(const GemmArgs& g, const DirectCtx<TM, TN>& c,
                                                f32x4 (&acc)[2 * TN][2 * TM], uint8_t* smem_d, int nk,
                                                bool stores_behind, bool staged, int n_base, u32x2 (&bias)[2 * TN]) {
  using Cfg = DirectCfg<TM, TN>;
  // One barrier per 64 k (loads one 64-k half of the rings ahead) or two (B three 32-k stages
  // ahead).  One is 1-3 % faster for every tile with a 256 side (4096^3 109.8 -> 108.3 us) and, when
  // two workgroups share a compute unit, 2-7 % for the 128 x 128 tile (M = 8192, N = 768, K = 3072:
  // 46.0 -> 42.9 us); a lone 128 x 128 workgroup has nobody to cover the shorter look-ahead
  // (2048^3 22.7 -> 24.2 us) and keeps two.
  // A transposed B lives in the rings as two 64-k stages like A and always takes the one-barrier form.
  const bool one_barrier = BT || TM * TN > 2 || g.one_barrier;
  uint8_t* const abuf = smem_d;
  uint8_t* const bbuf = smem_d + Cfg::kBBase;
  if (stores_behind) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(Cfg::kStagedStores) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  DirectFrags<TM, TN> f;
  direct_read_a<TM, TN, 0>(c, abuf, 0, f.a[0]);
#pragma unroll
  for (int i = 0; i < 2 * TN; ++i) f.b[i] = direct_read_b<TM, TN, BT>(c, bbuf, 0, i);
  int kt = 0;
  auto pair = [&](auto one) {
    uint8_t* a_cur = abuf + ((kt >> 1) & 1) * Cfg::kABytes;
    uint8_t* a_nxt = abuf + (((kt >> 1) + 1) & 1) * Cfg::kABytes;
    if constexpr (BT) {
      uint8_t* b_cur = bbuf + ((kt >> 1) & 1) * Cfg::kBtBytes;
      uint8_t* b_nxt = bbuf + (((kt >> 1) + 1) & 1) * Cfg::kBtBytes;
      direct_step_pair_1b<DT, TM, TN, true>(c, acc, f, a_cur, a_nxt, b_cur, b_nxt, a_cur, b_cur, b_cur, kt, nk,
                                            stores_behind);
    } else {
      uint8_t* b0 = bbuf + (kt & 3) * Cfg::kBBytes;
      uint8_t* b1 = bbuf + ((kt + 1) & 3) * Cfg::kBBytes;
      uint8_t* b2 = bbuf + ((kt + 2) & 3) * Cfg::kBBytes;
      if constexpr (decltype(one)::value) direct_step_pair_1b<DT>(c, acc, f, a_cur, a_nxt, b1, b2, a_cur, b0, b1, kt, nk, stores_behind);
      else direct_step_pair<DT>(c, acc, f, a_cur, a_nxt, b1, b2, a_cur, b0, b1, kt, nk);
    }
  };
  if constexpr (BT || TM * TN > 2) {
    for (; kt + 2 < nk; kt += 2) pair(std::true_type{});
  } else if (one_barrier) {
    for (; kt + 2 < nk; kt += 2) pair(std::true_type{});
  } else {
    for (; kt + 2 < nk; kt += 2) pair(std::false_type{});
  }
  {
    // Last two steps: nothing left to load; stage nk - 1 of B must have landed.
    const uint8_t* a_cur = abuf + ((kt >> 1) & 1) * Cfg::kABytes;
    const uint8_t* b1 = BT ? bbuf + ((kt >> 1) & 1) * Cfg::kBtBytes : bbuf + ((kt + 1) & 3) * Cfg::kBBytes;
    if (staged) direct_load_bias<TN, EDGE>(g, n_base, bias);
    direct_phase_lo<DT>(c, acc, f, a_cur, 0);
    if (!one_barrier) direct_wait_barrier<0>();  // (one barrier per pair: awaited at the pair before)
    direct_phase_hi<DT, TM, TN, BT>(c, acc, f, a_cur, b1, 1);
    direct_phase_lo<DT>(c, acc, f, a_cur, 1);
    direct_phase_hi<DT, TM, TN, BT, false>(c, acc, f, a_cur, b1, 0);
  }
}

// End of a tile: once every wave has left the rings, the first loads of the workgroup's NEXT tile
// are issued into them (their latency and the cold start of the pipeline hide behind this tile's
// stores), then the accumulators are written out.  16-bit outputs are staged through `stage`, an
// LDS area of its own (32 rows of the wave's sub-tile at a time, 16-byte chunk ^ ((row / 2) % chunks)
// against bank conflicts), and leave as full row segments of 16 bytes per lane.  `ring` and
// `stage` are separate restrict parameters so that the staging traffic does not wait for the
// asynchronous ring writes.
template <int DT, int TM, int TN, bool EDGE, bool HAS_NEXT, bool BT = false>
__device__ __forceinline__ void direct_finish(const GemmArgs& g, const DirectCtx<TM, TN>& next, int nk,
                                              uint8_t* __restrict__ ring, uint8_t* __restrict__ stage,
                                              const f32x4 (&acc)[2 * TN][2 * TM], const u32x2 (&bias)[2 * TN], int m0,
                                              int n0, int wm0, int wn0) {
  using Cfg = DirectCfg<TM, TN>;
  constexpr int WTN = Cfg::WTN;
  // The lane-dependent addresses below do not change from tile to tile; lane_now() has them
  // recomputed here instead of kept in registers (and spilled) across the main loop.
  // Accumulator acc[i][j][e] of a lane: row wm0 + 16 j + lane % 16, column wn0 + 16 i + 4 (lane / 16) + e.
  const int lane = lane_now();
  const int l16 = lane & 15, g4 = lane >> 4;
  const int n_base = n0 + wn0 + 4 * g4;
  if (g.out_dt != LH_F32 && !(g.flags & LH_GEMM_ACCUMULATE_C)) {
    // The bias values (loaded by the main loop, whose last wait covered them) are pinned down here:
    // a wait for them placed after the ring loads below would wait for those loads as well.
#pragma unroll
    for (int i = 0; i < 2 * TN; ++i)
#pragma unroll
      for (int e = 0; e < 2; ++e) asm volatile("" ::"v"(bias[i][e]));
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave is done with the rings
    if constexpr (HAS_NEXT) direct_prologue<TM, TN, BT>(next, nk, ring);
    constexpr int RB = WTN * 2;                // bytes of a staged row
    constexpr int chunks = RB / 16;            // 16-byte chunks per staged row
    constexpr int rows_per_pass = 64 / chunks;
    // With a next tile loading into the rings, 32 rows at a time go through the wave's slice of
    // `stage`; the last tile of a workgroup stages its whole sub-tile in the idle rings at once.
    constexpr int JB = HAS_NEXT ? 1 : TM;
    uint8_t* cw = HAS_NEXT ? stage + next.wave * (32 * RB) : ring + next.wave * (TM * 32 * RB);
    uint16_t* outp = reinterpret_cast<uint16_t*>(g.out);
    // One variant of the bias / activation code per tile, chosen here, not per element group.
    epi_dispatch(g, [&](auto variant) {
      using E = decltype(variant);
      // The bias of fragment i's 4 columns, converted where it is used (a converted copy of all of
      // them would be 8 TN more live registers in an epilogue that has none to spare).
      auto bias_of = [&](int i) -> f32x4 {
        if constexpr (!E::kAny && !E::kBias) return f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        const int n = n_base + 16 * i;
        return (g.bias_dt == LH_F32)
                   ? bias4<DT>(g, EDGE ? min(n, g.N - 4) : n)  // the bias row ends at N
                   : f32x4{unpack_lo<DT>(bias[i][0]), unpack_hi<DT>(bias[i][0]), unpack_lo<DT>(bias[i][1]),
                           unpack_hi<DT>(bias[i][1])};
      };
#pragma unroll
      for (int j0 = 0; j0 < TM; j0 += JB) {
#pragma unroll
        for (int jj = 0; jj < 2 * JB; ++jj)
#pragma unroll
          for (int i = 0; i < 2 * TN; ++i) {
            const int j = 2 * j0 + jj;           // 16-row fragment; staged row 16 jj + l16
            const u32x2 w = epi_pack4<DT, E>(g, bias_of(i), acc[i][j]);
            const int row = 16 * jj + l16;
            *reinterpret_cast<u32x2*>(cw + row * RB + (((2 * i + (g4 >> 1)) ^ ((row >> 1) & (chunks - 1))) << 4) +
                                      8 * (g4 & 1)) = w;
          }
        // Cfg::kStagedStores stores per lane in all; the main loop's first wait counts on it.
#pragma unroll
        for (int t = 0; t < JB * 32 / rows_per_pass; ++t) {
          const int row = rows_per_pass * t + lane / chunks, ch = lane % chunks;
          u32x4 w = *reinterpret_cast<const u32x4*>(cw + row * RB + ((ch ^ ((row >> 1) & (chunks - 1))) << 4));
          const int m = m0 + wm0 + 32 * j0 + row;
          if (!EDGE || (m < g.M && n0 + wn0 + ch * 8 < g.N))
            *reinterpret_cast<u32x4*>(outp + (int64_t)m * g.ldc + n0 + wn0 + ch * 8) = w;
        }
      }
    });
    return;
  }
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  if constexpr (HAS_NEXT) direct_prologue<TM, TN, BT>(next, nk, ring);
  {
    // f32 output (with or without an accumulator input), or a 16-bit output with an accumulator
    // input: the scaled f32 accumulators of a block of 32 rows x 16 NI columns go through the wave's
    // slice of `stage` so that the accumulator input is read and the result written as whole row
    // segments (4 elements per lane, 64 or 128 bytes per row) instead of pieces of 64 different
    // rows.  Order of operations as in epilogue4 (one rounding, after the sum).
    constexpr int NI = TN;                     // 16-column fragments per staged block (2 blocks per wave)
    constexpr int RB = NI * 64;                // bytes of a staged row
    constexpr int chunks = RB / 16;
    constexpr int rows_per_pass = 64 / chunks;
    uint8_t* cw = stage + next.wave * (32 * RB);
    const int ch = lane % chunks, row0 = lane / chunks;
    // The output type, the accumulator input and the bias / activation variant are fixed per tile:
    // out32 / has_c as compile-time booleans, the variant from epi_dispatch_linear (an activation
    // takes the variant that tests the flags).
    auto body = [&](auto variant, auto out32_c, auto has_c_c) {
      using E = decltype(variant);
      constexpr bool out32 = decltype(out32_c)::value, has_c = decltype(has_c_c)::value;
      // The 128 x 128 tile requests its whole accumulator input up front (8 row segments per lane, all
      // in flight at once) instead of block by block between the stores of the blocks before, which the
      // loads cannot pass (input and output may be the same buffer): one exposed memory latency per
      // tile instead of eight.  The larger tiles have no registers for that.
      constexpr bool kPreloadC = TM * TN == 2 && has_c;
      constexpr int NPASS = 32 / rows_per_pass;
      auto load_c = [&](int64_t off) -> f32x4 {
        if constexpr (out32) {
          return *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(g.c) + off);
        } else {
          const u32x2 cc = *reinterpret_cast<const u32x2*>(reinterpret_cast<const uint16_t*>(g.c) + off);
          return f32x4{unpack_lo<DT>(cc[0]), unpack_hi<DT>(cc[0]), unpack_lo<DT>(cc[1]), unpack_hi<DT>(cc[1])};
        }
      };
      f32x4 cin[kPreloadC ? 2 * TM * NPASS : 1];
      if constexpr (kPreloadC) {
#pragma unroll
        for (int ib = 0; ib < 2; ++ib)
#pragma unroll
          for (int j32 = 0; j32 < TM; ++j32)
#pragma unroll
            for (int t = 0; t < NPASS; ++t) {
              const int n = n0 + wn0 + 16 * NI * ib + 4 * ch;
              const int m = m0 + wm0 + 32 * j32 + rows_per_pass * t + row0;
              f32x4 c4 = {0.0f, 0.0f, 0.0f, 0.0f};
              if (!EDGE || (n < g.N && m < g.M)) c4 = load_c((int64_t)m * g.ldc + n);
              cin[(ib * TM + j32) * NPASS + t] = c4;
            }
      }
#pragma unroll
      for (int ib = 0; ib < 2; ++ib) {
        const int n = n0 + wn0 + 16 * NI * ib + 4 * ch;  // the lane's 4 output columns
        const bool n_ok = !EDGE || n < g.N;
        f32x4 b4 = {0.0f, 0.0f, 0.0f, 0.0f};
        if (epi_has_bias<E>(g)) b4 = bias4<DT>(g, EDGE ? min(n, g.N - 4) : n);
#pragma unroll
        for (int j32 = 0; j32 < TM; ++j32) {
#pragma unroll
          for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int ii = 0; ii < NI; ++ii) {
              const f32x4& a4 = acc[NI * ib + ii][2 * j32 + jj];
              f32x4 w = a4;
              if constexpr (E::kAlpha) w = f32x4{a4[0] * g.alpha, a4[1] * g.alpha, a4[2] * g.alpha, a4[3] * g.alpha};
              const int row = 16 * jj + l16;
              *reinterpret_cast<f32x4*>(cw + row * RB + (((4 * ii + g4) ^ ((row >> 1) & (chunks - 1))) << 4)) = w;
            }
#pragma unroll
          for (int t = 0; t < 32 / rows_per_pass; ++t) {
            const int row = rows_per_pass * t + row0;
            f32x4 v = *reinterpret_cast<const f32x4*>(cw + row * RB + ((ch ^ ((row >> 1) & (chunks - 1))) << 4));
            const int m = m0 + wm0 + 32 * j32 + row;
            if (EDGE && !(n_ok && m < g.M)) continue;
            const int64_t off = (int64_t)m * g.ldc + n;
            if constexpr (has_c) {
              f32x4 c4;
              if constexpr (kPreloadC) c4 = cin[(ib * TM + j32) * NPASS + t];
              else c4 = load_c(off);
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] += c4[e];
            }
            if constexpr (E::kAny) {
              if (g.flags & LH_GEMM_HAS_BIAS) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += b4[e];
              }
              if (g.flags & LH_GEMM_HAS_GELU) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
              }
              if (g.flags & LH_GEMM_HAS_RELU) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = relu_nan(v[e]);
              }
            } else if constexpr (E::kBias) {
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] += b4[e];
            }
            if constexpr (out32)
              *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(g.out) + off) = v;
            else
              *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(g.out) + off) =
                  u32x2{pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
          }
        }
      }
    };
    const bool out32 = g.out_dt == LH_F32;
    const bool has_c = (g.flags & LH_GEMM_ACCUMULATE_C) != 0;
    epi_dispatch_linear(g, [&](auto variant) {
      if (out32 && has_c) body(variant, std::true_type{}, std::true_type{});
      else if (out32) body(variant, std::true_type{}, std::false_type{});
      else body(variant, std::false_type{}, std::true_type{});  // a 16-bit output comes here only with an accumulator input
    });
  }
}

// Persistent workgroups: one (two for the 128 x 128 tile, whose LDS is 80 KiB) per CU, each
// walking the tile list with the grid as stride.  Tile ids congruent modulo 8 stay on one XCD,
// which is what xcd_remap assumes.  Launching one workgroup per tile instead costs a
// workgroup launch plus a cold prologue per tile, about a third of a K = 768 tile's time.
// SPLITK: the tile list is g.splits copies of the problem's tiles, copy sp working on its own K
// columns of A / rows of B and its own block of the (f32) output; a second kernel adds the blocks.
// For problems with few tiles and a long K (decode shapes), where the tile count cannot fill the CUs.
// BT: B is stored transposed ([N, K] with row stride ldb, the layout of a torch Linear weight); its
// panel goes through the rings like A's and no transposed copy is made.
template <int DT, int TM, int TN, bool EDGE, bool SPLITK = false, bool BT = false>
__global__ void __launch_bounds__(512) gemm16_direct(GemmArgs g) {
  using Cfg = DirectCfg<TM, TN>;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_d[];
  const int tiles1 = ((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
  const int ntiles = SPLITK ? tiles1 * g.splits : tiles1;
  GemmArgs g_cur = g, g_nxt = g;  // (SPLITK) the problem copy that the current / next tile belongs to
  auto select = [&](int t, GemmArgs& ga) -> int {  // -> the tile's id within its copy
    if constexpr (SPLITK) {
      const int sp = t / tiles1;
      ga.a = reinterpret_cast<const uint16_t*>(g.a) + (int64_t)sp * g.K;
      ga.b = reinterpret_cast<const uint16_t*>(g.b) + (BT ? (int64_t)sp * g.K : (int64_t)sp * g.K * g.ldb);
      ga.out = reinterpret_cast<float*>(g.out) + (int64_t)sp * g.M * g.ldc;
      ga.c = ga.out;
      return t - sp * tiles1;
    }
    return t;
  };
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int WN = 4;
  const int wm0 = (wave / WN) * Cfg::WTM, wn0 = (wave % WN) * Cfg::WTN;
  const int l16 = lane & 15, g4 = lane >> 4;

  DirectCtx<TM, TN> c;
  c.wave = wave;
  // A fragment jj (second MFMA operand): row wm0 + 16 jj + l16, logical 16-byte chunk 4 kc + g4 of
  // the row's 8 (physical chunk: ^ ((row / 2) % 8); 4 kc only flips bit 2).
  {
    const int r = wm0 + l16;
    c.a_rd[0] = r * 128 + ((g4 ^ ((r >> 1) & 7)) << 4);
    c.a_rd[1] = c.a_rd[0] ^ 64;
  }
  // B fragment i (first MFMA operand) through the transposing read: the 16 lanes of group g4
  // address k rows 8 g4 + l16 / 4 (+4 for the second read), columns wn0 + 16 i + 4 (l16 % 4) .. +4,
  // and each receives the 4 k-values of column wn0 + 16 i + l16.
  {
    const int krow = 8 * g4 + (l16 >> 2);
    const int col = wn0 + 4 * (l16 & 3);
    c.b_chunk = col >> 3;
    c.b_swz = (4 * (krow & 3)) ^ (2 * ((krow >> 3) & 1));
    c.b_off = krow * Cfg::kBRow + 8 * ((col >> 2) & 1);
  }
  // (transposed B: row wn0 + 16 i + l16 of the stage, like the A fragment)
  {
    const int r = wn0 + l16;
    c.bt_rd[0] = r * 128 + ((g4 ^ ((r >> 1) & 7)) << 4);
    c.bt_rd[1] = c.bt_rd[0] ^ 64;
  }

  const int nk = g.K / 32;  // even: K is a multiple of 64
  int t = blockIdx.x;       // < ntiles: the grid is never larger than the tile list
  int m0, n0;
  {
    const int id = select(t, g_cur);
    direct_place<TM, TN, EDGE, BT>(SPLITK ? g_cur : g, xcd_remap(id, tiles1), c, m0, n0);
  }
  direct_prologue<TM, TN, BT>(c, nk, smem_d);
  // Without EDGE every lane issues all stores of a staged epilogue.
  const bool staged = g.out_dt != LH_F32 && !(g.flags & LH_GEMM_ACCUMULATE_C);
  const bool counted_stores = !EDGE && staged;
  bool first = true;
  for (;;) {
    f32x4 acc[2 * TN][2 * TM];
#pragma unroll
    for (int i = 0; i < 2 * TN; ++i)
#pragma unroll
      for (int j = 0; j < 2 * TM; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0f;
    u32x2 bias[2 * TN];
    const GemmArgs& ga = SPLITK ? g_cur : g;
    direct_mainloop<DT, TM, TN, EDGE, BT>(ga, c, acc, smem_d, nk, counted_stores && !first, staged, n0 + wn0 + 4 * g4, bias);
    first = false;
    const int tn = t + (int)gridDim.x;
    const bool more = tn < ntiles;
    DirectCtx<TM, TN> cn = c;
    int m1 = 0, n1 = 0;
    uint8_t* const stage = smem_d + Cfg::kRingBytes;
    if (more) {
      const int idn = select(tn, g_nxt);
      direct_place<TM, TN, EDGE, BT>(SPLITK ? g_nxt : g, xcd_remap(idn, tiles1), cn, m1, n1);
      direct_finish<DT, TM, TN, EDGE, true, BT>(ga, cn, nk, smem_d, stage, acc, bias, m0, n0, wm0, wn0);
    } else {
      direct_finish<DT, TM, TN, EDGE, false, BT>(ga, cn, nk, smem_d, stage, acc, bias, m0, n0, wm0, wn0);
    }
    if (!more) break;
    if constexpr (SPLITK) g_cur = g_nxt;
    if constexpr (TN == 2) {
      // The next tile's load offsets are computed again rather than carried through the epilogue in
      // registers: the 256-wide tiles spilled them (16 bytes per lane), and a kernel that touches
      // scratch memory at all pays for it at every dispatch (4096^3 100.5 -> 99.4 us without).
      const int idn = select(tn, g_cur);
      direct_place<TM, TN, EDGE, BT>(SPLITK ? g_cur : g, xcd_remap(idn, tiles1), c, m0, n0);
    } else {
      c = cn;
      m0 = m1;
      n0 = n1;
    }
    t = tn;
  }
}

template <int DT, int TM, int TN, bool EDGE, bool BT = false>
static int launch_direct_edge(const GemmArgs& g, hipStream_t s) {
  using Cfg = DirectCfg<TM, TN>;
  auto kern = gemm16_direct<DT, TM, TN, EDGE, false, BT>;
  constexpr size_t lds = Cfg::kLdsBytes;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int ntiles = ((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
  const int resident = num_cus() * (2 * lds <= 160 * 1024 ? 2 : 1);
  GemmArgs ga = g;
  ga.one_barrier = ntiles > num_cus();
  LH_LAUNCH(kern, dim3(ntiles < resident ? ntiles : resident), dim3(512), lds, s, ga);
  return check_launch("gemm16_direct");
}

template <int DT, int TM, int TN>
static int launch_direct(const GemmArgs& g, hipStream_t s) {
  using Cfg = DirectCfg<TM, TN>;
  const bool whole = g.M % Cfg::BM == 0 && g.N % Cfg::BN == 0;
  if (g.flags & LH_GEMM_TRANSPOSE_B)
    return whole ? launch_direct_edge<DT, TM, TN, false, true>(g, s) : launch_direct_edge<DT, TM, TN, true, true>(g, s);
  return whole ? launch_direct_edge<DT, TM, TN, false>(g, s) : launch_direct_edge<DT, TM, TN, true>(g, s);
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
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  dim3 grid((g.M / BM) * (g.N / BN));
  LH_LAUNCH(kern, grid, dim3(WAVES_M * WAVES_N * 64), lds, s, g);
  return check_launch("gemm16_fast");
}

// Tile choice for the direct kernels: 0 = 256 x 256, 1 = 256 x 128, 2 = 128 x 256, 3 = 128 x 128.
// Cost model: rounds of resident workgroups times the tile area (edge tiles count in full) times a
// measured cost per flop relative to the 256 x 256 tile (256 x 128 1.19, 128 x 256 1.17; 128 x 128
// 1.19 with two workgroups on a CU, 1.05 of it for short K, 1.30 alone).  A last round that does
// not fill the CUs costs less than a full one: the persistent workgroups are not in step, so the
// extra tiles run while others still finish, and fewer busy CUs hold a higher clock.  Measured at
// M = 8192, K = 3072 and 4096: a fraction r of a round of the large tiles costs 0.6 + 0.4 r^2 of a
// round (also when it is the only one), of the 128 x 128 tile (two workgroups per CU) 0.12 + 0.88 r.
// The 128 x 128 tile runs two workgroups per CU, which share the CU's rate: a round is 2 CUs' worth
// of tiles at twice a tile's cost, except when no CU gets a second tile.  For short K a tile's
// prologue and epilogue weigh as much as its main loop, and the 128 x 128 tile, whose two
// co-resident workgroups cover each other's, costs little more per flop than the large ones.
// On 84 shapes (M 2048 ... 8192, N 768 ... 4096, K 768 ... 4096) the choice is within 1.3 % of the best
// explicit tile.  `slow_epilogue`:
// an accumulator input or an f32 output is staged block by block, which the tiles with a 256 side
// pay more for (M = 8192, N = 768, K = 3072 + residual: 49.1 / 49.6 us against 46.6 us for 128 x 128;
// without the residual 42.6 / 43.3 against 43.0).
static int direct_variant(int M, int N, int K, bool slow_epilogue) {
  static const int bm[4] = {256, 256, 128, 128}, bn[4] = {256, 128, 256, 128};
  const int cus = num_cus();
  const double big = slow_epilogue ? 1.08 : 1.0;
  int best = -1;
  double best_cost = 0.0;
  for (int v = 0; v < 4; ++v) {
    const int64_t tiles = (int64_t)((M + bm[v] - 1) / bm[v]) * ((N + bn[v] - 1) / bn[v]);
    double cost;
    if (v < 3) {
      const double per_flop = v == 0 ? 1.0 : v == 1 ? 1.19 : 1.17;
      const double r = (double)(tiles % cus) / cus;
      const double rounds = (double)(tiles / cus) + (r > 0.0 ? 0.6 + 0.4 * r * r : 0.0);
      cost = rounds * bm[v] * bn[v] * per_flop * big;
    } else if (tiles <= cus) {
      cost = 128.0 * 128.0 * (K <= 1536 ? 1.08 : 1.30);
    } else {
      const double r = (double)(tiles % (2 * cus)) / (2 * cus);
      const double rounds = (double)(tiles / (2 * cus)) + (r > 0.0 ? 0.12 + 0.88 * r : 0.0);
      cost = rounds * 2.0 * 128.0 * 128.0 * (K <= 1536 ? 1.05 : 1.19);
    }
    if (best < 0 || cost < best_cost) {
      best = v;
      best_cost = cost;
    }
  }
  return best;
}

// Sum of the split-K blocks (f32, [splits][M][N]) and the problem's own epilogue, 4 columns per thread.
template <int DT>
__global__ void __launch_bounds__(256) gemm16_splitk_reduce(GemmArgs g, const float* partial, int splits) {
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (idx >= (int64_t)g.M * g.N) return;
  const int m = (int)(idx / g.N), n = (int)(idx % g.N);
  const f32x4 v = splitk_sum4(partial + (int64_t)m * g.N + n, (int64_t)g.M * g.N, splits, blockDim.x == 64);
  epilogue4<DT>(g, m, n, v[0], v[1], v[2], v[3]);
}

// Decode shapes: so few 128 x 128 tiles that most CUs would idle, and a K long enough to cut.
// Returns 1 when the problem does not qualify.
// `request`: LH_GEMM_SPLITK_* bits of the call; an explicit 2 / 4 / 8 bypasses the criteria.
template <int DT>
static int gemm16_splitk(const GemmArgs& g, uint32_t request, hipStream_t s) {
  using Cfg = DirectCfg<2, 1>;
  const int cus = num_cus();
  const int64_t tiles = (int64_t)((g.M + Cfg::BM - 1) / Cfg::BM) * ((g.N + Cfg::BN - 1) / Cfg::BN);
  int splits = 1;
  if (request == LH_GEMM_SPLITK_NONE) return 1;
  if (request != LH_GEMM_SPLITK_AUTO) {
    splits = request == LH_GEMM_SPLITK_2 ? 2 : request == LH_GEMM_SPLITK_4 ? 4 : 8;
    LH_REQUIRE(g.K % (splits * kBK) == 0 && g.K / splits >= 2 * kBK,
               "gemm: a cut of K = %d into %d needs K / %d to be a multiple of %d and at least %d", g.K, splits, splits,
               kBK, 2 * kBK);
  } else {
    if (tiles * 2 > cus || g.K < 2048) return 1;
    // Doubling the cut is taken while the k steps it saves each workgroup outweigh the f32 blocks it
    // adds for the second kernel to read: 0.225 us per 32 k saved (half of that once the workgroups
    // outnumber the CUs and share them), 0.62 us per MB of blocks written and read back, 2.5 us for
    // the second kernel itself.  Measured optima this reproduces (M x N x K: cut): 1024 x 1024 x 4096: 4,
    // 128 x 4096 x 4096: 4, 128 x 8192 x 8192: 4, 16 x 8192 x 8192: 8, 32 x 4096 x 4096: 8,
    // 2048 x 768 x 3072: 2, 512 x 4096 x 4096: 2, 512 x 768 x 3072: 4, 512 x 4096 x 2048 and
    // 256 x 8192 x 2048: whole.
    const double block_mb = (double)g.M * g.N * sizeof(float) * 1e-6;
    while (splits < 8) {
      const int to = splits * 2;
      if (tiles * to > 2 * cus || (g.K / to) % kBK != 0 || g.K / to < 512) break;
      const double saved = (double)(g.K / splits - g.K / to) / 32 * 0.225 * (tiles * to > cus ? 0.5 : 1.0);
      const double added = (splits == 1 ? to * block_mb * 0.62 + 2.5 : (to - splits) * block_mb * 0.62);
      if (saved <= added) break;
      splits = to;
    }
    if (splits == 1) return 1;
  }
  void* taken = nullptr;
  if (int rc = scratch_take(g.ws, s, kScratchSplitK, (size_t)splits * g.M * g.N * sizeof(float), "gemm (split K)", &taken))
    return rc;
  float* partial = static_cast<float*>(taken);
  GemmArgs p = g;
  p.K = g.K / splits;
  p.splits = splits;
  p.out = partial;
  p.c = partial;
  p.ldc = g.N;
  p.out_dt = LH_F32;
  p.bias = nullptr;
  p.flags = 0;
  p.one_barrier = 0;  // B is streamed from memory here: the deeper look-ahead wins (M = 16, N = K = 8192: 26.7 against 27.4 us)
  const bool edge = g.M % Cfg::BM != 0 || g.N % Cfg::BN != 0;
  auto launch = [&](auto kern, bool& configured) -> int {
    if (!configured && !planning()) {
      LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)Cfg::kLdsBytes));
      configured = true;
    }
    const int64_t total = tiles * splits, resident = 2 * (int64_t)cus;
    LH_LAUNCH(kern, dim3((unsigned)(total < resident ? total : resident)), dim3(512), Cfg::kLdsBytes, s, p);
    return check_launch("gemm16_direct (split K)");
  };
  static bool configured_edge = false, configured_whole = false, configured_edge_bt = false, configured_whole_bt = false;
  int rc;
  if (g.flags & LH_GEMM_TRANSPOSE_B)
    rc = edge ? launch(gemm16_direct<DT, 2, 1, true, true, true>, configured_edge_bt)
              : launch(gemm16_direct<DT, 2, 1, false, true, true>, configured_whole_bt);
  else
    rc = edge ? launch(gemm16_direct<DT, 2, 1, true, true>, configured_edge)
              : launch(gemm16_direct<DT, 2, 1, false, true>, configured_whole);
  if (rc) return rc;
  const int64_t groups = (int64_t)g.M * g.N / 4;
  const int rb = reduce_block(groups);
  LH_LAUNCH(gemm16_splitk_reduce<DT>, dim3((unsigned)((groups + rb - 1) / rb)), dim3(rb), 0, s, g, partial, splits);
  return check_launch("gemm16_splitk_reduce");
}

template <int DT>
static int gemm16_dispatch(const GemmArgs& g_in, hipStream_t s) {
  GemmArgs g = g_in;
  // A transposed B ([N, K], k contiguous) with aligned rows goes through the direct kernels as it is
  // (its panel is loaded and read like A's); a transposed A is copied into [M, K] first.
  const bool b_in_place = (g.flags & LH_GEMM_TRANSPOSE_B) && g.ldb % 8 == 0 && aligned16(g.b) && g.K % kBK == 0;
  if ((g.flags & LH_GEMM_TILE_MASK) == LH_GEMM_TILE_AUTO && g.ldc % 8 == 0 && aligned16(g.out) &&
      (!(g.flags & LH_GEMM_HAS_BIAS) || aligned16(g.bias))) {
    if (b_in_place) g.flags &= ~(uint32_t)LH_GEMM_TRANSPOSE_B;
    const int rc = untranspose_operands<2>(g, kBK, 8, s);
    if (b_in_place) g.flags |= LH_GEMM_TRANSPOSE_B;
    if (rc < 0) return rc;
  }
  const bool ta = g.flags & LH_GEMM_TRANSPOSE_A;
  const bool tb = (g.flags & LH_GEMM_TRANSPOSE_B) && !b_in_place;  // a transposed B the direct kernels cannot take
  const bool vec_ok = !ta && g.K % kBK == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 && g.ldc % 4 == 0 &&
                      aligned16(g.a) && aligned16(g.b) && aligned16(g.out) &&
                      (!(g.flags & LH_GEMM_HAS_BIAS) || aligned16(g.bias));
  const uint32_t tile = g.flags & LH_GEMM_TILE_MASK;
  const uint32_t splitk = g.flags & LH_GEMM_SPLITK_MASK;
  const bool cut_requested = splitk > LH_GEMM_SPLITK_NONE;
  if (tile == LH_GEMM_TILE_AUTO && !cut_requested && !(vec_ok && !tb && g.ldc % 8 == 0 && g.N % 8 == 0) &&
      (int64_t)g.M * g.N * g.K >= (1 << 22)) {
    // not a shape for the direct kernels as it stands: run it on padded copies of the operands
    const int rc = gemm_padded<2>(g, kBK, 8, s, [&](const GemmArgs& p) { return gemm16_dispatch<DT>(p, s); });
    if (rc <= 0) return rc;
  }
  if (tile != LH_GEMM_TILE_AUTO) {
    static const int bm[4] = {256, 256, 128, 128}, bn[4] = {256, 128, 256, 128};
    const int v = (int)(tile >> 8) - 1;
    LH_REQUIRE(vec_ok && !tb && g.ldc % 8 == 0 && g.M % bm[v] == 0 && g.N % bn[v] == 0 && direct_offsets_fit(g),
               "gemm: the requested %d x %d tile needs an untransposed A, M %% %d == 0, N %% %d == 0, "
               "K %% 64 == 0 and 16-byte aligned rows, also of a transposed B (M=%d N=%d K=%d)",
               bm[v], bn[v], bm[v], bn[v], g.M, g.N, g.K);
  }
  if (cut_requested)
    LH_REQUIRE(vec_ok && !tb && g.ldc % 8 == 0 && g.N % 8 == 0 && direct_offsets_fit(g),
               "gemm: a split-K request needs an untransposed A, K %% 64 == 0, N %% 8 == 0 and 16-byte aligned rows, "
               "also of a transposed B (M=%d N=%d K=%d)", g.M, g.N, g.K);
  if (vec_ok) {
    if (!tb && g.ldc % 8 == 0 && g.N % 8 == 0 && direct_offsets_fit(g)) {
      if (tile == LH_GEMM_TILE_AUTO) {
        const int rc = gemm16_splitk<DT>(g, splitk, s);
        if (rc <= 0) return rc;
      }
      const int v = tile != LH_GEMM_TILE_AUTO ? (int)(tile >> 8) - 1 : direct_variant(g.M, g.N, g.K, g.out_dt == LH_F32 || (g.flags & LH_GEMM_ACCUMULATE_C) != 0);
      if (v == 0) return launch_direct<DT, 4, 2>(g, s);
      if (v == 1) return launch_direct<DT, 4, 1>(g, s);
      if (v == 2) return launch_direct<DT, 2, 2>(g, s);
      if (v == 3) return launch_direct<DT, 2, 1>(g, s);
    }
    const int cus = num_cus();
    const bool big = g.M % 256 == 0 && g.N % 256 == 0 && (int64_t)(g.M / 256) * (g.N / 256) >= cus;
    if (big) {
      return tb ? launch_fast<DT, 256, 256, 2, 4, true>(g, s) : launch_fast<DT, 256, 256, 2, 4, false>(g, s);
    }
    if (g.M % 128 == 0 && g.N % 128 == 0) {
      return tb ? launch_fast<DT, 128, 128, 2, 2, true>(g, s) : launch_fast<DT, 128, 128, 2, 2, false>(g, s);
    }
  }
  dim3 grid((g.N + 63) / 64, (g.M + 63) / 64);
  LH_LAUNCH(gemm16_generic<DT>, grid, dim3(256), 0, s, g);
  return check_launch("gemm16_generic");
}

int gemm16(const GemmArgs& g, int ab_dtype, hipStream_t s) {
  if (ab_dtype == LH_BF16) return gemm16_dispatch<LH_BF16>(g, s);
  return gemm16_dispatch<LH_F16>(g, s);
}

}  // namespace lh
