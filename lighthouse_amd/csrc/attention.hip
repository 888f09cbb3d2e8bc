// Fused attention forward for gfx950: O = softmax(Q K^T * scale [+ causal mask]) V, one
// kernel, never materialising the T x T scores.  Algorithm and rounding points follow
// ReplaceWithFusedAttentionOp (lighthouse/dialects/transform/transform_ext/ops/
// replace_with_fused_attention.py:332-455): running max m, running sum l and the output
// accumulator live in f32; P is rounded to the element type before P.V; the row sum uses
// the unrounded P; the output is acc / l rounded to the element type.
//
// Work split (16-bit kernel): a workgroup owns 256 query rows of one (batch, head); each of its
// 4 waves owns 64 rows.  K/V tiles of 64 keys are staged through a 4-deep LDS ring with
// asynchronous global -> LDS loads and shared by the 4 waves, one barrier per tile.
//
// Both products are computed TRANSPOSED on the matrix cores: S^T = K Q^T and O^T = V^T P^T.
// With the 32x32 MFMA accumulator layout a lane then owns ONE query row (column of S^T) and
// 16 of its keys per tile, so the row max / row sum are register reductions plus a single
// exchange between the two half-waves, the softmax state (m, l, alpha) is one scalar per
// lane, and the S^T accumulator registers, converted to 16 bit, ARE the second operand of
// the V^T P^T product (no LDS round trip or cross-lane shuffle for P).  V^T fragments are read
// from the row-major V tile with the transposing LDS read, in the key order the accumulator
// layout produces.
#include <type_traits>

#include "common.h"

namespace lh {

struct AttnArgs {
  void* out;
  const void* q;
  const void* k;
  const void* v;
  int Z, H, T;
  lh_strides3 so, sq, sk, sv;
  float scale_log2e;  // scale * log2(e)
  float scale;
  int causal;
  int cus;  // compute units of the device (causal launch order)
  int request = 0;  // LH_ATTN_ROWS_* | LH_ATTN_STAGES_* bits of the call (0: the library chooses)
  bool scale_f32 = false;  // LH_ATTN_SCALE_F32: Q stays as stored and the scores are scaled in f32
  int d = 0;        // head dimension of the call (the padded kernels mask the columns from d on)
  // Key range split between workgroups (few query blocks, long sequences): `kv_groups` workgroups
  // per query block each take a contiguous share of its key tiles and leave (unnormalised output,
  // offset, row sum) in `part`; attention16_merge combines them.  1: one workgroup per query block.
  int kv_groups = 1;
  float* part = nullptr;
  // Causal launches of up to a third more query blocks than fit the CUs at once (32 rows per wave,
  // three workgroups per CU): the grid is `chain` = 3 x CUs workgroups, all resident, and the first
  // third of them take a second query block each (see attention16_kernel).  0: one block per workgroup.
  int chain = 0;
  // 64 rows per wave, two workgroups per CU: of every 8 key tiles, the number for which the younger
  // workgroup's waves hold the higher priority (0: the two take turns tile by tile).
  int pair_bias = 0;
  bool allow_grid_split = true;  // the caller lets the launch take temporary memory for it
  Scratch* ws = nullptr;         // where that memory comes from: a caller workspace, or (nullptr) the stream's pool
};

template <int DT>
__device__ __forceinline__ f32x16 mfma16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (DT == LH_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
}

constexpr int kHeadDim = 64;
constexpr int kKvTile = 64;
constexpr int kQBlock = 128;        // query rows per workgroup of the f32 kernel and of the register-copy kernels
constexpr int kQBlock16 = 256;      // query rows per workgroup of the 16-bit kernel (4 waves x 64)
constexpr int kAttnStageBytes = 2 * kKvTile * kHeadDim * 2;  // K tile + V tile, 16 KiB
constexpr float kOffsetSlack = 1024.0f;  // largest partial row sum of P the softmax offset tolerates

typedef __attribute__((address_space(3))) void attn_lds_void_t;
typedef short attn_s16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its second.
// Fed the same value twice it leaves (low half, low half) in the first and (high half, high
// half) in the second register, so combining the two gives every lane f(x[lane], x[lane ^ 32]).
// Written as inline asm (with the wait states the instruction needs after a VALU write of its
// operands): the compiler builtin mis-assigns the second result register.
__device__ __forceinline__ void halfwave_swap(float& lo, float& hi) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float halfwave_max(float x) {
  float a = x, b = x;
  halfwave_swap(a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float halfwave_sum(float x) {
  float a = x, b = x;
  halfwave_swap(a, b);
  return a + b;
}

// 16 bytes per lane from a buffer resource (base + per-lane byte offset) straight into LDS, 1 KiB per
// wave from lds_wave_base.  The buffer form of the LDS-DMA load, not the global (flat-encoded) one:
// while a flat-encoded LDS access is in flight the compiler has to assume LDS operations complete
// out of order and waits for ALL of a wave's LDS reads (lgkmcnt(0)) before the first use of any;
// with the buffer form it counts them, and an MFMA waits for its own fragments only.
__device__ __forceinline__ void attn_dma16(const void* base, int lane_bytes, uint8_t* lds_wave_base) {
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0xffffffff, 0x00020000);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (attn_lds_void_t*)lds_wave_base, 16, lane_bytes, 0, 0, 0);
}

struct AttnCtx {
  const uint16_t* k_base;    // K and V of the workgroup's (batch, head), key 0 (uniform)
  const uint16_t* v_base;
  int k_src[2];              // lane's byte offset within a key tile for load i
  int v_src[2];
  int64_t k_step, v_step;    // elements per key tile
  int k_row, v_row;          // bytes per key (row strides), for the clamped loads of a partial tile
  int key_local[2];          // the key of the tile that load i of this lane fetches
  int wave, r32, h;
  // Fragment reads: lane-constant byte offsets within a stage, formed once per workgroup (a tile
  // then adds the stage's base to each: one vector instruction per address).
  int k_rd[4];               // K fragment of key sub-tile 0, k-step sd (sub-tile 1: + 32 rows = 4096 bytes)
  int v_rd[2];               // V^T fragment (transposing read) of head-dim sub-tile j, keys 0 .. 15 of the tile
};

// RAGGED (sequence length T no multiple of the key tile): keys of the last, partial tile that lie
// past the end are fetched from the last key instead (and masked by the consumer).  Branch-free,
// and a template parameter, so that the loads of the common case stay one addition each.
template <bool RAGGED>
__device__ __forceinline__ void attn_issue_loads(const AttnCtx& c, int jt, int T, uint8_t* __restrict__ stage) {
  // The resources start at the tile's first key, so lane offsets stay within 64 key rows.
  const uint16_t* kt = c.k_base + jt * c.k_step;
  const uint16_t* vt = c.v_base + jt * c.v_step;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int k_off = c.k_src[i], v_off = c.v_src[i];
    if constexpr (RAGGED) {
      const int back = max(jt * kKvTile + c.key_local[i] - (T - 1), 0);  // keys past the last one
      k_off -= back * c.k_row;
      v_off -= back * c.v_row;
    }
    attn_dma16(kt, k_off, stage + (4 * i + c.wave) * 1024);
    attn_dma16(vt, v_off, stage + 8192 + (4 * i + c.wave) * 1024);
  }
}

// One key tile (64 keys) for the wave's two 32-row query sub-tiles.  `rd` holds the tile, `wr`
// is the ring slot that receives a later tile meanwhile (separate restrict pointers so that LDS
// reads do not wait for the asynchronous writes).
// (KS only separates the instantiations of the two kernels that share the other parameters.)
// SX: Q holds the stored values, the accumulators start from zero and every score is scaled and
// offset in f32 afterwards (one fused multiply-add each): the reference's rounding points exactly
// (S scaled in f32, replace_with_fused_attention.py:386), at one more vector instruction per score.
template <int DT, int NQ, bool RAGGED, bool AHEAD, int KS = 1, bool SX = false>
__device__ __forceinline__ void attn_tile(const AttnCtx& c, const AttnArgs& a, const u32x4 (&qf)[NQ][4],
                                          f32x16 (&acc_o)[NQ][2], float (&m_run)[NQ], float (&l_run)[NQ],
                                          f32x16 (&neg_m)[NQ], bool (&has_offset)[NQ], const uint8_t* __restrict__ rd,
                                          uint8_t* __restrict__ wr, int next_jt,
                                          bool prefetch, int j0, int wq0, bool active, bool need_mask, bool first) {
  if (prefetch) attn_issue_loads<RAGGED>(c, next_jt, a.T, wr);
  if (!active) return;
  const uint8_t* ks = rd;
  const uint8_t* vs = rd + 8192;
  // S^T = K Q^T: key sub-tile i (32 keys) x query sub-tile qt (32 rows).  Q carries the factor
  // scale * log2(e) and the first MFMA of a sub-tile starts from neg_m (every element of a lane's
  // block = minus the softmax offset of the lane's query row), so the accumulators come out as
  // the exponents themselves: no per-element multiply-subtract before the exp.
  // AHEAD: all K fragments are requested before the first MFMA (the registers are free in this
  // phase); left to the compiler each read is followed by its wait, one exposed LDS latency per
  // pair of MFMAs.  (Not for the instantiation that runs three waves per SIMD on 168 registers.)
  f32x16 s_acc[NQ][2];
  u32x4 kf[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int sd = 0; sd < 4; ++sd)
      kf[i][sd] = *reinterpret_cast<const u32x4*>(ks + c.k_rd[sd] + 4096 * i);
  if constexpr (AHEAD) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int sd = 0; sd < 4; ++sd)
#pragma unroll
      for (int qt = 0; qt < NQ; ++qt)
        s_acc[qt][i] = mfma16<DT>(kf[i][sd], qf[qt][sd], sd == 0 ? (SX ? f32x16{} : neg_m[qt]) : s_acc[qt][i]);
  if constexpr (SX) {
    // exponent = S * scale * log2(e) - offset, in f32 (neg_m[qt][0] is minus the lane's offset)
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) s_acc[qt][i][v] = __builtin_fmaf(s_acc[qt][i][v], a.scale_log2e, neg_m[qt][0]);
  } else {
    // A use of neg_m behind its last MFMA: without it the compiler treats that MFMA as the end of the
    // block's life, accumulates in place and first copies the block (16 moves per tile and sub-tile).
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) asm volatile("" ::"v"(neg_m[qt]));
  }
  // s_acc[qt][i][v] = S[q = wq0 + 32 qt + r32][key = j0 + 32 i + 8 (v/4) + 4 h + v%4] scale log2e - offset
  u32x4 pf[NQ][2][2];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    if (need_mask) {
      // last visible key of the row: its own index under the causal mask, and never past the end
      const int last = a.causal ? min(wq0 + 32 * qt + c.r32, a.T - 1) : a.T - 1;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          int key = j0 + 32 * i + 8 * (v >> 2) + 4 * c.h + (v & 3);
          if (key > last) s_acc[qt][i][v] = -INFINITY;
        }
    }
    // Lazy offset: P = exp(S - offset) is first computed with the offset already in use.  Softmax
    // does not depend on the offset and 16-bit P is as accurate at 2^10 as below 1, so the offset
    // only has to move when P would grow without bound: the lane's partial row sum (needed anyway)
    // is the test.  It bounds every P of the lane and cannot exceed 32 while no score has passed
    // the offset.  A row that has no offset yet (m = -inf; computed against 0) always takes the
    // slow path, so that its first visible maximum becomes the offset and l >= 1 from then on.
    // Only there is the row maximum computed, the offset raised, l and acc rescaled and P
    // recomputed, for the whole wave.
    // `first` (the workgroup's first key tile: no row has an offset yet, l and acc are zero) goes
    // straight to the slow path, without the pass that would only find that out and without
    // rescaling zeros.
    // `has_offset` (wave-uniform, set on the slow path): every row of the sub-tile has an offset, so
    // the fast path's only test is the partial row sum; a sub-tile with a row that has none yet goes
    // straight to the slow path, like the first tile.
    const float mc = m_run[qt];
    float p[2][16];
    float l_tile = 0.0f;
    bool move_offset = true;
    if (!first && has_offset[qt]) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) p[i][v] = exp2_fast(s_acc[qt][i][v]);
      l_tile = p[0][0];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = (i == 0 ? 1 : 0); v < 16; ++v) l_tile += p[i][v];
      move_offset = __builtin_amdgcn_ballot_w64(!(l_tile <= kOffsetSlack)) != 0;
    }
    if (move_offset) {
      float mx = fmaxf(s_acc[qt][0][0], s_acc[qt][1][0]);
#pragma unroll
      for (int v = 1; v < 16; ++v) mx = fmaxf(fmaxf(mx, s_acc[qt][0][v]), s_acc[qt][1][v]);
      mx = halfwave_max(mx);  // relative to the offset in use (0 for a row without one)
      const float m_old = (mc == -INFINITY) ? 0.0f : mc;
      // The offset only moves up; a row with no visible key so far (mx = -inf) stays without one.
      const float m_new = (mc == -INFINITY) ? mx : mc + fmaxf(mx, 0.0f);
      const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
      const float delta = m_safe - m_old;
      const float alpha = exp2_fast(mc - m_safe);
      m_run[qt] = m_new;
      has_offset[qt] = __builtin_amdgcn_ballot_w64(m_new == -INFINITY) == 0;
      if (!first) {
        l_run[qt] *= alpha;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc_o[qt][j][v] *= alpha;
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) p[i][v] = exp2_fast(s_acc[qt][i][v] - delta);
      l_tile = p[0][0];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = (i == 0 ? 1 : 0); v < 16; ++v) l_tile += p[i][v];
#pragma unroll
      for (int v = 0; v < 16; ++v) neg_m[qt][v] = -m_safe;
      if constexpr (!SX) asm volatile("" : "+v"(neg_m[qt]));  // a register block, not a constant to re-create per tile
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int d = 0; d < 4; ++d) pf[qt][i][u][d] = pack2<DT>(p[i][8 * u + 2 * d], p[i][8 * u + 2 * d + 1]);
    l_run[qt] += l_tile;
  }
  // O^T += V^T P^T: head-dim sub-tile j (32 of d) x query sub-tile qt, over 4 k-steps of 16 keys.
  // The V^T fragments too are all requested first.
  u32x4 vf[2][2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint8_t* p0 = vs + (32 * i + 16 * u) * 128 + c.v_rd[j];
        attn_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) attn_s16x4*)p0);
        attn_s16x4 hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) attn_s16x4*)(p0 + 8 * 128));
        u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        vf[i][u][j] = u32x4{l2[0], l2[1], h2[0], h2[1]};
      }
  if constexpr (AHEAD) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int qt = 0; qt < NQ; ++qt) acc_o[qt][j] = mfma16<DT>(vf[i][u][j], pf[qt][i][u], acc_o[qt][j]);
}

// Launch order of a causal problem.  Causal work grows with the query block index.  Rank r
// (0 = heaviest) is query block nqb - 1 - r / bhn of (batch, head) r % bhn.  With more workgroups
// than 2 per CU, or at most 1, the 1-D grid simply lists the ranks heaviest first (workgroups
// start as slots free up, so the long ones must not come last).  In between every workgroup is
// resident at once, workgroup L on CU L % cus, so the first n2 = grid - cus CUs run two: they get
// the lightest of the first `cus` ranks, lightest first, each joined by the next of the remaining
// ranks (sums stay level), and the other CUs get the heaviest ranks alone.
// `three`: the kernel runs three workgroups per CU; a grid of more than two and at most three per CU is
// then resident at once as well, and every second round of R workgroups is dealt in reverse (CU c
// gets ranks c, 2R - 1 - c, 2R + c: heavy + light + what is left, sums within a few tiles of each
// other instead of the heaviest three against the lightest three).  [8,12,1024]: +3 %.
// top - L for a round of R workgroups dealt in reverse, but with L's last three bits: workgroup ids
// that agree modulo 8 share an XCD, and with a multiple of 8 (batch, head) pairs per query block the
// blocks of a head then stay on one XCD's L2 (ranks move by less than 8 places).
__device__ __forceinline__ int mirrored_rank(int top, int L, int R) {
  return R % 8 == 0 ? (((top - L) & ~7) | (L & 7)) : top - L;
}

__device__ __forceinline__ void causal_block_of(int L, int G, int R, int nqb, int bhn, int& qb, int& bh,
                                                bool three = false) {
  int r = L;
  if (G > R && G <= 2 * R) {
    const int n2 = G - R;
    if (L < n2) r = R - 1 - L;
    else if (L < R) r = L - n2;
  } else if (three && G > 2 * R && G <= 3 * R && L >= R && L < 2 * R) {
    r = mirrored_rank(3 * R - 1, L, R);
  }
  qb = nqb - 1 - r / bhn;
  bh = r % bhn;
}

// Launch order of a non-causal problem.  Workgroups are dealt to the 8 XCDs in turn (linear id
// modulo 8), and each XCD has an L2 of its own: the query blocks of one (batch, head), which all read
// that head's K and V, are given ids that agree modulo 8, so that a K/V tile comes from memory once
// per head and not once per query block.  (With the plain (query block, head) grid and 8 query
// blocks, every block of a head sat on a different XCD.)
__device__ __forceinline__ void xcd_block_of(int L, int nqb, int bhn, int& qb, int& bh) {
  if (bhn % 8 == 0) {
    bh = (L % 8) + 8 * (L / (8 * nqb));
    qb = (L / 8) % nqb;
  } else {
    qb = L % nqb;
    bh = L / nqb;
  }
}

// 16-bit kernel.  A workgroup owns 256 query rows of one (batch, head): 4 waves x 64 rows (two
// 32-row sub-tiles per wave share every K and V fragment).  K/V tiles of 64 keys go global ->
// LDS with buffer_load_dwordx4 ... lds through a ring of NS stages; K fragments are 16-byte LDS
// reads, V^T fragments come from ds_read_b64_tr_b16 on the row-major V tile.  Rows of a tile
// are 128 bytes and cannot be padded (a wave-wide load writes 1 KiB contiguous), so the
// 16-byte chunk a lane fetches is XOR-swizzled: K chunk ^ ((key / 2) % 8), V chunk ^ 4 ((key / 2) % 2).
// KS = 2: the workgroup has two such groups of 4 waves on the SAME 256 query rows, each with a ring
// of its own and its own half of the key tiles; at the end the second group hands its (unnormalised
// output, offset, row sum) over through LDS and the first combines the two.  Same waves per CU as
// two workgroups of 4, but the two halves of a query block's key range run side by side and end
// together: the chain of key tiles a causal problem's heaviest query block has to walk is half as long.
// GS = 2 (causal, NQ = 1, NS = 3): a workgroup may take a second query block (see the loop below).
// GS = 1: the key range of a query block is split between a.kv_groups WORKGROUPS (1-D grid, query
// blocks heaviest first, the groups of one block next to each other); each leaves its partial
// result in a.part and attention16_merge finishes the block.
template <int DT, int NQ, int NS, bool RAGGED, int KS = 1, int GS = 0, bool SX = false>
__global__ void __launch_bounds__(256 * KS, (NQ == 1 && NS == 3 ? 3 : 2)) attention16_kernel(AttnArgs a_arg) {
  static_assert(!(SX && (KS != 1 || GS == 1)), "scores scaled in f32: one group of four waves per workgroup, no grid split");
  static_assert(!(GS == 1 && (KS != 1 || RAGGED)), "the grid split runs four waves per workgroup on whole key tiles");
  static_assert(GS != 2 || (NQ == 1 && NS == 3 && KS == 1), "second query blocks: the 32-rows-per-wave kernel with three workgroups per CU");
  // The instantiation whose workgroups may take a second query block reads its arguments through
  // the kernel argument pointer, made opaque once per block: the argument loads then stay inside the
  // loop over the blocks (held across it they cost 30 scalar registers more than there are, and
  // their spills the last vector registers of a kernel that runs three waves per SIMD).
  constexpr bool chained = GS == 2;
  typedef const __attribute__((address_space(4))) AttnArgs* kernarg_ptr_t;
  kernarg_ptr_t arg_ptr = (kernarg_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
  const int chain_nqb = (a_arg.T + 32 * NQ * 4 - 1) / (32 * NQ * 4), chain_bhn = a_arg.Z * a_arg.H, chain_s = a_arg.chain;
  for (int link = 0;; ++link) {
  if constexpr (chained) asm volatile("" : "+s"(arg_ptr));
  const AttnArgs& a = chained ? *(const AttnArgs*)arg_ptr : a_arg;
  constexpr int kRowsPerWave = 32 * NQ, kRowsPerGroup = 4 * kRowsPerWave;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_attn_all[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_wg = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave = wave_wg & 3, ksplit = wave_wg >> 2;  // row group within the 256 rows, key half
  uint8_t* const smem_attn = smem_attn_all + ksplit * (NS * kAttnStageBytes);
  const int r32 = lane & 31, h = lane >> 5;
  const int nqb = (a.T + kRowsPerGroup - 1) / kRowsPerGroup;
  // Chained causal launch (a.chain = S = 3 R workgroups for R CUs, resident at once, workgroup L on CU
  // L % R; at most 4 R query blocks, ranked heaviest first): the first block of a workgroup is dealt
  // as causal_block_of deals three per CU (CU c: ranks c, 2 R - 1 - c, 2 R + c), and the blocks
  // beyond 3 R go to the workgroups that hold the heaviest, lightest to heaviest (rank 4 R - 1 - c
  // after rank c), so that every CU has the same number of key tiles from the start.  With one
  // block per workgroup those blocks start wherever a slot frees first, 30 us into a [4,16,2048]
  // launch, and the launch ends with a quarter of the CUs working on them alone: 45.7 -> 43.7 us.
  // (Appended to the CU's lightest workgroup instead: 45.9; to the middle one: 48.5.  The oldest
  // workgroup of a CU wins the contested issue slots and walks its chain at a lone workgroup's pace,
  // 1.09 us per tile, whatever else the CU holds; the younger ones share what is left.)
  int qb, bh, grp = 0;
  if constexpr (chained) {
    const int R = chain_s / 3, L = (int)blockIdx.x;
    int r = L;
    if (link == 0) {
      if (L >= R && L < 2 * R) r = mirrored_rank(3 * R - 1, L, R);
    } else {
      r = (link == 1 && L < R) ? mirrored_rank(4 * R - 1, L, R) : chain_nqb * chain_bhn;
    }
    if (r >= chain_nqb * chain_bhn) break;
    qb = chain_nqb - 1 - r / chain_bhn;
    bh = r % chain_bhn;
    // (every wave has left the rings of the block before)
    if (link > 0) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  } else if constexpr (GS == 1) {
    const int per = a.Z * a.H * a.kv_groups, rem = (int)blockIdx.x % per;
    qb = nqb - 1 - (int)blockIdx.x / per;
    bh = rem / a.kv_groups;
    grp = rem % a.kv_groups;
  } else if (a.causal) {
    // (KS = 2: one workgroup per CU at a time, the others start as CUs free up: plainly heaviest first.)
    causal_block_of(blockIdx.x, gridDim.x, KS == 2 ? (int)gridDim.x : a.cus, nqb, a.Z * a.H, qb, bh, NQ == 1 && NS == 3);
  } else {
    xcd_block_of((int)(blockIdx.y * gridDim.x + blockIdx.x), nqb, a.Z * a.H, qb, bh);
  }
  const int z = bh / a.H, hd = bh % a.H;
  const int q0 = qb * kRowsPerGroup;
  const int wq0 = q0 + wave * kRowsPerWave;
  // A wave whose rows all lie past the end (last workgroup only) still takes part in the loads
  // and barriers; rows past the end inside a valid wave compute on the last row and are not stored.
  const bool wave_valid = wq0 < a.T;
  const int wq_load = wave_valid ? wq0 : 0;

  const uint16_t* Q = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)z * a.sq.z + (int64_t)hd * a.sq.h;
  const uint16_t* K = reinterpret_cast<const uint16_t*>(a.k) + (int64_t)z * a.sk.z + (int64_t)hd * a.sk.h;
  const uint16_t* V = reinterpret_cast<const uint16_t*>(a.v) + (int64_t)z * a.sv.z + (int64_t)hd * a.sv.h;
  uint16_t* O = reinterpret_cast<uint16_t*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h;

  AttnCtx c;
  c.wave = wave; c.r32 = r32; c.h = h;
  c.k_base = K;
  c.v_base = V;
  c.k_step = (int64_t)kKvTile * a.sk.t;
  c.v_step = (int64_t)kKvTile * a.sv.t;
  c.k_row = (int)a.sk.t * 2;
  c.v_row = (int)a.sv.t * 2;
  // Loader: load i of wave w fills keys (4 i + w) 8 .. +8 of the tile; lane -> key += lane / 8,
  // LDS chunk p = lane % 8 holds global chunk p ^ swizzle(key).
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int key = (4 * i + wave) * 8 + (lane >> 3);
    const int p = lane & 7;
    c.key_local[i] = key;
    c.k_src[i] = key * c.k_row + ((p ^ ((key >> 1) & 7)) << 4);
    c.v_src[i] = key * c.v_row + ((p ^ (4 * ((key >> 1) & 1))) << 4);
  }
  // K fragment (first MFMA operand of S^T): key 32 i + r32, logical chunk 2 sd + h.
  // (key sub-tile 1, 32 rows further on, has the same swizzle: 32 / 2 is a multiple of 8)
#pragma unroll
  for (int sd = 0; sd < 4; ++sd) c.k_rd[sd] = r32 * 128 + (((2 * sd + h) ^ ((r32 >> 1) & 7)) << 4);
  // V^T fragment (first MFMA operand of O^T) through the transposing read.  Lane (grp = lane/16,
  // j16 = lane % 16) addresses key row 4 h + j16 / 4 of the k-step (+8 for the second read),
  // head-dim columns 32 j + 16 (grp % 2) + 4 (j16 % 4) .. +4.  The slot order of the 8 values a
  // lane receives (keys 4h..4h+3, then 8+4h..8+4h+3) is exactly the key order of the packed
  // S^T accumulator registers it is multiplied with.
  {
    const int j16 = lane & 15, grp = lane >> 4;
    const int krow = 4 * h + (j16 >> 2);
    const int col = 16 * (grp & 1) + 4 * (j16 & 3);
    const int v_swz = 4 * ((krow >> 1) & 1);  // unchanged by + 8, + 16 u, + 32 i
    const int v_off = krow * 128 + 8 * ((col >> 2) & 1) + ((col >> 3) << 4);
#pragma unroll
    for (int j = 0; j < 2; ++j) c.v_rd[j] = v_off + (((4 * j) ^ v_swz) << 4);
  }
  // Q fragments: second MFMA operand of S^T = K Q^T; lane (q = r32, half h) holds
  // Q[q][16 sd + 8 h .. +8] for the 4 k-steps over the head dimension, for both sub-tiles.
  u32x4 qf[NQ][4];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
    for (int sd = 0; sd < 4; ++sd) {
      const int row = RAGGED ? min(wq_load + 32 * qt + r32, a.T - 1) : wq_load + 32 * qt + r32;
      const u32x4 raw = *reinterpret_cast<const u32x4*>(Q + (int64_t)row * a.sq.t + 16 * sd + 8 * h);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        qf[qt][sd][e] = SX ? raw[e]
                           : pack2<DT>(unpack_lo<DT>(raw[e]) * a.scale_log2e, unpack_hi<DT>(raw[e]) * a.scale_log2e);
    }

  f32x16 acc_o[NQ][2];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc_o[qt][j][v] = 0.0f;
  float m_run[NQ], l_run[NQ];
  f32x16 neg_m[NQ];  // minus the softmax offset of the lane's row, 16 times: the C operand of S
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    m_run[qt] = -INFINITY;
    l_run[qt] = 0.0f;
#pragma unroll
    for (int v = 0; v < 16; ++v) neg_m[qt][v] = 0.0f;
    if constexpr (!SX) asm volatile("" : "+v"(neg_m[qt]));
  }

  const int kv_end = a.causal ? min(a.T, q0 + kRowsPerGroup) : a.T;
  const int ntiles_all = (kv_end + kKvTile - 1) / kKvTile;
  // This group's key tiles are t_first .. t_first + ntiles - 1; every wave of the workgroup walks
  // `steps` iterations (the larger of the two counts), because the barrier in the loop is the
  // workgroup's: a group that has run out of tiles neither loads nor computes in the rest.
  const int share = GS == 1 ? (ntiles_all + a.kv_groups - 1) / a.kv_groups : 0;  // key tiles per workgroup of a split block
  const int t_first = GS == 1 ? grp * share : ksplit * ((ntiles_all + 1) / 2);
  const int ntiles = GS == 1 ? max(0, min(share, ntiles_all - t_first))
                        : (KS == 2 ? (ksplit ? ntiles_all - (ntiles_all + 1) / 2 : (ntiles_all + 1) / 2) : ntiles_all);
  const int steps = GS == 1 ? ntiles : (KS == 2 ? (ntiles_all + 1) / 2 : ntiles_all);
  constexpr int kAttnStages = NS;  // K/V ring depth, 3 or 4
#pragma unroll
  for (int st = 0; st < kAttnStages - 1; ++st)
    if (st < ntiles) attn_issue_loads<RAGGED>(c, t_first + st, a.T, smem_attn + st * kAttnStageBytes);

  bool has_offset[NQ];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) has_offset[qt] = false;
  for (int it = 0; it < steps; ++it) {
    // 4 loads per lane and stage; the NS - 2 younger stages may stay in flight.  One asm block: a
    // __syncthreads() would add a fence that waits for ALL outstanding loads.
    const int younger = min(ntiles - 1 - it, kAttnStages - 2);
    if (younger >= 2) asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
    else if (younger == 1) asm volatile("s_waitcnt vmcnt(4)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    if constexpr (NQ == 2 && KS == 1) {
      // Two workgroups share a CU, one wave of each per SIMD, and at equal priority the older wave
      // wins every contested issue slot: the workgroup that started first runs ahead (its 32 key
      // tiles of a [4,16,2048] launch in 51 us against 65 us for its partner, which then finishes
      // alone at a lone workgroup's lower rate).  Taking turns at the higher priority, tile by tile
      // and in opposite phase on the two wave slots, keeps the pair closer together (0.8 % of the
      // launch; 3.5 % before the query blocks of a head shared an XCD).  The 32-row kernels, three
      // workgroups per CU or long causal chains, lost 3-5 % with it.
      // Even so the older workgroup of every CU ends first ([4,16,2048]: at 58.5 us, its partner at 61.9,
      // alone for the difference).  Where a launch is a single round of two workgroups per CU the
      // younger one therefore holds the higher priority for a.pair_bias = 6 of every 8 tiles: 72.2 ->
      // 70.6 us (7 of 8: 71.4; 3 of 4: 71.1).  Launches of several rounds lose 1-2 % with any such bias
      // (the slot that frees first takes the next workgroup) and keep the even turns.
      const unsigned slot = __builtin_amdgcn_s_getreg((3u << 11) | (0u << 6) | 4u);  // HW_ID: wave slot within its SIMD
      unsigned high = ((unsigned)it ^ slot) & 1u;
      if (a.pair_bias) {
        const unsigned phase = (unsigned)it & 7u;
        high = (slot & 1u) ? (phase < (unsigned)a.pair_bias) : (phase >= (unsigned)a.pair_bias);
      }
      if (high) __builtin_amdgcn_s_setprio(1);
      else __builtin_amdgcn_s_setprio(0);
    }
    const int jt = t_first + it;
    const int j0 = jt * kKvTile;
    const bool active = wave_valid && (KS == 1 || it < ntiles) && (!a.causal || (j0 <= wq0 + kRowsPerWave - 1));
    const bool need_mask = (a.causal && (j0 + kKvTile - 1 > wq0)) || (RAGGED && j0 + kKvTile > a.T);
    const int nxt = it + kAttnStages - 1;
    attn_tile<DT, NQ, RAGGED, !(NQ == 1 && NS == 3) && !(NQ == 2 && RAGGED), KS + 2 * GS, SX>(
        c, a, qf, acc_o, m_run, l_run, neg_m, has_offset, smem_attn + (it % kAttnStages) * kAttnStageBytes,
        smem_attn + (nxt % kAttnStages) * kAttnStageBytes, t_first + nxt, nxt < ntiles, j0, wq0, active, need_mask, it == 0);
  }

  if constexpr (GS == 1) {
    // This workgroup's share of the block: accumulators in the order of the hand-over below
    // (block (wave, qt, j), four 16-byte groups of 64 lanes each), then offsets and row sums.  A
    // workgroup without a visible key tile leaves offset -inf, sum 0 and zeros.
    constexpr size_t kAccVec = (size_t)4 * NQ * 2 * 4 * 64;  // f32x4 elements
    float* const mine = a.part + ((size_t)(qb * (a.Z * a.H) + bh) * a.kv_groups + grp) * (kAccVec * 4 + 4 * NQ * 2 * 64);
    f32x4* const po = reinterpret_cast<f32x4*>(mine);
    float* const ps = mine + kAccVec * 4;
    if (wave_valid) {
#pragma unroll
      for (int qt = 0; qt < NQ; ++qt) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            po[(((wave * NQ + qt) * 2 + j) * 4 + g) * 64 + lane] =
                f32x4{acc_o[qt][j][4 * g], acc_o[qt][j][4 * g + 1], acc_o[qt][j][4 * g + 2], acc_o[qt][j][4 * g + 3]};
        ps[((wave * NQ + qt) * 2 + 0) * 64 + lane] = m_run[qt];
        ps[((wave * NQ + qt) * 2 + 1) * 64 + lane] = l_run[qt];
      }
    }
    return;
  }

  if constexpr (KS == 2) {
    // Hand-over through the (now idle) rings: block (wave, qt, j), four 16-byte groups of 64 lanes each,
    // then the offsets and row sums.  Every wave of the workgroup passes both barriers.
    f32x4* const xo = reinterpret_cast<f32x4*>(smem_attn_all);
    float* const xs = reinterpret_cast<float*>(smem_attn_all + 4 * NQ * 2 * 4 * 64 * 16);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (ksplit == 1 && wave_valid) {
#pragma unroll
      for (int qt = 0; qt < NQ; ++qt) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            xo[(((wave * NQ + qt) * 2 + j) * 4 + g) * 64 + lane] =
                f32x4{acc_o[qt][j][4 * g], acc_o[qt][j][4 * g + 1], acc_o[qt][j][4 * g + 2], acc_o[qt][j][4 * g + 3]};
        xs[((wave * NQ + qt) * 2 + 0) * 64 + lane] = m_run[qt];
        xs[((wave * NQ + qt) * 2 + 1) * 64 + lane] = l_run[qt];
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (ksplit == 1 || !wave_valid) return;
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
      // Offsets are per query row (equal in the two lanes that share it), sums per lane.  A side that
      // saw no visible key has offset -inf, sum 0 and a zero accumulator, and gets the factor 0.
      const float m_b = xs[((wave * NQ + qt) * 2 + 0) * 64 + lane];
      const float l_b = xs[((wave * NQ + qt) * 2 + 1) * 64 + lane];
      const float m_a = m_run[qt];
      const float m_ab = fmaxf(m_a, m_b);
      const float f_a = (m_a == -INFINITY) ? 0.0f : exp2_fast(m_a - m_ab);
      const float f_b = (m_b == -INFINITY) ? 0.0f : exp2_fast(m_b - m_ab);
      l_run[qt] = l_run[qt] * f_a + l_b * f_b;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 o_b = xo[(((wave * NQ + qt) * 2 + j) * 4 + g) * 64 + lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc_o[qt][j][4 * g + e] = acc_o[qt][j][4 * g + e] * f_a + o_b[e] * f_b;
        }
    }
  }

  // acc_o[qt][j][v] = O[q = wq0 + 32 qt + r32][d = 32 j + 8 (v/4) + 4 h + v%4] * l
  if (wave_valid) {
#pragma unroll
    for (int qt = 0; qt < NQ; ++qt) {
      const float inv_l = 1.0f / halfwave_sum(l_run[qt]);
      if (RAGGED && wq0 + 32 * qt + r32 >= a.T) continue;  // (after the cross-lane sum, which needs every lane)
      uint16_t* orow = O + (int64_t)(wq0 + 32 * qt + r32) * a.so.t;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          u32x2 w = {pack2<DT>(acc_o[qt][j][4 * g] * inv_l, acc_o[qt][j][4 * g + 1] * inv_l),
                     pack2<DT>(acc_o[qt][j][4 * g + 2] * inv_l, acc_o[qt][j][4 * g + 3] * inv_l)};
          *reinterpret_cast<u32x2*>(orow + 32 * j + 8 * g + 4 * h) = w;
        }
    }
  }
  if (!chained) break;
  }  // (the workgroup's next query block)
}

template <int DT, int NQ, int NS, bool RAGGED, int KS = 1, bool SX = false>
static int attention16_launch_ragged(const AttnArgs& a, hipStream_t s) {
  if constexpr (KS == 1 && !SX) {
    if (a.scale_f32) return attention16_launch_ragged<DT, NQ, NS, RAGGED, 1, true>(a, s);
  }
  constexpr bool kCanChain = NQ == 1 && NS == 3 && KS == 1;
  const bool chained = kCanChain && a.causal && a.chain > 0;
  auto kern = attention16_kernel<DT, NQ, NS, RAGGED, KS, 0, SX>;
  constexpr size_t lds = (size_t)KS * NS * kAttnStageBytes;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int nqb = (a.T + 128 * NQ - 1) / (128 * NQ);
  if constexpr (kCanChain) {
    if (chained) {
      auto kern2 = attention16_kernel<DT, NQ, NS, RAGGED, KS, 2, SX>;
      static bool configured2 = false;
      if (!configured2 && !planning()) {
        LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern2), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds));
        configured2 = true;
      }
      LH_LAUNCH(kern2, dim3(a.chain), dim3(256 * KS), lds, s, a);
      return check_launch("attention16");
    }
  }
  const dim3 grid = a.causal ? dim3(nqb * a.Z * a.H) : dim3(nqb, a.Z * a.H);
  LH_LAUNCH(kern, grid, dim3(256 * KS), lds, s, a);
  return check_launch("attention16");
}

// Second kernel of a launch whose query blocks were split between workgroups: one workgroup per
// query block reads the kv_groups partial results in the order of the groups (so the result does
// not depend on which finished first), rescales them to the common offset, normalises and writes
// the rows.  Same thread -> element mapping as the attention kernel's own epilogue.
template <int DT, int NQ>
__global__ void __launch_bounds__(256) attention16_merge(AttnArgs a) {
  constexpr int kRowsPerWave = 32 * NQ, kRowsPerGroup = 4 * kRowsPerWave;
  constexpr size_t kAccVec = (size_t)4 * NQ * 2 * 4 * 64, kPartFloats = kAccVec * 4 + 4 * NQ * 2 * 64;
  constexpr int kMaxGroups = 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, h = lane >> 5;
  const int bhn = a.Z * a.H, G = a.kv_groups;
  const int qb = (int)blockIdx.x / bhn, bh = (int)blockIdx.x % bhn;
  // blockIdx.y: which 4 columns x 64 lanes piece of the wave's rows (sub-tile qt, column block j, group q4)
  const int qt = (int)blockIdx.y / 8, j = ((int)blockIdx.y / 4) & 1, q4 = (int)blockIdx.y & 3;
  const int z = bh / a.H, hd = bh % a.H;
  const int wq0 = qb * kRowsPerGroup + wave * kRowsPerWave;
  if (wq0 >= a.T) return;
  const float* const base = a.part + (size_t)(qb * bhn + bh) * G * kPartFloats;
  // Offsets are per query row (equal in the two lanes that share it), sums per lane; a group that
  // saw no visible key has offset -inf and counts as zero.  All loads of a pass are independent.
  float f[kMaxGroups], lg[kMaxGroups];
  f32x4 v[kMaxGroups];
#pragma unroll
  for (int g = 0; g < kMaxGroups; ++g) {
    const float* p = base + (size_t)min(g, G - 1) * kPartFloats;
    f[g] = p[kAccVec * 4 + ((wave * NQ + qt) * 2 + 0) * 64 + lane];
    lg[g] = p[kAccVec * 4 + ((wave * NQ + qt) * 2 + 1) * 64 + lane];
    v[g] = reinterpret_cast<const f32x4*>(p)[(((wave * NQ + qt) * 2 + j) * 4 + q4) * 64 + lane];
  }
  float m_all = -INFINITY;
#pragma unroll
  for (int g = 0; g < kMaxGroups; ++g) m_all = fmaxf(m_all, f[g]);  // (slots from G on repeat the last group)
  float l = 0.0f;
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int g = 0; g < kMaxGroups; ++g) {
    const float w = (g >= G || f[g] == -INFINITY) ? 0.0f : exp2_fast(f[g] - m_all);
    l += lg[g] * w;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += v[g][e] * w;
  }
  const float inv_l = 1.0f / halfwave_sum(l);
  uint16_t* orow = reinterpret_cast<uint16_t*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h +
                   (int64_t)(wq0 + 32 * qt + r32) * a.so.t;
  u32x2 w = {pack2<DT>(acc[0] * inv_l, acc[1] * inv_l), pack2<DT>(acc[2] * inv_l, acc[3] * inv_l)};
  *reinterpret_cast<u32x2*>(orow + 32 * j + 8 * q4 + 4 * h) = w;
}

// Query blocks split between `groups` workgroups each (a.T a multiple of the key tile): the
// attention kernel leaves partial results in temporary memory, the merge kernel finishes.
template <int DT, int NQ>
static int attention16_launch_split(const AttnArgs& a_in, int groups, hipStream_t s) {
  constexpr size_t kPartFloats = (size_t)4 * NQ * 2 * 4 * 64 * 4 + 4 * NQ * 2 * 64;
  constexpr size_t lds = (size_t)4 * kAttnStageBytes;
  auto kern = attention16_kernel<DT, NQ, 4, false, 1, 1>;
  auto merge = attention16_merge<DT, NQ>;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int nqb = (a_in.T + 128 * NQ - 1) / (128 * NQ), bhn = a_in.Z * a_in.H;
  void* part = nullptr;
  if (int rc = scratch_take(a_in.ws, s, kScratchAttention, (size_t)nqb * bhn * groups * kPartFloats * sizeof(float),
                            "attention (key range split between workgroups)", &part))
    return rc;
  AttnArgs a = a_in;
  a.kv_groups = groups;
  a.part = static_cast<float*>(part);
  LH_LAUNCH(kern, dim3(nqb * bhn * groups), dim3(256), lds, s, a);
  if (int rc = check_launch("attention16 (split)")) return rc;
  LH_LAUNCH(merge, dim3(nqb * bhn, NQ * 8), dim3(256), 0, s, a);
  return check_launch("attention16_merge");
}

// Sequence lengths that are no multiple of the key tile take the instantiation that clamps the
// last tile's loads, masks it and skips rows past the end.
template <int DT, int NQ, int NS>
static int attention16_launch_nq(const AttnArgs& a, hipStream_t s) {
  if constexpr (NQ == 1) {
    if (a.T % kKvTile != 0) return attention16_launch_ragged<DT, NQ, NS, true>(a, s);
  }
  return attention16_launch_ragged<DT, NQ, NS, false>(a, s);
}

// 64 query rows per wave share every K/V fragment between two sub-tiles; 32 rows per wave give
// twice the workgroups, each half as long, which is what a problem needs that would otherwise
// leave CUs with fewer than two workgroups or hang on its heaviest causal block.
template <int DT>
static int attention16_launch(const AttnArgs& a, hipStream_t s) {
  const int64_t groups64 = (int64_t)((a.T + kQBlock16 - 1) / kQBlock16) * a.Z * a.H;
  // Measured on [4,16,2048]: 32 rows per wave 105 us non-causal (64 rows: 99) but 54 us causal
  // (64 rows: 58), hence the different limits.
  // Causal launches of sequences up to 1024 stay on the 32-row kernel up to four 256-row groups per
  // CU (the masked diagonal is a larger share of a 256-row block: [1,192,1024] 42.7 vs 44.8 us,
  // [1,512,512] 41.1 vs 43.3; beyond that the 64-row kernel is ahead again, [1,512,1024] 108 vs 113).
  const int64_t limit = !a.causal ? 2 * (int64_t)a.cus : (a.T <= 1024 ? 4 : 2) * (int64_t)a.cus + 1;
  // Short sequences that do not fill their last 256-row block waste less of a 128-row one
  // ([64,16,257]: 80 -> 57 us, [128,12,300]: 111 -> 82 us).
  const bool short_rows = a.T <= 640 && a.T % kQBlock16 != 0;
  // (A partial last key tile also takes the 32-rows-per-wave kernels: the 64-row one has no
  // registers left for the clamped loads and would spill.)
  const int rows_req = a.request & LH_ATTN_ROWS_MASK, stages_req = a.request & LH_ATTN_STAGES_MASK;
  const int ksplit_req = a.request & LH_ATTN_KSPLIT_MASK;
  if (rows_req == LH_ATTN_ROWS_64 && ksplit_req != LH_ATTN_KSPLIT_2) {
    LH_REQUIRE(a.T % kKvTile == 0, "attention: 64 query rows per wave need a sequence length that is a multiple of %d",
               kKvTile);
    LH_REQUIRE(stages_req != LH_ATTN_STAGES_3, "attention: the 64-rows-per-wave kernel has a 4-stage ring only");
    return attention16_launch_nq<DT, 2, 4>(a, s);
  }
  if (ksplit_req == LH_ATTN_KSPLIT_2) {
    LH_REQUIRE(!a.scale_f32, "attention: LH_ATTN_SCALE_F32 exists for one group of four waves per workgroup (not with LH_ATTN_KSPLIT_2)");
    // Two groups of four waves per workgroup, each on half of the key tiles (64 rows per wave, 4 stages).
    LH_REQUIRE(rows_req != LH_ATTN_ROWS_32 && stages_req != LH_ATTN_STAGES_3,
               "attention: the split key range exists for 64 query rows per wave and a 4-stage ring only");
    LH_REQUIRE(a.T % kKvTile == 0, "attention: 64 query rows per wave need a sequence length that is a multiple of %d",
               kKvTile);
    return attention16_launch_ragged<DT, 2, 4, false, 2>(a, s);
  }
  // Few query blocks and many key tiles (long sequences of a few heads): the key range of every
  // block is split between workgroups and a second kernel merges the partial results (temporary
  // memory: 68 KiB per workgroup).  Without the split such a problem runs one 128-row workgroup on
  // at most every CU, each walking the whole key range (causal: the heaviest does): about 5 us +
  // 0.77 us per key tile.  With it a workgroup walks 1 / groups of the range at 1.075 us per tile
  // (1.61 when two share a CU, whose start-up also costs 5 us less than a lone workgroup's) and the
  // launch pays 7.2 us (second launch, first loads) + 0.027 us per workgroup for writing and reading
  // the partial results.  Fitted on [1,1,8192] 93.7 -> 31 us,
  // [1,4,4096] 49.9 -> 33.5, [1,4,8192] 104 -> 83 -> (4 groups), [1,1,16384] 183 -> 78, and on
  // [2,8,2048], which stays whole (28.4 us against 34.7 split).
  if (!ksplit_req && !rows_req && !stages_req && !a.scale_f32 && a.allow_grid_split && a.T % kKvTile == 0 &&
      2 * groups64 <= a.cus) {
    const int ntiles = a.T / kKvTile;
    const double whole = 5.0 + 0.77 * ntiles;
    int best_groups = 1;
    double best = 0.9 * whole;  // the split has to win by a margin
    for (int groups = 2; groups <= 16 && ntiles / groups >= 2; groups *= 2) {
      const int64_t wgs = groups64 * groups;
      const double t = (wgs <= a.cus ? 12.2 : 7.2) + 0.027 * (double)wgs +
                       (double)((ntiles + groups - 1) / groups) * (wgs <= a.cus ? 1.075 : 1.61);
      if (wgs <= 2 * (int64_t)a.cus && t < best) {
        best = t;
        best_groups = groups;
      }
    }
    if (best_groups > 1) return attention16_launch_split<DT, 2>(a, best_groups, s);
  }
  // Unasked, the split pays where at most one 256-row workgroup falls on a CU but more than half
  // the CUs get one: a lone group of four waves leaves each SIMD with a single wave, and splitting the
  // rows instead (the 32-row kernel) halves the reuse of every K/V fragment.  Non-causal
  // [1,16,4096] 77 -> 72 us, [1,8,8192] 152 -> 132 us.  Causal problems are bound by the
  // total of their key tiles, not by the longest chain ([4,16,2048] 47 -> 53 us with the split).
  if (!ksplit_req && !rows_req && !stages_req && !a.scale_f32 && !a.causal && a.T % kKvTile == 0 && groups64 <= a.cus &&
      2 * groups64 > a.cus)
    return attention16_launch_ragged<DT, 2, 4, false, 2>(a, s);
  if (rows_req == LH_ATTN_ROWS_32 || stages_req) {
    const int64_t groups32 = (int64_t)((a.T + 127) / 128) * a.Z * a.H;
    const bool three = stages_req ? stages_req == LH_ATTN_STAGES_3 : groups32 >= 3 * (int64_t)a.cus;
    if (three) return attention16_launch_nq<DT, 1, 3>(a, s);
    return attention16_launch_nq<DT, 1, 4>(a, s);
  }
  if (groups64 < limit || short_rows || a.T % kKvTile != 0) {
    // With three 128-row workgroups or more per CU a ring of 3 stages (48 KiB) lets three of them
    // share a CU instead of two ([8,12,1024] causal 26.7 -> 25.3 us, [16,16,512] causal 24.2 ->
    // 22.3); a problem that cannot put a third one there is better off with the deeper ring
    // (causal [1,16,4096] 57.9 -> 53.9 us, [1,8,8192] 108 -> 98.8, [2,16,2048] 32.7 -> 30.6, [1,40,2048] 36.2 -> 33.7).
    const int64_t groups32 = (int64_t)((a.T + 127) / 128) * a.Z * a.H;
    if (groups32 >= 3 * (int64_t)a.cus) {
      // Causal, 3.5 to 4 per CU, sequences from 1000 on: all resident, a second block for a third of them
      // ([4,16,2048] 45.7 -> 43.7 us, [2,16,4096] 80.9 -> 77.8, [7,16,1024] 25.8 -> 24.9, [7,18,1000] 32.2 -> 29.6;
      // at 3.25 per CU, or with 512-key sequences, the plain launch is 2-3 % ahead).
      if (a.causal && a.T >= 1000 && 2 * groups32 >= 7 * (int64_t)a.cus && groups32 <= 4 * (int64_t)a.cus) {
        AttnArgs ac = a;
        ac.chain = 3 * a.cus;
        return attention16_launch_nq<DT, 1, 3>(ac, s);
      }
      return attention16_launch_nq<DT, 1, 3>(a, s);
    }
    return attention16_launch_nq<DT, 1, 4>(a, s);
  }
  if (!a.causal && groups64 == 2 * (int64_t)a.cus) {  // exactly one round of two workgroups per CU (fewer take the 32-row kernels)
    AttnArgs ab = a;
    ab.pair_bias = 6;
    return attention16_launch_nq<DT, 2, 4>(ab, s);
  }
  return attention16_launch_nq<DT, 2, 4>(a, s);
}

// How the register-copy kernels below treat a head dimension d under their compiled width D:
// kRowsExact: d == D.  kRowsChunks: rows are 16-byte aligned and d is a whole number of 16-byte
// chunks; a chunk from column d on reads as zeros (its load goes to the row's first chunk and is
// dropped: no branch) and is not stored.  kRowsElements: any d, any alignment; element loads and
// stores, a column from d on reads as zero (its load goes to the row's last element).
constexpr int kRowsExact = 0, kRowsChunks = 1, kRowsElements = 2;

// Columns c .. c + 7 of a 16-bit row.
template <int ROWS>
__device__ __forceinline__ u32x4 row_chunk16(const uint16_t* row, int c, int d) {
  if constexpr (ROWS == kRowsElements) {
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c0 = c + 2 * e, c1 = c0 + 1;
      uint32_t lo = row[min(c0, d - 1)], hi = row[min(c1, d - 1)];
      if (c0 >= d) lo = 0u;
      if (c1 >= d) hi = 0u;
      r[e] = lo | (hi << 16);
    }
    return r;
  } else {
    const bool inside = ROWS == kRowsExact || c < d;
    u32x4 raw = *reinterpret_cast<const u32x4*>(row + (inside ? c : 0));
    if (ROWS != kRowsExact && !inside) raw = u32x4{0u, 0u, 0u, 0u};
    return raw;
  }
}
// Columns c .. c + 3 of a 16-bit row, stored.
template <int ROWS>
__device__ __forceinline__ void store_chunk16(uint16_t* row, int c, int d, u32x2 w) {
  if constexpr (ROWS == kRowsElements) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (c + e < d) row[c + e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
  } else {
    if (ROWS == kRowsExact || c < d) *reinterpret_cast<u32x2*>(row + c) = w;
  }
}
// Columns c .. c + 3 of an f32 row.
template <int ROWS>
__device__ __forceinline__ f32x4 row_chunk32(const float* row, int c, int d) {
  if constexpr (ROWS == kRowsElements) {
    f32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[e] = row[min(c + e, d - 1)];
      if (c + e >= d) r[e] = 0.0f;
    }
    return r;
  } else {
    const bool inside = ROWS == kRowsExact || c < d;
    f32x4 raw = *reinterpret_cast<const f32x4*>(row + (inside ? c : 0));
    if (ROWS != kRowsExact && !inside) raw = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    return raw;
  }
}
template <int ROWS>
__device__ __forceinline__ void store_chunk32(float* row, int c, int d, f32x4 w) {
  if constexpr (ROWS == kRowsElements) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (c + e < d) row[c + e] = w[e];
  } else {
    if (ROWS == kRowsExact || c < d) *reinterpret_cast<f32x4*>(row + c) = w;
  }
}

// 16-bit tensors, head dimension D = 32 DB (32, 96, 128, 192, 256; 64 and 128 for padded calls): the same
// transposed formulation on the matrix cores (S^T = K Q^T, O^T = V^T P^T, a lane owns a query row)
// without the streaming machinery of the head-dimension-64 kernel.  A workgroup owns 128 query
// rows (4 waves x 32); a tile of 64 keys is copied through registers into LDS, K and V row-major
// with rows padded by 16 bytes (V^T fragments through ds_read_b64_tr_b16), two barriers per tile.  Row statistics follow the plain online-softmax recurrence (maximum per
// tile).  Any sequence length: keys past the end are loaded from the last key and masked, rows
// past the end are computed on the last row and not stored.
// ROWS != kRowsExact: the head dimension a.d lies below D (or the rows are not 16-byte aligned).
// The columns of Q, K and V from a.d on are zeros in registers and LDS (they add nothing to S, and
// their output columns are not stored), so the result is that of head dimension a.d exactly.
template <int DT, int DB, int ROWS>
__global__ void __launch_bounds__(256, (DB <= 2 || (DB == 3 && ROWS != kRowsElements) ? 2 : 1)) attention16_anyd_kernel(AttnArgs a) {
  constexpr int D = 32 * DB;
  const int d_real = ROWS != kRowsExact ? a.d : D;
  constexpr int KROW = D + 8;  // elements per LDS row
  extern __shared__ __attribute__((aligned(16))) uint8_t smem_anyd[];
  uint16_t* Ks = reinterpret_cast<uint16_t*>(smem_anyd);  // [64][KROW]
  uint16_t* Vs = Ks + kKvTile * KROW;                     // [64][KROW]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int nqb = (a.T + 127) / 128;
  // Causal work grows with the query block: a 1-D grid lists the blocks heaviest first over ALL
  // (batch, head) pairs, so that the long ones do not start last.
  const int bhn = a.Z * a.H;
  int qb = nqb - 1 - (int)blockIdx.x / bhn, bh = (int)blockIdx.x % bhn;
  if (!a.causal) xcd_block_of((int)(blockIdx.y * gridDim.x + blockIdx.x), nqb, bhn, qb, bh);
  const int z = bh / a.H, hd = bh % a.H;
  const int q0 = qb * 128, wq0 = q0 + 32 * wave;
  const bool wave_valid = wq0 < a.T;

  const uint16_t* Q = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)z * a.sq.z + (int64_t)hd * a.sq.h;
  const uint16_t* K = reinterpret_cast<const uint16_t*>(a.k) + (int64_t)z * a.sk.z + (int64_t)hd * a.sk.h;
  const uint16_t* V = reinterpret_cast<const uint16_t*>(a.v) + (int64_t)z * a.sv.z + (int64_t)hd * a.sv.h;
  uint16_t* O = reinterpret_cast<uint16_t*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h;

  // Q fragments (second MFMA operand of S^T), times scale * log2(e): lane (row r32, half h) holds
  // Q[row][16 sd + 8 h .. +8].  They live in registers, or for the largest head dimension (whose
  // output accumulators alone take 128 registers) in the wave's own 16 KiB of LDS, in fragment order.
  constexpr bool Q_LDS = DB >= 8;
  u32x4 qf[Q_LDS ? 1 : D / 16];
  u32x4* q_lds = reinterpret_cast<u32x4*>(Vs + kKvTile * KROW) + wave * (D / 16) * 64 + lane;
  {
    const int row = min(wq0 + r32, a.T - 1);
#pragma unroll
    for (int sd = 0; sd < D / 16; ++sd) {
      const u32x4 raw = row_chunk16<ROWS>(Q + (int64_t)row * a.sq.t, 16 * sd + 8 * h, d_real);
      u32x4 scaled;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        scaled[e] = pack2<DT>(unpack_lo<DT>(raw[e]) * a.scale_log2e, unpack_hi<DT>(raw[e]) * a.scale_log2e);
      if constexpr (Q_LDS) q_lds[sd * 64] = scaled;
      else qf[sd] = scaled;
      if constexpr (ROWS == kRowsElements) asm volatile("" ::: "memory");  // (one chunk's element loads at a time)
    }
  }
  f32x16 acc_o[DB];
#pragma unroll
  for (int j = 0; j < DB; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_o[j][v] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  f32x16 neg_m;
#pragma unroll
  for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
  asm volatile("" : "+v"(neg_m));

  const int kv_end = a.causal ? min(a.T, q0 + 128) : a.T;
  const int ntiles = (kv_end + kKvTile - 1) / kKvTile;
  for (int jt = 0; jt < ntiles; ++jt) {
    const int j0 = jt * kKvTile;
    __syncthreads();  // the previous tile has been consumed
    // (opaque per tile: the masks and clamped columns that depend on it are formed where they are used
    // and not kept in registers across the loop)
    int d_tile = d_real;
    if constexpr (ROWS != kRowsExact) asm volatile("" : "+s"(d_tile));
    // 8 D 16-byte chunks per tile and tensor, DB per thread: chunk c = key c / (D / 8), columns 8 (c % (D / 8)) .. +8.
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      const int c = tid + 256 * i, key = c / (D / 8), ch = c % (D / 8);
      const int kg = min(j0 + key, a.T - 1);
      const u32x4 kv = row_chunk16<ROWS>(K + (int64_t)kg * a.sk.t, 8 * ch, d_tile);
      const u32x4 vv = row_chunk16<ROWS>(V + (int64_t)kg * a.sv.t, 8 * ch, d_tile);
      *reinterpret_cast<u32x4*>(Ks + key * KROW + 8 * ch) = kv;
      *reinterpret_cast<u32x4*>(Vs + key * KROW + 8 * ch) = vv;
      if constexpr (ROWS == kRowsElements) asm volatile("" ::: "memory");  // (16 element loads in flight, not 16 DB)
    }
    __syncthreads();
    if (!wave_valid || (a.causal && j0 > wq0 + 31)) continue;
    // S^T = K Q^T - offset: the first MFMA of a sub-tile starts from neg_m (minus the lane's softmax
    // offset, 16 times), so the accumulators are the exponents; lazy offset as in attn_tile.
    f32x16 s_acc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int sd = 0; sd < D / 16; ++sd) {
        const u32x4 kf = *reinterpret_cast<const u32x4*>(Ks + (32 * i + r32) * KROW + 16 * sd + 8 * h);
        if constexpr (Q_LDS) s_acc[i] = mfma16<DT>(kf, q_lds[sd * 64], sd == 0 ? neg_m : s_acc[i]);
        else s_acc[i] = mfma16<DT>(kf, qf[sd], sd == 0 ? neg_m : s_acc[i]);
      }
    asm volatile("" ::"v"(neg_m));  // (alive past its last MFMA: no accumulator copies)
    if ((a.causal && j0 + kKvTile - 1 > wq0) || j0 + kKvTile > a.T) {
      const int last = a.causal ? min(wq0 + r32, a.T - 1) : a.T - 1;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (j0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3) > last) s_acc[i][v] = -INFINITY;
    }
    const float mc = m_run;
    float p[2][16];
    float l_tile = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        p[i][v] = exp2_fast(s_acc[i][v]);
        l_tile += p[i][v];
      }
    if (__builtin_amdgcn_ballot_w64(!(l_tile <= kOffsetSlack) || mc == -INFINITY) != 0) {
      float mx = fmaxf(s_acc[0][0], s_acc[1][0]);
#pragma unroll
      for (int v = 1; v < 16; ++v) mx = fmaxf(fmaxf(mx, s_acc[0][v]), s_acc[1][v]);
      mx = halfwave_max(mx);  // relative to the offset in use (0 for a row without one)
      const float m_old = (mc == -INFINITY) ? 0.0f : mc;
      const float m_new = (mc == -INFINITY) ? mx : mc + fmaxf(mx, 0.0f);
      const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
      const float delta = m_safe - m_old;
      const float alpha = exp2_fast(mc - m_safe);
      l_run *= alpha;
      m_run = m_new;
#pragma unroll
      for (int j = 0; j < DB; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_o[j][v] *= alpha;
      l_tile = 0.0f;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          p[i][v] = exp2_fast(s_acc[i][v] - delta);
          l_tile += p[i][v];
        }
#pragma unroll
      for (int v = 0; v < 16; ++v) neg_m[v] = -m_safe;
      asm volatile("" : "+v"(neg_m));
    }
    l_run += l_tile;
    // O^T += V^T P^T.  V^T fragments come from the row-major tile through the transposing read:
    // lane (g4 = lane / 16, j16 = lane % 16) addresses key row 4 h + j16 / 4 of the 16-key step
    // (+8 for the second read), columns 32 j + 16 (g4 % 2) + 4 (j16 % 4) .. +4, and receives 8 keys
    // of one column in exactly the key order of the packed P registers.
    const int tr_row = 4 * h + ((lane & 15) >> 2), tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x4 pf;
#pragma unroll
        for (int d = 0; d < 4; ++d) pf[d] = pack2<DT>(p[i][8 * u + 2 * d], p[i][8 * u + 2 * d + 1]);
#pragma unroll
        for (int j = 0; j < DB; ++j) {
          const uint16_t* p0 = Vs + (32 * i + 16 * u + tr_row) * KROW + 32 * j + tr_col;
          const attn_s16x4 lo =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) attn_s16x4*)p0);
          const attn_s16x4 hi =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) attn_s16x4*)(p0 + 8 * KROW));
          const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          acc_o[j] = mfma16<DT>(u32x4{l2[0], l2[1], h2[0], h2[1]}, pf, acc_o[j]);
        }
      }
  }
  // acc_o[j][v] = O[q = wq0 + r32][d = 32 j + 8 (v / 4) + 4 h + v % 4] * l
  if (!wave_valid) return;
  const float inv_l = 1.0f / halfwave_sum(l_run);
  if (wq0 + r32 >= a.T) return;
  uint16_t* orow = O + (int64_t)(wq0 + r32) * a.so.t;
#pragma unroll
  for (int j = 0; j < DB; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w = {pack2<DT>(acc_o[j][4 * g] * inv_l, acc_o[j][4 * g + 1] * inv_l),
                 pack2<DT>(acc_o[j][4 * g + 2] * inv_l, acc_o[j][4 * g + 3] * inv_l)};
      store_chunk16<ROWS>(orow, 32 * j + 8 * g + 4 * h, d_real, w);
    }
}

// Head dimension 128, 16-bit: the kernel above with the key tiles brought in by LDS-DMA
// (buffer_load_dwordx4 ... lds, no registers, no LDS stores) into two unpadded stages, the load of tile
// j + 1 running under the arithmetic of tile j, one barrier per tile.  Rows are 256 bytes = the 64
// LDS banks, so the 16-byte chunk a lane fetches is XOR-swizzled with the key's low four bits
// (LDS chunk p of key row k holds global chunk p ^ (k % 16)); a wave-wide load fills 4 key rows.
constexpr int kD128TileBytes = kKvTile * 256;          // one tensor's tile
constexpr int kD128StageBytes = 2 * kD128TileBytes;    // K tile + V tile, 32 KiB

struct Attn128Ctx {
  const uint16_t* k_base;    // K and V of the workgroup's (batch, head), key 0 (uniform)
  const uint16_t* v_base;
  int chunk_bytes[4];        // byte offset of the 16-byte chunk of a key row that load i of this lane fetches
  int key_local[4];          // the key of a tile that load i of this lane fetches
  int64_t k_row, v_row;      // elements per key
  int wave;
};

__device__ __forceinline__ void attn128_issue(const Attn128Ctx& c, int jt, int T, uint8_t* __restrict__ stage) {
  // The resources start at the tile's first key, so lane offsets stay within 64 key rows.
  const uint16_t* kt = c.k_base + (int64_t)jt * kKvTile * c.k_row;
  const uint16_t* vt = c.v_base + (int64_t)jt * kKvTile * c.v_row;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // keys past the end repeat the last one (masked later)
    const int key = min(c.key_local[i], T - 1 - jt * kKvTile);
    attn_dma16(kt, key * (int)c.k_row * 2 + c.chunk_bytes[i], stage + (4 * i + c.wave) * 1024);
    attn_dma16(vt, key * (int)c.v_row * 2 + c.chunk_bytes[i], stage + kD128TileBytes + (4 * i + c.wave) * 1024);
  }
}

// One key tile for the wave's 32 query rows.  `rd` holds the tile, `wr` receives the next one
// meanwhile (separate restrict pointers so that LDS reads do not wait for the asynchronous writes).
template <int DT>
__device__ __forceinline__ void attn128_tile(const Attn128Ctx& c, const AttnArgs& a, const u32x4 (&qf)[8],
                                             f32x16 (&acc_o)[4], float& m_run, float& l_run, f32x16& neg_m,
                                             const uint8_t* __restrict__ rd, uint8_t* __restrict__ wr, int next_jt,
                                             bool prefetch, int j0, int wq0, bool active, int lane) {
  if (prefetch) attn128_issue(c, next_jt, a.T, wr);
  if (!active) return;
  const int r32 = lane & 31, h = lane >> 5;
  const uint8_t* ks = rd;
  const uint8_t* vs = rd + kD128TileBytes;
  // S^T = K Q^T - offset: Q carries scale * log2(e) and the first MFMA of a sub-tile starts from
  // neg_m (minus the softmax offset of the lane's row, 16 times), so the accumulators are the
  // exponents; the offset is lazy as in the head-dimension-64 kernel (attn_tile).
  f32x16 s_acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int sd = 0; sd < 8; ++sd) {
      const u32x4 kf = *reinterpret_cast<const u32x4*>(ks + (32 * i + r32) * 256 + (((2 * sd + h) ^ (r32 & 15)) << 4));
      s_acc[i] = mfma16<DT>(kf, qf[sd], sd == 0 ? neg_m : s_acc[i]);
    }
  asm volatile("" ::"v"(neg_m));  // (alive past its last MFMA: no accumulator copies)
  if ((a.causal && j0 + kKvTile - 1 > wq0) || j0 + kKvTile > a.T) {
    const int last = a.causal ? min(wq0 + r32, a.T - 1) : a.T - 1;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if (j0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3) > last) s_acc[i][v] = -INFINITY;
  }
  const float mc = m_run;
  float p[2][16];
  float l_tile = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      p[i][v] = exp2_fast(s_acc[i][v]);
      l_tile += p[i][v];
    }
  if (__builtin_amdgcn_ballot_w64(!(l_tile <= kOffsetSlack) || mc == -INFINITY) != 0) {
    float mx = fmaxf(s_acc[0][0], s_acc[1][0]);
#pragma unroll
    for (int v = 1; v < 16; ++v) mx = fmaxf(fmaxf(mx, s_acc[0][v]), s_acc[1][v]);
    mx = halfwave_max(mx);  // relative to the offset in use (0 for a row without one)
    const float m_old = (mc == -INFINITY) ? 0.0f : mc;
    const float m_new = (mc == -INFINITY) ? mx : mc + fmaxf(mx, 0.0f);
    const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
    const float delta = m_safe - m_old;
    const float alpha = exp2_fast(mc - m_safe);
    l_run *= alpha;
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc_o[j][v] *= alpha;
    l_tile = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        p[i][v] = exp2_fast(s_acc[i][v] - delta);
        l_tile += p[i][v];
      }
#pragma unroll
    for (int v = 0; v < 16; ++v) neg_m[v] = -m_safe;
    asm volatile("" : "+v"(neg_m));
  }
  l_run += l_tile;
  // V^T fragments through the transposing read (lane -> key row 4 h + j16 / 4 of the 16-key step,
  // +8 for the second read; columns 32 j + 16 (g4 % 2) + 4 (j16 % 4) .. +4).
  const int tr_row = 4 * h + ((lane & 15) >> 2), tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int ch0 = tr_col >> 3, off = (tr_col & 7) * 2;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      u32x4 pf;
#pragma unroll
      for (int d = 0; d < 4; ++d) pf[d] = pack2<DT>(p[i][8 * u + 2 * d], p[i][8 * u + 2 * d + 1]);
      const uint8_t* row0 = vs + (32 * i + 16 * u + tr_row) * 256 + off;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* p0 = row0 + (((4 * j + ch0) ^ tr_row) << 4);
        const uint8_t* p1 = row0 + 8 * 256 + (((4 * j + ch0) ^ (tr_row + 8)) << 4);
        const attn_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) attn_s16x4*)p0);
        const attn_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) attn_s16x4*)p1);
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        acc_o[j] = mfma16<DT>(u32x4{l2[0], l2[1], h2[0], h2[1]}, pf, acc_o[j]);
      }
    }
}

template <int DT>
__global__ void __launch_bounds__(256, 2) attention16_d128_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_d128[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int nqb = (a.T + 127) / 128;
  const int bhn = a.Z * a.H;
  int qb = nqb - 1 - (int)blockIdx.x / bhn, bh = (int)blockIdx.x % bhn;  // causal: heaviest first over all heads
  if (!a.causal) xcd_block_of((int)(blockIdx.y * gridDim.x + blockIdx.x), nqb, bhn, qb, bh);
  const int z = bh / a.H, hd = bh % a.H;
  const int q0 = qb * 128, wq0 = q0 + 32 * wave;
  const bool wave_valid = wq0 < a.T;

  const uint16_t* Q = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)z * a.sq.z + (int64_t)hd * a.sq.h;
  const uint16_t* K = reinterpret_cast<const uint16_t*>(a.k) + (int64_t)z * a.sk.z + (int64_t)hd * a.sk.h;
  const uint16_t* V = reinterpret_cast<const uint16_t*>(a.v) + (int64_t)z * a.sv.z + (int64_t)hd * a.sv.h;
  uint16_t* O = reinterpret_cast<uint16_t*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h;

  Attn128Ctx c;
  c.wave = wave;
  c.k_base = K;
  c.v_base = V;
  c.k_row = a.sk.t;
  c.v_row = a.sv.t;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int key = (4 * i + wave) * 4 + (lane >> 4);  // the row this lane fills, chunk lane % 16
    const int gc = (lane & 15) ^ (key & 15);
    c.key_local[i] = key;
    c.chunk_bytes[i] = 16 * gc;
  }
  u32x4 qf[8];
  {
    const int row = min(wq0 + r32, a.T - 1);
#pragma unroll
    for (int sd = 0; sd < 8; ++sd) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(Q + (int64_t)row * a.sq.t + 16 * sd + 8 * h);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        qf[sd][e] = pack2<DT>(unpack_lo<DT>(raw[e]) * a.scale_log2e, unpack_hi<DT>(raw[e]) * a.scale_log2e);
    }
  }
  f32x16 acc_o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_o[j][v] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  f32x16 neg_m;
#pragma unroll
  for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
  asm volatile("" : "+v"(neg_m));

  const int kv_end = a.causal ? min(a.T, q0 + 128) : a.T;
  const int ntiles = (kv_end + kKvTile - 1) / kKvTile;
  attn128_issue(c, 0, a.T, smem_d128);
  for (int jt = 0; jt < ntiles; ++jt) {
    // The tile's 8 loads per lane have had a whole tile's time; one asm block, because a
    // __syncthreads() would add a fence of its own.
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    const int j0 = jt * kKvTile;
    const bool active = wave_valid && (!a.causal || j0 <= wq0 + 31);
    attn128_tile<DT>(c, a, qf, acc_o, m_run, l_run, neg_m, smem_d128 + (jt & 1) * kD128StageBytes,
                     smem_d128 + ((jt + 1) & 1) * kD128StageBytes, jt + 1, jt + 1 < ntiles, j0, wq0, active, lane);
  }
  if (!wave_valid) return;
  const float inv_l = 1.0f / halfwave_sum(l_run);
  if (wq0 + r32 >= a.T) return;
  uint16_t* orow = O + (int64_t)(wq0 + r32) * a.so.t;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w = {pack2<DT>(acc_o[j][4 * g] * inv_l, acc_o[j][4 * g + 1] * inv_l),
                 pack2<DT>(acc_o[j][4 * g + 2] * inv_l, acc_o[j][4 * g + 3] * inv_l)};
      *reinterpret_cast<u32x2*>(orow + 32 * j + 8 * g + 4 * h) = w;
    }
}

template <int DT>
static int attention16_d128_launch(const AttnArgs& a, hipStream_t s) {
  constexpr size_t lds = 2 * kD128StageBytes;
  auto kern = attention16_d128_kernel<DT>;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int nqb = (a.T + 127) / 128;
  const dim3 grid = a.causal ? dim3(nqb * a.Z * a.H) : dim3(nqb, a.Z * a.H);
  LH_LAUNCH(kern, grid, dim3(256), lds, s, a);
  return check_launch("attention16_d128");
}

template <int DT, int DB, int ROWS = kRowsExact>
static int attention16_anyd_launch(const AttnArgs& a, hipStream_t s) {
  constexpr int D = 32 * DB;
  constexpr size_t lds = (size_t)2 * kKvTile * (D + 8) * 2 + (DB >= 8 ? 4 * 32 * D * 2 : 0);
  auto kern = attention16_anyd_kernel<DT, DB, ROWS>;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int nqb = (a.T + 127) / 128;
  const dim3 grid = a.causal ? dim3(nqb * a.Z * a.H) : dim3(nqb, a.Z * a.H);
  LH_LAUNCH(kern, grid, dim3(256), lds, s, a);
  return check_launch("attention16_anyd");
}

// `chunks`: rows are 16-byte aligned and d is a multiple of 8.  Returns 1 when d is out of range.
template <int DT>
static int attention16_anyd_dispatch(const AttnArgs& a, int d, bool chunks, hipStream_t s) {
  if (d < 1 || d > 256) return 1;
  if (chunks) {
    switch (d) {
      case 32: return attention16_anyd_launch<DT, 1>(a, s);
      case 96: return attention16_anyd_launch<DT, 3>(a, s);
      case 128: return attention16_d128_launch<DT>(a, s);
      case 192: return attention16_anyd_launch<DT, 6>(a, s);
      case 256: return attention16_anyd_launch<DT, 8>(a, s);
      default: break;
    }
    // Other multiples of 8: the next instantiated width, the columns from d on masked.
    if (d < 32) return attention16_anyd_launch<DT, 1, kRowsChunks>(a, s);
    if (d < 64) return attention16_anyd_launch<DT, 2, kRowsChunks>(a, s);
    if (d < 96) return attention16_anyd_launch<DT, 3, kRowsChunks>(a, s);
    if (d < 128) return attention16_anyd_launch<DT, 4, kRowsChunks>(a, s);
    if (d < 192) return attention16_anyd_launch<DT, 6, kRowsChunks>(a, s);
    return attention16_anyd_launch<DT, 8, kRowsChunks>(a, s);
  }
  // Any other head dimension or alignment: the same kernels with element loads and stores.
  if (d <= 32) return attention16_anyd_launch<DT, 1, kRowsElements>(a, s);
  if (d <= 64) return attention16_anyd_launch<DT, 2, kRowsElements>(a, s);
  if (d <= 96) return attention16_anyd_launch<DT, 3, kRowsElements>(a, s);
  if (d <= 128) return attention16_anyd_launch<DT, 4, kRowsElements>(a, s);
  if (d <= 192) return attention16_anyd_launch<DT, 6, kRowsElements>(a, s);
  return attention16_anyd_launch<DT, 8, kRowsElements>(a, s);
}

int attention16_anyd(const AttnArgs& a, int d, int dtype, bool chunks, hipStream_t s) {
  if (dtype == LH_BF16) return attention16_anyd_dispatch<LH_BF16>(a, d, chunks, s);
  if (dtype == LH_F16) return attention16_anyd_dispatch<LH_F16>(a, d, chunks, s);
  return 1;
}

// f32 tensors (all of Q, K, V and the output f32; v_mfma_f32_32x32x2_f32, D = 32 DB columns): the
// structure of attention16_anyd_kernel, with P kept in f32.  A workgroup owns 128 query rows
// (4 waves x 32); K and V tiles of 64 keys are copied through registers into LDS rows of D + 8
// floats (with that pad the V reads of the two half waves, 4 key rows apart, fall on different
// banks), two barriers per tile.  The copy is not overlapped with the arithmetic of the same
// workgroup: a tile is 2 D MFMAs of 64 cycles per wave, and up to D = 128 a second workgroup on
// the CU computes meanwhile.  (For D = 64 a kernel that streamed the tiles by LDS-DMA one tile ahead
// into a second stage measured 1.5 to 3.5 % slower than this one, [4,16,2048,64] 612 against 600 us,
// and is gone.)  Scores are scaled in f32 after the product (exp(x) as exp2(x log2 e): v_exp_f32 is
// accurate to about 1 ulp and the scaled argument, |x| < 100, to 1e-5 absolute, well inside the f32
// tolerance of the payload); the statistics follow the plain online-softmax recurrence.  Q
// fragments live in registers up to D = 96; above, each tile re-reads them from global memory
// (32 KiB per wave at most, cache hits) and the registers go to the output accumulators.  Any
// sequence length: keys past the end are loaded from the last key and masked, rows past the end are
// computed on the last row and not stored.
// ROWS != kRowsExact: the head dimension a.d lies below D (or the rows are not 16-byte aligned); the
// columns of Q, K and V from a.d on are zeros, and output columns from a.d on are not stored.
template <int DB, int ROWS>
__global__ void __launch_bounds__(256, (DB <= 4 ? 2 : 1)) attention32_anyd_kernel(AttnArgs a) {
  constexpr int D = 32 * DB;
  constexpr int KROW = D + 8;  // floats per LDS row
  const int d_real = ROWS != kRowsExact ? a.d : D;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem_anyd32[];
  float* Ks = reinterpret_cast<float*>(smem_anyd32);  // [64][KROW]
  float* Vs = Ks + kKvTile * KROW;                    // [64][KROW]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int nqb = (a.T + kQBlock - 1) / kQBlock;
  // Causal blocks heaviest first; where two (three) workgroups fit a CU, a grid of up to two (three) per
  // CU is resident at once and is dealt so that the CUs' sums stay level.
  const int bhn = a.Z * a.H;
  int qb = nqb - 1 - (int)blockIdx.x / bhn, bh = (int)blockIdx.x % bhn;
  if (!a.causal) xcd_block_of((int)(blockIdx.y * gridDim.x + blockIdx.x), nqb, bhn, qb, bh);
  else if constexpr (DB <= 4) causal_block_of(blockIdx.x, gridDim.x, a.cus, nqb, bhn, qb, bh, DB <= 2);
  const int z = bh / a.H, hd = bh % a.H;
  const int q0 = qb * kQBlock, wq0 = q0 + 32 * wave;
  const bool wave_valid = wq0 < a.T;

  const float* Q = reinterpret_cast<const float*>(a.q) + (int64_t)z * a.sq.z + (int64_t)hd * a.sq.h;
  const float* K = reinterpret_cast<const float*>(a.k) + (int64_t)z * a.sk.z + (int64_t)hd * a.sk.h;
  const float* V = reinterpret_cast<const float*>(a.v) + (int64_t)z * a.sv.z + (int64_t)hd * a.sv.h;
  float* O = reinterpret_cast<float*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h;

  // Lane (q = r32, half h) holds Q[q][8 kk + 4 h + t], kk = 0 .. D / 8 - 1, t = 0 .. 3.
  const float* qrow = Q + (int64_t)min(wq0 + r32, a.T - 1) * a.sq.t;
  auto q_fragment = [&](const float* qrow, int kk, int d) -> f32x4 { return row_chunk32<ROWS>(qrow, 8 * kk + 4 * h, d); };
  constexpr bool Q_REGS = DB <= 3;
  f32x4 qf[Q_REGS ? D / 8 : 1];
  if constexpr (Q_REGS) {
#pragma unroll
    for (int kk = 0; kk < D / 8; ++kk) qf[kk] = q_fragment(qrow, kk, d_real);
  }

  f32x16 acc_o[DB];
#pragma unroll
  for (int j = 0; j < DB; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_o[j][v] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  constexpr int CPR = D / 4;                           // 16-byte chunks per key row
  constexpr int RPP = 256 / CPR;                       // key rows per pass of the 256 threads
  constexpr int NPASS = (kKvTile + RPP - 1) / RPP;
  const int row0 = tid / CPR, ch = tid % CPR;
  const bool loader = row0 < RPP;  // (256 is no multiple of CPR for some D: the last threads copy nothing)
  const int kv_end = a.causal ? min(a.T, q0 + kQBlock) : a.T;
  const int ntiles = (kv_end + kKvTile - 1) / kKvTile;
  for (int jt = 0; jt < ntiles; ++jt) {
    const int j0 = jt * kKvTile;
    __syncthreads();  // the previous tile has been consumed
    // (opaque per tile: the masks and clamped columns that depend on it are formed where they are used
    // and not kept in registers across the loop)
    int d_tile = d_real;
    if constexpr (ROWS != kRowsExact) asm volatile("" : "+s"(d_tile));
    // D / 4 16-byte chunks per key row: thread (row0, ch) copies chunk ch of rows row0, row0 + RPP, ...
    // (a thread's column, and whether it lies inside the head dimension, never change).
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      const int key = pass * RPP + row0;
      if (loader && ((pass + 1) * RPP <= kKvTile || key < kKvTile)) {
        const int kg = min(j0 + key, a.T - 1);
        const f32x4 kv = row_chunk32<ROWS>(K + (int64_t)kg * a.sk.t, 4 * ch, d_tile);
        const f32x4 vv = row_chunk32<ROWS>(V + (int64_t)kg * a.sv.t, 4 * ch, d_tile);
        *reinterpret_cast<f32x4*>(Ks + key * KROW + 4 * ch) = kv;
        *reinterpret_cast<f32x4*>(Vs + key * KROW + 4 * ch) = vv;
      }
      // (at most 8 passes, 64 registers, in flight; 2 passes, 16 loads, when they are element loads)
      if (pass % 8 == 7 || (ROWS == kRowsElements && pass % 2 == 1)) asm volatile("" ::: "memory");
    }
    __syncthreads();
    if (!wave_valid || (a.causal && j0 > wq0 + 31)) continue;
    f32x16 s_acc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) s_acc[i][v] = 0.0f;
    // (the address is opaque per tile: the loads stay inside the loop and the fragments out of registers)
    const float* qrow_tile = qrow;
    if constexpr (!Q_REGS) asm volatile("" : "+v"(qrow_tile));
    // The two key sub-tiles alternate so that consecutive MFMAs never depend on each other.
#pragma unroll
    for (int kk = 0; kk < D / 8; ++kk) {
      f32x4 q4;
      if constexpr (Q_REGS) q4 = qf[kk];
      else q4 = q_fragment(qrow_tile, kk, d_tile);
      if constexpr (!Q_REGS) {
        // (no more than 4 fragments fetched ahead; 2 when they are element loads)
        if (kk % 4 == 3 || (ROWS == kRowsElements && kk % 2 == 1)) asm volatile("" ::: "memory");
      }
      f32x4 kf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) kf[i] = *reinterpret_cast<const f32x4*>(Ks + (32 * i + r32) * KROW + 8 * kk + 4 * h);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 2; ++i) s_acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[i][t], q4[t], s_acc[i], 0, 0, 0);
    }
    // s_acc[i][v] = S[q = wq0 + r32][key = j0 + 32 i + 8 (v / 4) + 4 h + v % 4] (unscaled)
    if ((a.causal && j0 + kKvTile - 1 > wq0) || j0 + kKvTile > a.T) {
      // last visible key of the row: its own index under the causal mask, and never past the end
      const int last = a.causal ? min(wq0 + r32, a.T - 1) : a.T - 1;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (j0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3) > last) s_acc[i][v] = -INFINITY;
    }
    float mx = fmaxf(s_acc[0][0], s_acc[1][0]);
#pragma unroll
    for (int v = 1; v < 16; ++v) mx = fmaxf(fmaxf(mx, s_acc[0][v]), s_acc[1][v]);
    mx = halfwave_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
    const float alpha = exp2_fast((m_run - m_safe) * a.scale_log2e);
    const float mc = m_safe * a.scale_log2e;
    float l_tile = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s_acc[i][v] = exp2_fast(s_acc[i][v] * a.scale_log2e - mc);
        l_tile += s_acc[i][v];
      }
    l_run = l_run * alpha + l_tile;
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < DB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc_o[j][v] *= alpha;
    // O^T += V^T P^T, one key pair per MFMA: lane (d = r32, half h) reads V[key][32 j + r32].
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float* vrow = Vs + (32 * i + 8 * (v >> 2) + 4 * h + (v & 3)) * KROW + r32;
#pragma unroll
        for (int j = 0; j < DB; ++j)
          acc_o[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * j], s_acc[i][v], acc_o[j], 0, 0, 0);
        if (v % 4 == 3) asm volatile("" ::: "memory");  // (V fragments of 4 keys fetched ahead, not of all 64)
      }
  }
  // acc_o[j][v] = O[q = wq0 + r32][d = 32 j + 8 (v / 4) + 4 h + v % 4] * l
  if (!wave_valid) return;
  const float inv_l = 1.0f / halfwave_sum(l_run);
  if (wq0 + r32 >= a.T) return;  // (after the cross-lane sum, which needs every lane)
  float* orow = O + (int64_t)(wq0 + r32) * a.so.t;
#pragma unroll
  for (int j = 0; j < DB; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 w = {acc_o[j][4 * g] * inv_l, acc_o[j][4 * g + 1] * inv_l, acc_o[j][4 * g + 2] * inv_l,
                       acc_o[j][4 * g + 3] * inv_l};
      store_chunk32<ROWS>(orow, 32 * j + 8 * g + 4 * h, d_real, w);
    }
}

template <int DB, int ROWS>
static int attention32_anyd_launch(const AttnArgs& a, hipStream_t s) {
  constexpr size_t lds = (size_t)2 * kKvTile * (32 * DB + 8) * 4;
  auto kern = attention32_anyd_kernel<DB, ROWS>;
  static bool configured = false;
  if (!configured && !planning()) {
    LH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    configured = true;
  }
  const int nqb = (a.T + kQBlock - 1) / kQBlock;
  const dim3 grid = a.causal ? dim3(nqb * a.Z * a.H) : dim3(nqb, a.Z * a.H);
  LH_LAUNCH(kern, grid, dim3(256), lds, s, a);
  return check_launch("attention32_anyd");
}

template <int DB>
static int attention32_anyd_rows(const AttnArgs& a, int d, bool chunks, hipStream_t s) {
  if (!chunks) return attention32_anyd_launch<DB, kRowsElements>(a, s);
  if (d != 32 * DB) return attention32_anyd_launch<DB, kRowsChunks>(a, s);
  return attention32_anyd_launch<DB, kRowsExact>(a, s);
}

// f32 tensors on the kernel above.  `chunks`: rows are 16-byte aligned and d is a multiple of 4.
// Returns 1 when d is out of range.
int attention32_anyd(const AttnArgs& a, int d, bool chunks, hipStream_t s) {
  if (d < 1 || d > 256) return 1;
  switch ((d + 31) / 32) {
    case 1: return attention32_anyd_rows<1>(a, d, chunks, s);
    case 2: return attention32_anyd_rows<2>(a, d, chunks, s);
    case 3: return attention32_anyd_rows<3>(a, d, chunks, s);
    case 4: return attention32_anyd_rows<4>(a, d, chunks, s);
    case 5: return attention32_anyd_rows<5>(a, d, chunks, s);
    case 6: return attention32_anyd_rows<6>(a, d, chunks, s);
    case 7: return attention32_anyd_rows<7>(a, d, chunks, s);
    default: return attention32_anyd_rows<8>(a, d, chunks, s);
  }
}

constexpr int kMaxHeadDim = 256;

int attention_launch(const AttnArgs& a, int dtype, hipStream_t s) {
  if (dtype == LH_BF16) return attention16_launch<LH_BF16>(a, s);
  return attention16_launch<LH_F16>(a, s);
}

}  // namespace lh

using namespace lh;

// `ws`: the call's temporary memory comes from this workspace (nullptr: from the stream's pool, unless
// a NoAttentionScratchScope forbids that).
static int attention_run(void* out, const void* q, const void* k, const void* v, int64_t Z, int64_t H, int64_t T,
                         int64_t d, lh_strides3 so, lh_strides3 sq, lh_strides3 sk, lh_strides3 sv, float scale,
                         int32_t causal, int32_t dtype, void* stream, Scratch* ws) {
  LH_REQUIRE(out && q && k && v, "lh_hip_attention: null pointer");
  LH_REQUIRE(dtype == LH_BF16 || dtype == LH_F16 || dtype == LH_F32, "lh_hip_attention: unsupported dtype %d", dtype);
  LH_REQUIRE(Z > 0 && H > 0 && T > 0, "lh_hip_attention: empty problem Z=%lld H=%lld T=%lld", (long long)Z,
             (long long)H, (long long)T);
  if (d < 1 || d > kMaxHeadDim)
    return fail(LH_ERR_UNSUPPORTED, "lh_hip_attention: head_dim %lld not supported (1 .. %d)", (long long)d, kMaxHeadDim);
  LH_REQUIRE(Z * H <= 65535 && T < (1 << 30), "lh_hip_attention: problem too large");
  const lh_strides3* ss[4] = {&so, &sq, &sk, &sv};
  const void* ps[4] = {out, q, k, v};
  for (int i = 0; i < 4; ++i) LH_REQUIRE(ss[i]->t >= d, "lh_hip_attention: row stride of tensor %d is below head_dim", i);
  // The streaming kernels need 16-bit tensors, head_dim 64 and 16-byte aligned rows; the register-copy
  // kernels take every other problem, with 16-byte accesses where rows and head_dim allow them.
  const int vec = (dtype == LH_F32) ? 4 : 8;  // elements per 16-byte access
  // (the kernels mask a partial last key tile and skip rows past the end themselves)
  bool aligned = true, near = true;
  for (int i = 0; i < 4; ++i) {
    aligned = aligned && ss[i]->t % vec == 0 && ss[i]->h % vec == 0 && ss[i]->z % vec == 0 && aligned16(ps[i]);
    near = near && ss[i]->t < (1 << 24);  // (the streaming kernels address a key tile's rows with 32-bit byte offsets)
  }
  const bool fast = aligned && near && d == kHeadDim && dtype != LH_F32;
  if (scale <= 0.0f) scale = 1.0f / sqrtf((float)d);
  AttnArgs a;
  a.out = out; a.q = q; a.k = k; a.v = v;
  a.Z = (int)Z; a.H = (int)H; a.T = (int)T;
  a.so = so; a.sq = sq; a.sk = sk; a.sv = sv;
  a.scale = scale;
  a.scale_log2e = scale * 1.4426950408889634f;
  a.d = (int)d;
  a.ws = ws;
  a.allow_grid_split = ws != nullptr || attention_scratch_allowed();
  LH_REQUIRE((causal & ~(int32_t)(LH_ATTN_CAUSAL | LH_ATTN_ROWS_MASK | LH_ATTN_STAGES_MASK | LH_ATTN_KSPLIT_MASK |
                                  LH_ATTN_SCALE_F32)) == 0 &&
                 (causal & LH_ATTN_ROWS_MASK) != LH_ATTN_ROWS_MASK && (causal & LH_ATTN_STAGES_MASK) != LH_ATTN_STAGES_MASK &&
                 (causal & LH_ATTN_KSPLIT_MASK) != LH_ATTN_KSPLIT_MASK,
             "lh_hip_attention: unknown bits 0x%x in the causal / request word", causal);
  a.causal = (causal & LH_ATTN_CAUSAL) ? 1 : 0;
  a.request = causal & (LH_ATTN_ROWS_MASK | LH_ATTN_STAGES_MASK | LH_ATTN_KSPLIT_MASK);
  a.scale_f32 = (causal & LH_ATTN_SCALE_F32) != 0;
  LH_REQUIRE((a.request == 0 && !a.scale_f32) || fast,
             "lh_hip_attention: query-row / ring-depth / score-scaling requests apply to 16-bit tensors with head_dim %d "
             "and aligned rows", kHeadDim);
  a.cus = num_cus();
  if (!fast) {
    const hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const bool chunks = aligned && d % vec == 0;
    const int rc = dtype == LH_F32 ? attention32_anyd(a, (int)d, chunks, st) : attention16_anyd(a, (int)d, dtype, chunks, st);
    if (rc > 0) return fail(LH_ERR_UNSUPPORTED, "lh_hip_attention: no kernel for head_dim %lld", (long long)d);
    return rc;
  }
  return attention_launch(a, dtype, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int lh_hip_attention(void* out, const void* q, const void* k, const void* v, int64_t Z, int64_t H,
                                int64_t T, int64_t d, lh_strides3 so, lh_strides3 sq, lh_strides3 sk, lh_strides3 sv,
                                float scale, int32_t causal, int32_t dtype, void* stream) {
  return attention_run(out, q, k, v, Z, H, T, d, so, sq, sk, sv, scale, causal, dtype, stream, nullptr);
}

extern "C" size_t lh_hip_attention_workspace_bytes(int64_t Z, int64_t H, int64_t T, int64_t d, lh_strides3 so,
                                                   lh_strides3 sq, lh_strides3 sk, lh_strides3 sv, int32_t causal,
                                                   int32_t dtype) {
  PlanningScope plan;
  Scratch ws;
  void* const fake = reinterpret_cast<void*>(uintptr_t(1) << 20);
  const int rc = attention_run(fake, fake, fake, fake, Z, H, T, d, so, sq, sk, sv, 0.0f, causal, dtype, nullptr, &ws);
  return rc ? 0 : ws.need;
}

extern "C" int lh_hip_attention_ws(void* out, const void* q, const void* k, const void* v, int64_t Z, int64_t H,
                                   int64_t T, int64_t d, lh_strides3 so, lh_strides3 sq, lh_strides3 sk,
                                   lh_strides3 sv, float scale, int32_t causal, int32_t dtype, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  LH_REQUIRE(workspace != nullptr || workspace_bytes == 0, "lh_hip_attention_ws: null workspace of %zu bytes",
             workspace_bytes);
  LH_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, "lh_hip_attention_ws: workspace must be 256-byte aligned");
  Scratch ws;
  // An empty workspace still must not fall back to the pool: the base stays non-null.
  ws.base = workspace ? static_cast<char*>(workspace) : reinterpret_cast<char*>(uintptr_t(256));
  ws.bytes = workspace_bytes;
  return attention_run(out, q, k, v, Z, H, T, d, so, sq, sk, sv, scale, causal, dtype, stream, &ws);
}
