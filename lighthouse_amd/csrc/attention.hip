// Fused attention forward for gfx950: O = softmax(Q K^T * scale [+ causal mask]) V, one
// kernel, never materialising the T x T scores.  Algorithm and rounding points follow
// ReplaceWithFusedAttentionOp (lighthouse/dialects/transform/transform_ext/ops/
// replace_with_fused_attention.py:332-455): running max m, running sum l and the output
// accumulator live in f32; P is rounded to the element type before P.V; the row sum uses
// the unrounded P; the output is acc / l rounded to the element type.
//
// Work split: a workgroup owns 128 query rows of one (batch, head); each of its 4 waves owns
// 32 rows.  K/V tiles of 64 keys are staged through LDS (double buffered, one barrier per
// tile) and shared by the 4 waves.
//
// Both products are computed TRANSPOSED on the matrix cores: S^T = K Q^T and O^T = V^T P^T.
// With the 32x32 MFMA accumulator layout a lane then owns ONE query row (column of S^T) and
// 16 of its keys per tile, so the row max / row sum are register reductions plus a single
// exchange between the two half-waves, the softmax state (m, l, alpha) is one scalar per
// lane, and the S^T accumulator registers, converted to 16 bit, ARE the second operand of
// the V^T P^T product (no LDS round trip or cross-lane shuffle for P).  V is transposed in
// registers on its way into LDS, with the keys of every group of 16 stored in the order the
// accumulator layout produces them.
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
constexpr int kQBlock = 128;
constexpr int kAttnStride = 72;  // 16-bit elements per LDS row (64 + 8 pad)

template <int DT>
__global__ void __launch_bounds__(256) attention16_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][kKvTile * kAttnStride];   // [key][d]
  __shared__ __attribute__((aligned(16))) uint16_t Vts[2][kHeadDim * kAttnStride];  // [d][key slot]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, h = lane >> 5;
  const int nqb = a.T / kQBlock;
  // Causal: the last query blocks have the most key tiles; start them first.
  const int qb = a.causal ? (nqb - 1 - (int)blockIdx.x) : (int)blockIdx.x;
  const int bh = blockIdx.y;
  const int z = bh / a.H, hd = bh % a.H;
  const int q0 = qb * kQBlock;
  const int wq0 = q0 + wave * 32;

  const uint16_t* Q = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)z * a.sq.z + (int64_t)hd * a.sq.h;
  const uint16_t* K = reinterpret_cast<const uint16_t*>(a.k) + (int64_t)z * a.sk.z + (int64_t)hd * a.sk.h;
  const uint16_t* V = reinterpret_cast<const uint16_t*>(a.v) + (int64_t)z * a.sv.z + (int64_t)hd * a.sv.h;
  uint16_t* O = reinterpret_cast<uint16_t*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h;

  // Q fragment: second MFMA operand of S^T = K Q^T; lane (q = r32, half h) holds
  // Q[q][16s + 8h .. +8] for the 4 k-steps s over the head dimension.
  u32x4 qf[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
    qf[s] = *reinterpret_cast<const u32x4*>(Q + (int64_t)(wq0 + r32) * a.sq.t + 16 * s + 8 * h);

  // Global -> register staging of one K/V tile.
  u32x4 rk[2];
  u32x2 rv[4];
  const int k_row = tid >> 3, k_chunk = tid & 7;  // + 32 rows for the second chunk
  const int v_dgrp = tid & 15, v_kq = tid >> 4;   // 4 keys x 4 d per thread
  auto load_tile = [&](int j0) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      rk[i] = *reinterpret_cast<const u32x4*>(K + (int64_t)(j0 + k_row + 32 * i) * a.sk.t + k_chunk * 8);
#pragma unroll
    for (int r = 0; r < 4; ++r)
      rv[r] = *reinterpret_cast<const u32x2*>(V + (int64_t)(j0 + 4 * v_kq + r) * a.sv.t + v_dgrp * 4);
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      *reinterpret_cast<u32x4*>(&Ks[buf][(k_row + 32 * i) * kAttnStride + k_chunk * 8]) = rk[i];
    // Keys 4*kq .. 4*kq+3 of this thread go to slot 16*(kq/4) + 8*(kq%2) + 4*((kq%4)/2) + r:
    // within each group of 16 keys the order is the one the S^T accumulator produces.
    const int slot = 16 * (v_kq >> 2) + 8 * (v_kq & 1) + 4 * ((v_kq & 3) >> 1);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
      u32x2 w;
      w[0] = __builtin_amdgcn_perm(rv[1][c >> 1], rv[0][c >> 1], sel);
      w[1] = __builtin_amdgcn_perm(rv[3][c >> 1], rv[2][c >> 1], sel);
      *reinterpret_cast<u32x2*>(&Vts[buf][(v_dgrp * 4 + c) * kAttnStride + slot]) = w;
    }
  };

  f32x16 acc_o[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_o[j][v] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const int kv_end = a.causal ? min(a.T, q0 + kQBlock) : a.T;
  const int ntiles = (kv_end + kKvTile - 1) / kKvTile;
  load_tile(0);
  store_tile(0);
  __syncthreads();

  for (int jt = 0; jt < ntiles; ++jt) {
    const int buf = jt & 1;
    const int j0 = jt * kKvTile;
    if (jt + 1 < ntiles) load_tile(j0 + kKvTile);

    // A wave whose 32 rows all precede this tile has nothing to do in it (causal only).
    const bool active = !a.causal || (j0 <= wq0 + 31);
    if (active) {
      f32x16 s_acc[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s_acc[i][v] = 0.0f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          u32x4 kf = *reinterpret_cast<const u32x4*>(&Ks[buf][(32 * i + r32) * kAttnStride + 16 * s + 8 * h]);
          s_acc[i] = mfma16<DT>(kf, qf[s], s_acc[i]);
        }
      }
      // s_acc[i][v] = S[q = wq0 + r32][key = j0 + 32 i + 8 (v/4) + 4 h + v%4] (unscaled)
      if (a.causal && (j0 + kKvTile - 1 > wq0)) {
        const int qrow = wq0 + r32;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            int key = j0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
            if (key > qrow) s_acc[i][v] = -INFINITY;
          }
      }
      float mx = s_acc[0][0];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s_acc[i][v]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
      const float mc = m_safe * a.scale_log2e;
      const float alpha = exp2f(m_run * a.scale_log2e - mc);
      float l_tile = 0.0f;
      u32x4 pf[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          p[v] = exp2f(s_acc[i][v] * a.scale_log2e - mc);
          l_tile += p[v];
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int d = 0; d < 4; ++d) pf[i][u][d] = pack2<DT>(p[8 * u + 2 * d], p[8 * u + 2 * d + 1]);
      }
      l_run = l_run * alpha + l_tile;
      m_run = m_new;
      if (alpha != 1.0f) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc_o[j][v] *= alpha;
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            u32x4 vf =
                *reinterpret_cast<const u32x4*>(&Vts[buf][(32 * j + r32) * kAttnStride + 32 * i + 16 * u + 8 * h]);
            acc_o[j] = mfma16<DT>(vf, pf[i][u], acc_o[j]);
          }
    }

    if (jt + 1 < ntiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // acc_o[j][v] = O[q = wq0 + r32][d = 32 j + 8 (v/4) + 4 h + v%4] * l
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv_l = 1.0f / l_tot;
  uint16_t* orow = O + (int64_t)(wq0 + r32) * a.so.t;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w = {pack2<DT>(acc_o[j][4 * g] * inv_l, acc_o[j][4 * g + 1] * inv_l),
                 pack2<DT>(acc_o[j][4 * g + 2] * inv_l, acc_o[j][4 * g + 3] * inv_l)};
      *reinterpret_cast<u32x2*>(orow + 32 * j + 8 * g + 4 * h) = w;
    }
}

// f32 variant (all tensors f32, f32 MFMA): same structure; P stays f32, K and V tiles keep
// their global orientation in LDS because the f32 MFMA takes a single value per lane.
constexpr int kAttn32KStride = 68;  // floats per K row (64 + 4): 16-byte reads of 16 rows conflict free
constexpr int kAttn32VStride = 72;  // floats per V row: rows 4 apart land 32 banks apart

__global__ void __launch_bounds__(256) attention32_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) float Ks[kKvTile * kAttn32KStride];
  __shared__ __attribute__((aligned(16))) float Vs[kKvTile * kAttn32VStride];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, h = lane >> 5;
  const int nqb = a.T / kQBlock;
  const int qb = a.causal ? (nqb - 1 - (int)blockIdx.x) : (int)blockIdx.x;
  const int bh = blockIdx.y;
  const int z = bh / a.H, hd = bh % a.H;
  const int q0 = qb * kQBlock;
  const int wq0 = q0 + wave * 32;
  const float* Q = reinterpret_cast<const float*>(a.q) + (int64_t)z * a.sq.z + (int64_t)hd * a.sq.h;
  const float* K = reinterpret_cast<const float*>(a.k) + (int64_t)z * a.sk.z + (int64_t)hd * a.sk.h;
  const float* V = reinterpret_cast<const float*>(a.v) + (int64_t)z * a.sv.z + (int64_t)hd * a.sv.h;
  float* O = reinterpret_cast<float*>(a.out) + (int64_t)z * a.so.z + (int64_t)hd * a.so.h;

  // Lane (q = r32, half h) holds Q[q][8 kk + 4 h + t], kk = 0..7, t = 0..3.
  f32x4 qf[8];
#pragma unroll
  for (int kk = 0; kk < 8; ++kk)
    qf[kk] = *reinterpret_cast<const f32x4*>(Q + (int64_t)(wq0 + r32) * a.sq.t + 8 * kk + 4 * h);

  f32x16 acc_o[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_o[j][v] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int kv_end = a.causal ? min(a.T, q0 + kQBlock) : a.T;

  for (int j0 = 0; j0 < kv_end; j0 += kKvTile) {
    __syncthreads();
    for (int c = tid; c < kKvTile * 16; c += 256) {
      int row = c >> 4, ch = c & 15;
      *reinterpret_cast<f32x4*>(&Ks[row * kAttn32KStride + ch * 4]) =
          *reinterpret_cast<const f32x4*>(K + (int64_t)(j0 + row) * a.sk.t + ch * 4);
      *reinterpret_cast<f32x4*>(&Vs[row * kAttn32VStride + ch * 4]) =
          *reinterpret_cast<const f32x4*>(V + (int64_t)(j0 + row) * a.sv.t + ch * 4);
    }
    __syncthreads();
    const bool active = !a.causal || (j0 <= wq0 + 31);
    if (!active) continue;
    f32x16 s_acc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s_acc[i][v] = 0.0f;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        f32x4 kf = *reinterpret_cast<const f32x4*>(&Ks[(32 * i + r32) * kAttn32KStride + 8 * kk + 4 * h]);
#pragma unroll
        for (int t = 0; t < 4; ++t) s_acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[t], qf[kk][t], s_acc[i], 0, 0, 0);
      }
    }
    if (a.causal && (j0 + kKvTile - 1 > wq0)) {
      const int qrow = wq0 + r32;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          int key = j0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
          if (key > qrow) s_acc[i][v] = -INFINITY;
        }
    }
    float mx = s_acc[0][0];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s_acc[i][v]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
    // f32 path: exact exp (not the exp2 shortcut) to stay within the f32 tolerance.
    const float alpha = expf((m_run - m_safe) * a.scale);
    float l_tile = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s_acc[i][v] = expf((s_acc[i][v] - m_safe) * a.scale);
        l_tile += s_acc[i][v];
      }
    l_run = l_run * alpha + l_tile;
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc_o[j][v] *= alpha;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float vf = Vs[key * kAttn32VStride + 32 * j + r32];
          acc_o[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf, s_acc[i][v], acc_o[j], 0, 0, 0);
        }
      }
  }
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv_l = 1.0f / l_tot;
  float* orow = O + (int64_t)(wq0 + r32) * a.so.t;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 w = {acc_o[j][4 * g] * inv_l, acc_o[j][4 * g + 1] * inv_l, acc_o[j][4 * g + 2] * inv_l,
                 acc_o[j][4 * g + 3] * inv_l};
      *reinterpret_cast<f32x4*>(orow + 32 * j + 8 * g + 4 * h) = w;
    }
}

int attention_launch(const AttnArgs& a, int dtype, hipStream_t s) {
  dim3 grid(a.T / kQBlock, a.Z * a.H);
  if (dtype == LH_BF16) hipLaunchKernelGGL(attention16_kernel<LH_BF16>, grid, dim3(256), 0, s, a);
  else if (dtype == LH_F16) hipLaunchKernelGGL(attention16_kernel<LH_F16>, grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL(attention32_kernel, grid, dim3(256), 0, s, a);
  return check_launch("attention");
}

}  // namespace lh

using namespace lh;

extern "C" int lh_hip_attention(void* out, const void* q, const void* k, const void* v, int64_t Z, int64_t H,
                                int64_t T, int64_t d, lh_strides3 so, lh_strides3 sq, lh_strides3 sk, lh_strides3 sv,
                                float scale, int32_t causal, int32_t dtype, void* stream) {
  LH_REQUIRE(out && q && k && v, "lh_hip_attention: null pointer");
  LH_REQUIRE(dtype == LH_BF16 || dtype == LH_F16 || dtype == LH_F32, "lh_hip_attention: unsupported dtype %d", dtype);
  LH_REQUIRE(Z > 0 && H > 0 && T > 0, "lh_hip_attention: empty problem Z=%lld H=%lld T=%lld", (long long)Z,
             (long long)H, (long long)T);
  if (d != kHeadDim) return fail(LH_ERR_UNSUPPORTED, "lh_hip_attention: head_dim %lld not supported (only 64)", (long long)d);
  if (T % kQBlock != 0)
    return fail(LH_ERR_UNSUPPORTED, "lh_hip_attention: seq_len %lld must be a multiple of %d", (long long)T, kQBlock);
  LH_REQUIRE(Z * H <= 65535 && T < (1 << 30), "lh_hip_attention: problem too large");
  const int vec = (dtype == LH_F32) ? 4 : 8;  // elements per 16-byte access
  const lh_strides3* ss[4] = {&so, &sq, &sk, &sv};
  const void* ps[4] = {out, q, k, v};
  for (int i = 0; i < 4; ++i) {
    LH_REQUIRE(ss[i]->t >= d && ss[i]->t % vec == 0 && ss[i]->h % vec == 0 && ss[i]->z % vec == 0,
               "lh_hip_attention: strides of tensor %d must be multiples of %d elements", i, vec);
    LH_REQUIRE(aligned16(ps[i]), "lh_hip_attention: tensor %d is not 16-byte aligned", i);
  }
  if (scale <= 0.0f) scale = 1.0f / sqrtf((float)d);
  AttnArgs a;
  a.out = out; a.q = q; a.k = k; a.v = v;
  a.Z = (int)Z; a.H = (int)H; a.T = (int)T;
  a.so = so; a.sq = sq; a.sk = sk; a.sv = sv;
  a.scale = scale;
  a.scale_log2e = scale * 1.4426950408889634f;
  a.causal = causal ? 1 : 0;
  return attention_launch(a, dtype, reinterpret_cast<hipStream_t>(stream));
}
