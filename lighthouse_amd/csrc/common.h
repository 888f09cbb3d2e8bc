// Shared declarations for the gfx950 kernels behind liblighthouse_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "lighthouse_hip.h"

namespace lh {

// ---- error reporting -------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

#define LH_HIP_CHECK(expr)                                                                   \
  do {                                                                                       \
    hipError_t _e = (expr);                                                                  \
    if (_e != hipSuccess)                                                                    \
      return ::lh::fail(LH_ERR_RUNTIME, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                        __FILE__, __LINE__);                                                 \
  } while (0)

#define LH_REQUIRE(cond, ...)                                 \
  do {                                                        \
    if (!(cond)) return ::lh::fail(LH_ERR_INVALID, __VA_ARGS__); \
  } while (0)

bool planning();
inline int check_launch(const char* what) {
  if (planning()) return LH_OK;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(LH_ERR_RUNTIME, "launch of %s failed: %s", what, hipGetErrorString(e));
  return LH_OK;
}

inline size_t dtype_size(int32_t dt) {
  switch (dt) {
    case LH_F32: return 4;
    case LH_BF16: return 2;
    case LH_F16: return 2;
    case LH_F8E4M3: return 1;
    case LH_F64: return 8;
    case LH_I8: return 1;
    case LH_I16: return 2;
    case LH_I32: return 4;
    case LH_I64: return 8;
    default: return 0;
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- vector types ------------------------------------------------------------
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x8 __attribute__((ext_vector_type(8)));

// ---- scalar conversions (device) ----------------------------------------------
// float -> bfloat16 bits, round to nearest even, quiet NaN (arith.truncf semantics).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return (float)__builtin_bit_cast(_Float16, b);
}

// Pack two floats into one dword of two 16-bit values (lo = a, hi = b), round to nearest
// even; one v_cvt_pk_bf16_f32 for bf16.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
  f32x2 v = {a, b};
  if constexpr (DT == LH_BF16) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  } else {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
}
template <int DT>
__device__ __forceinline__ float unpack_lo(uint32_t w) {
  if constexpr (DT == LH_BF16) return __builtin_bit_cast(float, w << 16);
  else return f16_bits_to_f32((uint16_t)(w & 0xffffu));
}
template <int DT>
__device__ __forceinline__ float unpack_hi(uint32_t w) {
  if constexpr (DT == LH_BF16) return __builtin_bit_cast(float, w & 0xffff0000u);
  else return f16_bits_to_f32((uint16_t)(w >> 16));
}

// Load / store one element of a run-time-typed buffer as float.
template <int DT>
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i) {
  if constexpr (DT == LH_F32) return reinterpret_cast<const float*>(p)[i];
  else if constexpr (DT == LH_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  else return f16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
}
template <int DT>
__device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v) {
  if constexpr (DT == LH_F32) reinterpret_cast<float*>(p)[i] = v;
  else if constexpr (DT == LH_BF16) reinterpret_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else reinterpret_cast<uint16_t*>(p)[i] = f32_to_f16_bits(v);
}
// Round a float to the named type and back (the rounding point of a conversion).
template <int DT>
__device__ __forceinline__ float round_through(float v) {
  if constexpr (DT == LH_F32) return v;
  else if constexpr (DT == LH_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  else return f16_bits_to_f32(f32_to_f16_bits(v));
}

// arith.maximumf(x, 0): NaN propagates (lighthouse/ingress/mlir_gen/named.py:28-32).
__device__ __forceinline__ float relu_nan(float v) { return (v != v) ? v : fmaxf(v, 0.0f); }

// tanh-GELU, 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))), via one exp:
// 0.5 (1 + tanh(u)) = 1 / (1 + exp(-2u)).
// exp(-2u) = exp2(x (c + 0.044715 c x^2)) with c = -2 sqrt(2/pi) log2(e); the quotient uses the
// hardware reciprocal (1 ulp).  7 instructions per element.
__device__ __forceinline__ float gelu_tanh(float x) {
  const float c = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x * x, 0.044715f * c, c));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// The lane's index in its wave, recomputed from the execution mask at the point of the call (the
// opaque zero keeps the compiler from computing it once and holding it in a register).  Persistent
// kernels use it for per-tile address setup so that lane-dependent offsets do not stay live, or
// get spilled, across a register-bound main loop.  Requires all 64 lanes active.
__device__ __forceinline__ int lane_now() {
  int zero = 0;
  asm volatile("" : "+v"(zero));
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, zero));
}

// Workgroup id -> tile id so that the workgroups resident on one XCD (ids congruent
// modulo 8 are dispatched to the same XCD) cover a compact patch of tiles and share
// their operand panels through that XCD's L2.
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
  const int nx = 8;
  if (nblocks % nx != 0) return bid;
  int per = nblocks / nx;
  return (bid % nx) * per + bid / nx;
}

hipStream_t default_stream();
// out[c][r] = in[r][c] for an R x C matrix of 2- or 4-byte elements (row strides in elements).
int transpose_matrix(void* out, const void* in, int R, int C, int64_t ld_in, int64_t ld_out, int elem_bytes,
                     hipStream_t s);
// dst (rows_dst x cols_dst) = src (rows_src x cols_src) padded with zeros or cut; any alignment.
int pad_copy_matrix(void* dst, int64_t ld_dst, int rows_dst, int cols_dst, const void* src, int64_t ld_src, int rows_src,
                    int cols_src, int elem_bytes, hipStream_t s);

// ---- temporary device memory of a call ------------------------------------------------------
// Kernels that need memory beyond their operands (transposed or zero-padded operand copies, the
// f32 blocks of a launch cut along K, hidden activations of the MLP payload) take it from a Scratch:
//  * base != nullptr: a workspace the caller handed in, given out front to back in 256-byte
//    granules; a request that does not fit fails with LH_ERR_INVALID and nothing is allocated;
//  * base == nullptr (or no Scratch at all): the library's pool, one buffer per purpose ("slot")
//    and per (device, stream), so that calls on different streams never share memory.  A buffer
//    that is too small is replaced by a larger one; the old one is kept until
//    lh_hip_release_scratch() because enqueued work may still use it (no hipFree, hence no
//    device-wide synchronisation, inside a call).
// While planning() is true (a *_workspace_bytes query on this thread) nothing is launched or
// allocated: takes return a dummy address and add their size to `need`.
enum ScratchSlot { kScratchTranspose = 0, kScratchPad, kScratchSplitK, kScratchSkinny, kScratchMlp, kScratchAttention, kScratchSlots };
struct Scratch {
  char* base = nullptr;
  size_t bytes = 0;
  size_t used = 0;
  size_t need = 0;
};
int scratch_take(Scratch* ws, hipStream_t s, int slot, size_t bytes, const char* what, void** out);
bool planning();
struct PlanningScope {  // marks the calling thread as running a size query
  PlanningScope();
  ~PlanningScope();
};
// Entry points that run on a caller's workspace only (the nanoGPT block and forward) keep their
// attention launches from taking pool memory: while such a scope is alive on the calling thread,
// lh_hip_attention does not split key ranges between workgroups.
bool attention_scratch_allowed();
struct NoAttentionScratchScope {
  NoAttentionScratchScope();
  ~NoAttentionScratchScope();
};
#define LH_LAUNCH(...)                                        \
  do {                                                        \
    if (!::lh::planning()) hipLaunchKernelGGL(__VA_ARGS__);   \
  } while (0)
// The current device's statically allocated scratch array (runtime.hip): its device address and size.
int static_scratch(char** base, size_t* bytes);
// lh_hip_layer_norm with the choice of store: `streaming` (what the public entry point uses) writes
// the rows with non-temporal stores; a caller whose next kernel reads them at once passes false.
int layer_norm(void* out, const void* x, const float* gamma, const float* beta, int64_t M, int64_t N, float eps,
               int32_t x_dtype, int32_t out_dtype, bool streaming, void* stream);
// Compute units of the current device (cached; 256 if the query fails).
int num_cus();

}  // namespace lh
