// Runtime part of the C ABI: error state, device info, device memory helpers.
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "common.h"

namespace lh {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

hipStream_t default_stream() { return nullptr; }

int num_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

// Transpose through a padded 64 x 64 LDS tile: rows of 64 elements are read and written whole.
template <typename T>
__global__ void __launch_bounds__(256) transpose_tiles(T* out, const T* in, int R, int C, int64_t ld_in, int64_t ld_out) {
  __shared__ T tile[64][65];
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    if (r < R && c < C) tile[i][tx] = in[(int64_t)r * ld_in + c];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, r = r0 + tx;
    if (c < C && r < R) out[(int64_t)c * ld_out + r] = tile[tx][i];
  }
}

// 16-bit elements with R, C and both strides multiples of 8 and 16-byte aligned bases: 16-byte
// global accesses on both sides, the transposition happens in the 2-byte LDS writes.
__global__ void __launch_bounds__(256) transpose_tiles16(uint16_t* out, const uint16_t* in, int R, int C,
                                                         int64_t ld_in, int64_t ld_out) {
  __shared__ __attribute__((aligned(16))) uint16_t tile[64][72];  // [column][row], rows of 144 bytes
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int idx = threadIdx.x + 256 * p, r = idx >> 3, cg = idx & 7;
    if (r0 + r < R && c0 + 8 * cg < C) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(in + (int64_t)(r0 + r) * ld_in + c0 + 8 * cg);
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[8 * cg + e][r] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
    }
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int idx = threadIdx.x + 256 * p, c = idx >> 3, rg = idx & 7;
    if (c0 + c < C && r0 + 8 * rg < R)
      *reinterpret_cast<u32x4*>(out + (int64_t)(c0 + c) * ld_out + r0 + 8 * rg) =
          *reinterpret_cast<const u32x4*>(&tile[c][8 * rg]);
  }
}

int transpose_matrix(void* out, const void* in, int R, int C, int64_t ld_in, int64_t ld_out, int elem_bytes,
                     hipStream_t s) {
  const dim3 grid((C + 63) / 64, (R + 63) / 64);
  if (elem_bytes == 2 && R % 8 == 0 && C % 8 == 0 && ld_in % 8 == 0 && ld_out % 8 == 0 && aligned16(out) && aligned16(in))
    LH_LAUNCH(transpose_tiles16, grid, dim3(256), 0, s, static_cast<uint16_t*>(out),
                       static_cast<const uint16_t*>(in), R, C, ld_in, ld_out);
  else if (elem_bytes == 2)
    LH_LAUNCH(transpose_tiles<uint16_t>, grid, dim3(256), 0, s, static_cast<uint16_t*>(out),
                       static_cast<const uint16_t*>(in), R, C, ld_in, ld_out);
  else if (elem_bytes == 4)
    LH_LAUNCH(transpose_tiles<uint32_t>, grid, dim3(256), 0, s, static_cast<uint32_t*>(out),
                       static_cast<const uint32_t*>(in), R, C, ld_in, ld_out);
  else
    return fail(LH_ERR_UNSUPPORTED, "transpose: element size %d", elem_bytes);
  return check_launch("transpose_tiles");
}

// dst[r][c] = src[r][c] inside the source matrix, 0 outside: the copies of a GEMM whose K or N the
// fast kernels cannot take (and the copy of its padded result back).  Any alignment on either side;
// a thread handles 8 consecutive elements of a row.
template <typename T>
__global__ void __launch_bounds__(256) pad_copy_kernel(T* dst, int64_t ld_dst, int rows_dst, int cols_dst, const T* src,
                                                       int64_t ld_src, int rows_src, int cols_src) {
  const int r = blockIdx.y;
  const int c0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (c0 >= cols_dst) return;
  T* d = dst + (int64_t)r * ld_dst + c0;
  const T* sp = src + (int64_t)r * ld_src + c0;
  const bool row_in = r < rows_src;
#pragma unroll
  for (int e = 0; e < 8; ++e)
    if (c0 + e < cols_dst) d[e] = (row_in && c0 + e < cols_src) ? sp[e] : (T)0;
}

int pad_copy_matrix(void* dst, int64_t ld_dst, int rows_dst, int cols_dst, const void* src, int64_t ld_src, int rows_src,
                    int cols_src, int elem_bytes, hipStream_t s) {
  if (rows_dst <= 0 || cols_dst <= 0) return LH_OK;
  const dim3 grid((cols_dst + 2047) / 2048, rows_dst);
  if (elem_bytes == 2)
    LH_LAUNCH(pad_copy_kernel<uint16_t>, grid, dim3(256), 0, s, static_cast<uint16_t*>(dst), ld_dst, rows_dst,
                       cols_dst, static_cast<const uint16_t*>(src), ld_src, rows_src, cols_src);
  else if (elem_bytes == 4)
    LH_LAUNCH(pad_copy_kernel<uint32_t>, grid, dim3(256), 0, s, static_cast<uint32_t*>(dst), ld_dst, rows_dst,
                       cols_dst, static_cast<const uint32_t*>(src), ld_src, rows_src, cols_src);
  else if (elem_bytes == 1)
    LH_LAUNCH(pad_copy_kernel<uint8_t>, grid, dim3(256), 0, s, static_cast<uint8_t*>(dst), ld_dst, rows_dst,
                       cols_dst, static_cast<const uint8_t*>(src), ld_src, rows_src, cols_src);
  else
    return fail(LH_ERR_UNSUPPORTED, "pad copy: element size %d", elem_bytes);
  return check_launch("pad_copy");
}

// ---- temporary device memory (see common.h) ------------------------------------------------
static thread_local int g_planning = 0;
bool planning() { return g_planning > 0; }
PlanningScope::PlanningScope() { ++g_planning; }
PlanningScope::~PlanningScope() { --g_planning; }
static thread_local int g_no_attention_scratch = 0;
bool attention_scratch_allowed() { return g_no_attention_scratch == 0; }
NoAttentionScratchScope::NoAttentionScratchScope() { ++g_no_attention_scratch; }
NoAttentionScratchScope::~NoAttentionScratchScope() { --g_no_attention_scratch; }

namespace {
struct PoolBuffer {
  char* p = nullptr;
  size_t bytes = 0;
};
struct StreamPool {
  PoolBuffer slot[kScratchSlots];
};
std::mutex g_pool_mutex;
std::map<std::pair<int, hipStream_t>, StreamPool> g_pools;
std::vector<std::pair<int, void*>> g_retired;  // (device, buffer) replaced by a larger one
constexpr size_t kGranule = 256;
size_t round_granule(size_t b) { return (b + kGranule - 1) / kGranule * kGranule; }
}  // namespace

int scratch_take(Scratch* ws, hipStream_t s, int slot, size_t bytes, const char* what, void** out) {
  *out = nullptr;
  if (bytes == 0) bytes = kGranule;
  if (planning()) {
    if (ws) ws->need += round_granule(bytes);
    *out = reinterpret_cast<void*>(uintptr_t(1) << 20);  // aligned, never dereferenced
    return LH_OK;
  }
  if (ws && ws->base) {
    const size_t at = round_granule(ws->used);
    if (at + bytes > ws->bytes)
      return fail(LH_ERR_INVALID, "%s: workspace too small: %zu more bytes needed, %zu of %zu in use", what, bytes, at,
                  ws->bytes);
    ws->used = at + bytes;
    *out = ws->base + at;
    return LH_OK;
  }
  int dev = 0;
  LH_HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  PoolBuffer& b = g_pools[{dev, s}].slot[slot];
  if (bytes > b.bytes) {
    // At least double, so that the buffers left behind add up to less than the live one.
    size_t want = round_granule(bytes > 2 * b.bytes ? bytes : 2 * b.bytes);
    char* p = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&p), want);
    if (e != hipSuccess && want > round_granule(bytes)) {
      (void)hipGetLastError();
      want = round_granule(bytes);
      e = hipMalloc(reinterpret_cast<void**>(&p), want);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(LH_ERR_RUNTIME, "%s: hipMalloc of %zu bytes failed: %s", what, want, hipGetErrorString(e));
    }
    if (b.p) g_retired.emplace_back(dev, b.p);
    b.p = p;
    b.bytes = want;
  }
  *out = b.p;
  return LH_OK;
}

// ---- statically allocated scratch ------------------------------------------------------------
// Temporary memory for the one entry point that must not allocate (lh_hip_gemm_static): an array
// in the library's device image, so every GPU the library runs on holds its own copy from the
// moment the code object is loaded until the process ends.  In host code the array's name is only
// a handle for the runtime; the address kernels may use comes from hipGetSymbolAddress, asked once
// per device with that device current, and kept.
static __device__ __align__(256) unsigned char scratch[LH_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
static std::mutex g_static_mutex;
static char* g_static_ptr[kMaxDevices] = {};

int static_scratch(char** base, size_t* bytes) {
  int dev = 0;
  LH_HIP_CHECK(hipGetDevice(&dev));
  LH_REQUIRE(dev >= 0 && dev < kMaxDevices, "static scratch: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    LH_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    LH_REQUIRE(p != nullptr && (reinterpret_cast<uintptr_t>(p) & 255u) == 0, "static scratch: bad device address %p", p);
    g_static_ptr[dev] = static_cast<char*>(p);
  }
  *base = g_static_ptr[dev];
  *bytes = LH_STATIC_SCRATCH_BYTES;
  return LH_OK;
}

static int release_pool_of_current_device() {
  int dev = 0;
  LH_HIP_CHECK(hipGetDevice(&dev));
  LH_HIP_CHECK(hipDeviceSynchronize());
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  hipError_t first = hipSuccess;
  auto release = [&](void* p) {
    const hipError_t e = hipFree(p);
    if (e != hipSuccess && first == hipSuccess) first = e;
  };
  for (auto it = g_pools.begin(); it != g_pools.end();) {
    if (it->first.first != dev) {
      ++it;
      continue;
    }
    for (PoolBuffer& b : it->second.slot)
      if (b.p) release(b.p);
    it = g_pools.erase(it);
  }
  std::vector<std::pair<int, void*>> keep;
  for (auto& r : g_retired) {
    if (r.first == dev) release(r.second);
    else keep.push_back(r);
  }
  g_retired.swap(keep);
  if (first != hipSuccess) {
    (void)hipGetLastError();
    return fail(LH_ERR_RUNTIME, "lh_hip_release_scratch: hipFree failed: %s", hipGetErrorString(first));
  }
  return LH_OK;
}

}  // namespace lh

using namespace lh;

extern "C" {

const char* lh_hip_last_error(void) { return g_error; }

int lh_hip_device_count(int32_t* out) {
  LH_REQUIRE(out != nullptr, "lh_hip_device_count: out is null");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  *out = n;
  return LH_OK;
}

int lh_hip_device_info(lh_device_info* out) {
  LH_REQUIRE(out != nullptr, "lh_hip_device_info: out is null");
  int dev = 0;
  LH_HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t p;
  LH_HIP_CHECK(hipGetDeviceProperties(&p, dev));
  std::memset(out, 0, sizeof(*out));
  std::strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
  std::strncpy(out->name, p.name, sizeof(out->name) - 1);
  out->compute_units = p.multiProcessorCount;
  out->clock_khz = p.clockRate;
  out->memory_clock_khz = p.memoryClockRate;
  out->memory_bus_bits = p.memoryBusWidth;
  out->lds_bytes_per_cu = (int32_t)p.maxSharedMemoryPerMultiProcessor;
  out->wavefront_size = p.warpSize;
  out->hbm_bytes = (int64_t)p.totalGlobalMem;
  return LH_OK;
}

int lh_hip_alloc(void** dev_ptr, size_t bytes) {
  LH_REQUIRE(dev_ptr != nullptr, "lh_hip_alloc: dev_ptr is null");
  *dev_ptr = nullptr;
  if (bytes == 0) bytes = 16;
  LH_HIP_CHECK(hipMalloc(dev_ptr, bytes));
  return LH_OK;
}

int lh_hip_free(void* dev_ptr) {
  if (dev_ptr == nullptr) return LH_OK;
  LH_HIP_CHECK(hipFree(dev_ptr));
  return LH_OK;
}

int lh_hip_memcpy_h2d(void* dev_dst, const void* host_src, size_t bytes) {
  LH_REQUIRE(dev_dst != nullptr && host_src != nullptr, "lh_hip_memcpy_h2d: null pointer");
  if (bytes == 0) return LH_OK;
  LH_HIP_CHECK(hipMemcpy(dev_dst, host_src, bytes, hipMemcpyHostToDevice));
  return LH_OK;
}

int lh_hip_memcpy_d2h(void* host_dst, const void* dev_src, size_t bytes) {
  LH_REQUIRE(host_dst != nullptr && dev_src != nullptr, "lh_hip_memcpy_d2h: null pointer");
  if (bytes == 0) return LH_OK;
  LH_HIP_CHECK(hipMemcpy(host_dst, dev_src, bytes, hipMemcpyDeviceToHost));
  return LH_OK;
}

int lh_hip_memcpy_d2d(void* dev_dst, const void* dev_src, size_t bytes) {
  LH_REQUIRE(dev_dst != nullptr && dev_src != nullptr, "lh_hip_memcpy_d2d: null pointer");
  if (bytes == 0) return LH_OK;
  LH_HIP_CHECK(hipMemcpy(dev_dst, dev_src, bytes, hipMemcpyDeviceToDevice));
  return LH_OK;
}

int lh_hip_memset(void* dev_ptr, int value, size_t bytes) {
  LH_REQUIRE(dev_ptr != nullptr, "lh_hip_memset: null pointer");
  if (bytes == 0) return LH_OK;
  LH_HIP_CHECK(hipMemset(dev_ptr, value, bytes));
  return LH_OK;
}

int lh_hip_release_scratch(void) { return release_pool_of_current_device(); }

int lh_hip_sync(void* stream) {
  LH_HIP_CHECK(hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)));
  return LH_OK;
}

}  // extern "C"
