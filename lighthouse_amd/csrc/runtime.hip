// Runtime part of the C ABI: error state, device info, device memory helpers.
#include <cstring>

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

int lh_hip_sync(void* stream) {
  LH_HIP_CHECK(hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)));
  return LH_OK;
}

}  // extern "C"
