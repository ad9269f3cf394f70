// Library set-up, error strings, per-stream scratch arenas, small fill kernels.
#include <stdarg.h>
#include <string.h>

#include <map>
#include <mutex>
#include <utility>

#include "common.h"
#include "grid.h"

namespace insc {

static thread_local char g_err[512] = "";
static int g_device = -1;

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char *what, const char *file, int line) {
  const char *base = strrchr(file, '/');
  set_error("HIP error %d (%s) in %s at %s:%d", (int)e, hipGetErrorString(e), what, base ? base + 1 : file, line);
  return INSC_ERR_HIP;
}

struct Arena {
  void *p = nullptr;
  size_t bytes = 0;
};
static std::mutex g_ws_mu;
static std::map<std::pair<int, std::pair<int, hipStream_t>>, Arena> g_ws;

static int arena_get(int which, hipStream_t stream, size_t bytes, void **out) {
  int dev = 0;
  INSC_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lk(g_ws_mu);
  Arena &a = g_ws[std::make_pair(which, std::make_pair(dev, stream))];
  if (a.bytes < bytes) {
    if (a.p) {
      // the old block may still be read by work in flight on this stream
      INSC_HIP(hipStreamSynchronize(stream));
      INSC_HIP(hipFree(a.p));
      a.p = nullptr;
      a.bytes = 0;
    }
    size_t want = bytes + bytes / 2;
    if (want < (1u << 20)) want = 1u << 20;
    INSC_HIP(hipMalloc(&a.p, want));
    a.bytes = want;
  }
  *out = a.p;
  return INSC_OK;
}
int workspace(int which, hipStream_t stream, size_t bytes, void **out) { return arena_get(which, stream, bytes, out); }

// int32 counters per (device, stream) that are zero whenever a kernel starts: zeroed when the
// block is created or grown, and every kernel that uses them puts them back to zero.
struct Counters {
  int32_t *p = nullptr;
  size_t count = 0;
};
static std::map<std::pair<int, hipStream_t>, Counters> g_counters;
int zero_counters(hipStream_t stream, size_t count, int32_t **out) {
  int dev = 0;
  INSC_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lk(g_ws_mu);
  Counters &c = g_counters[std::make_pair(dev, stream)];
  if (c.count < count) {
    if (c.p) {
      INSC_HIP(hipStreamSynchronize(stream));
      INSC_HIP(hipFree(c.p));
      c.p = nullptr;
      c.count = 0;
    }
    size_t want = count < 16384 ? 16384 : count + count / 2;
    INSC_HIP(hipMalloc((void **)&c.p, want * sizeof(int32_t)));
    INSC_HIP(hipMemsetAsync(c.p, 0, want * sizeof(int32_t), stream));
    c.count = want;
  }
  *out = c.p;
  return INSC_OK;
}


__global__ void fill_u8_kernel(uint8_t *p, int64_t n, uint8_t v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}
__global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t v) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

}  // namespace insc

namespace insc {
// compute units of the current device (queried once per device)
int device_cus() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cus[dev]) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cus[dev] = v;
  }
  return cus[dev];
}
}  // namespace insc

using namespace insc;

extern "C" {

int insc_init(int device) {
  int count = 0;
  INSC_HIP(hipGetDeviceCount(&count));
  INSC_REQUIRE(device >= 0 && device < count, INSC_ERR_ARG, "insc_init: device %d not in [0,%d)", device, count);
  INSC_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  INSC_HIP(hipGetDeviceProperties(&prop, device));
  INSC_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0, INSC_ERR_STATE,
               "insc_init: device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
  g_device = device;
  return grid_noalloc_setup();
}

const char *insc_last_error(void) { return g_err; }
const char *insc_version(void) { return "insc 0.1 (gfx950)"; }

int insc_fill_u8(uint8_t *d_p, int64_t n, int value, void *stream) {
  INSC_REQUIRE(n >= 0 && (d_p || n == 0), INSC_ERR_ARG, "insc_fill_u8: bad arguments");
  if (n == 0) return INSC_OK;
  hipLaunchKernelGGL(fill_u8_kernel, dim3(grid_for(n, 256, 4096)), dim3(256), 0, (hipStream_t)stream, d_p, n,
                     (uint8_t)value);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

int insc_fill_i32(int32_t *d_p, int64_t n, int32_t value, void *stream) {
  INSC_REQUIRE(n >= 0 && (d_p || n == 0), INSC_ERR_ARG, "insc_fill_i32: bad arguments");
  if (n == 0) return INSC_OK;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(n, 256, 4096)), dim3(256), 0, (hipStream_t)stream, d_p, n,
                     value);
  INSC_LAUNCH_CHECK();
  return INSC_OK;
}

}  // extern "C"
