// lib.hip — library-level entry points and host helpers of libtriton_int_hip.so.
#include <stdarg.h>
#include <string.h>

#include "ti_common.h"

namespace ti {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// The kernels are written for gfx950 only (MFMA shapes, 160 KB LDS, buffer loads into LDS); on
// any other device the launch would fail or fault, so refuse early with a clear message.
int check_device() {
  static int checked[64];  // 0 unknown, 1 ok, -1 wrong arch
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= 64) return TI_OK;
  if (checked[dev] == 0) {
    hipDeviceProp_t prop;
    err = hipGetDeviceProperties(&prop, dev);
    if (err != hipSuccess) return fail((int)err, "hipGetDeviceProperties: %s", hipGetErrorString(err));
    checked[dev] = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    if (checked[dev] < 0) set_error("device %d is %s; this library only runs on gfx950", dev, prop.gcnArchName);
  }
  if (checked[dev] < 0) {
    set_error("device %d is not gfx950", dev);
    return TI_E_DEVICE;
  }
  return TI_OK;
}

int launch_status(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail((int)err, "launch of %s failed: %s", what, hipGetErrorString(err));
  return TI_OK;
}

// ---- MFMA issue-rate probe ---------------------------------------------------------------------
// Back-to-back v_mfma_i32_32x32x32_i8 on register operands only (no LDS, no memory): the rate the
// matrix pipes sustain at the clock the power management settles on.  With random operand bytes
// that clock is far below the nominal one, so this, not the data-sheet peak, is the ceiling a
// GEMM on random int8 data can approach.
constexpr int PROBE_BLOCKS = 1024, PROBE_THREADS = 256, PROBE_ACC = 8;
__device__ int g_probe_sink[PROBE_BLOCKS * PROBE_THREADS];

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

__global__ __launch_bounds__(PROBE_THREADS) void mfma_probe_kernel(int iters, int random_operands) {
  v4i a[PROBE_ACC], b[PROBE_ACC];
#pragma unroll
  for (int i = 0; i < PROBE_ACC; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned s = (blockIdx.x * PROBE_THREADS + threadIdx.x) * 64u + i * 8u + j;
      a[i][j] = random_operands ? (int)probe_hash(s) : 0x01010101;
      b[i][j] = random_operands ? (int)probe_hash(s + 4u) : 0x02020202;
    }
  v16i acc[PROBE_ACC];
#pragma unroll
  for (int i = 0; i < PROBE_ACC; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < PROBE_ACC; ++i)
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[i], acc[i], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < PROBE_ACC; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  g_probe_sink[blockIdx.x * PROBE_THREADS + threadIdx.x] = s;
}

}  // namespace ti

extern "C" {

int ti_version(void) { return 2; }

int ti_mfma_i8_probe(int iters, int random_operands, void* stream, double* ops_out) {
  if (iters < 0) return ti::fail(TI_E_SHAPE, "negative iteration count");
  int rc = ti::check_device();
  if (rc != TI_OK) return rc;
  ti::mfma_probe_kernel<<<dim3(ti::PROBE_BLOCKS), dim3(ti::PROBE_THREADS), 0, (hipStream_t)stream>>>(iters, random_operands);
  if (ops_out)
    *ops_out = (double)ti::PROBE_BLOCKS * (ti::PROBE_THREADS / 64) * (double)iters * ti::PROBE_ACC * 65536.0;
  return ti::launch_status("mfma_probe_kernel");
}

const char* ti_last_error(void) { return ti::g_err; }

}  // extern "C"
