// Error channel, identification and the row-normalisation helpers of the C-ABI.

#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "lnx_common.h"

namespace {
thread_local char g_error[512] = "";
}

int lnx_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char* lnx_last_error(void) { return g_error; }
extern "C" int lnx_abi_version(void) { return 2; }

// ---- optional per-kernel timing with HIP events on the caller's stream.  Process-wide (one
// mutex-guarded list) because a framework may run the backward entry point on another thread. ----
namespace {
struct Profile {
  bool on = false;
  int n = 0;  // events recorded
  hipEvent_t ev[LNX_PROFILE_MAX + 1];
  const char* name[LNX_PROFILE_MAX];
  int created = 0;
};
Profile g_prof;
std::mutex g_prof_mutex;
}  // namespace

void lnx_profile_mark(const char* kernel_name, hipStream_t st) {
  Profile& P = g_prof;
  if (!P.on) return;  // unguarded fast path: timing is off in normal use
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  if (!P.on || P.n > LNX_PROFILE_MAX) return;
  if (kernel_name != nullptr && P.n == LNX_PROFILE_MAX) return;  // keep one slot for the closing mark
  if (P.created <= P.n) {
    if (hipEventCreate(&P.ev[P.created]) != hipSuccess) return;
    ++P.created;
  }
  if (hipEventRecord(P.ev[P.n], st) != hipSuccess) return;
  if (P.n < LNX_PROFILE_MAX) P.name[P.n] = kernel_name;
  ++P.n;
}

extern "C" int lnx_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof.on = on != 0;
  g_prof.n = 0;
  return LNX_OK;
}

extern "C" int lnx_profile_read(int capacity, const char** names, float* ms) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  Profile& P = g_prof;
  int out = 0;
  for (int i = 0; i + 1 < P.n && i < LNX_PROFILE_MAX; ++i) {
    if (P.name[i] == nullptr) continue;  // a closing mark: the gap to the next entry point
    if (hipEventSynchronize(P.ev[i + 1]) != hipSuccess) break;
    float t = 0.f;
    if (hipEventElapsedTime(&t, P.ev[i], P.ev[i + 1]) != hipSuccess) break;
    if (out < capacity) { names[out] = P.name[i]; ms[out] = t; }
    ++out;
  }
  P.n = 0;
  return out;
}
namespace {

// One wavefront per row: y = x / (|x| + eps).
template <typename T>
__global__ __launch_bounds__(256) void l2norm_fwd_kernel(const T* x, T* y, int64_t rows, int d) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const T* xr = x + row * d;
  float ss = 0.f;
  for (int i = lane; i < d; i += 64) { const float t = to_f32(xr[i]); ss += t * t; }
  const float inv = 1.f / (sqrtf(wave_sum(ss)) + LNX_L2_EPS);
  for (int i = lane; i < d; i += 64) y[row * d + i] = from_f32<T>(to_f32(xr[i]) * inv);
}

// dx = dy / s - x <x, dy> / (n s^2),  n = |x|, s = n + eps.
template <typename T>
__global__ __launch_bounds__(256) void l2norm_bwd_kernel(const T* x, const T* dy, T* dx, int64_t rows, int d) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const T* xr = x + row * d;
  const T* gr = dy + row * d;
  float ss = 0.f, dot = 0.f;
  for (int i = lane; i < d; i += 64) {
    const float t = to_f32(xr[i]);
    ss += t * t;
    dot += t * to_f32(gr[i]);
  }
  const float n = sqrtf(wave_sum(ss));
  dot = wave_sum(dot);
  const float s = n + LNX_L2_EPS;
  const float c = dot / (fmaxf(n, 1e-30f) * s * s);
  for (int i = lane; i < d; i += 64) dx[row * d + i] = from_f32<T>(to_f32(gr[i]) / s - to_f32(xr[i]) * c);
}

int check_norm_args(const void* a, const void* b, int64_t rows, int d, int dtype) {
  if (rows < 0 || d <= 0) return lnx_set_error(LNX_ERR_SHAPE, "l2norm: rows=%lld d=%d", (long long)rows, d);
  if (rows > 0 && (!a || !b)) return lnx_set_error(LNX_ERR_NULL, "l2norm: NULL tensor");  // empty tensors may be null
  if (dtype != LNX_F32 && dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "l2norm: dtype %d", dtype);
  return LNX_OK;
}

int finish(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return LNX_OK;
}

}  // namespace

extern "C" int lnx_l2norm_fwd(const void* x, void* y, int64_t rows, int32_t d, int32_t dtype, void* stream) {
  int rc = check_norm_args(x, y, rows, d, dtype);
  if (rc != LNX_OK || rows == 0) return rc;
  dim3 grid((unsigned)((rows + 3) / 4));
  if (dtype == LNX_BF16)
    hipLaunchKernelGGL(l2norm_fwd_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x, (bf16_t*)y, rows, d);
  else
    hipLaunchKernelGGL(l2norm_fwd_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)x, (float*)y, rows, d);
  return finish("l2norm_fwd");
}

extern "C" int lnx_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t d, int32_t dtype,
                              void* stream) {
  int rc = check_norm_args(x, dy, rows, d, dtype);
  if (rc != LNX_OK) return rc;
  if (!dx) return lnx_set_error(LNX_ERR_NULL, "l2norm_bwd: dx is NULL");
  if (rows == 0) return LNX_OK;
  dim3 grid((unsigned)((rows + 3) / 4));
  if (dtype == LNX_BF16)
    hipLaunchKernelGGL(l2norm_bwd_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x, (const bf16_t*)dy, (bf16_t*)dx, rows, d);
  else
    hipLaunchKernelGGL(l2norm_bwd_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float*)x, (const float*)dy, (float*)dx, rows, d);
  return finish("l2norm_bwd");
}
