// Error channel, identification and the row-normalisation helpers of the C-ABI.

#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "mma_tiles.h"

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
extern "C" int lnx_abi_version(void) { return 8; }

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
  // a capturing stream takes no marks: an event created or recorded here would become part of the caller's graph
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return;
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

// Vector forms for rows of LPR 16-byte vectors (LPR a power of two <= 64): LPR lanes share a row, a
// wavefront covers 64 / LPR rows per pass and four passes per step (all loads of a step issued
// before the first reduction), so the kernels run at streaming bandwidth.
template <typename T, int LPR>
__global__ __launch_bounds__(256) void l2norm_fwd_vec_kernel(const T* x, T* y, int64_t rows) {
  typedef typename Vec16<T>::V V;
  constexpr int VN = Vec16<T>::N, RPW = 64 / LPR, UNR = 4, D = LPR * VN;
  const int lane = threadIdx.x & 63, sub = lane / LPR, li = lane % LPR;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t r0 = wave * (RPW * UNR) + sub;
  V xv[UNR];
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t r = r0 + u * RPW;
    xv[u] = vec_zero<T>();
    if (r < rows) xv[u] = *reinterpret_cast<const V*>(x + r * D + li * VN);
  }
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t r = r0 + u * RPW;
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < VN; ++e) { const float t = to_f32(xv[u][e]); ss += t * t; }
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, LNX_WAVE);
    const float inv = 1.f / (sqrtf(ss) + LNX_L2_EPS);
    V out;
#pragma unroll
    for (int e = 0; e < VN; ++e) out[e] = from_f32<T>(to_f32(xv[u][e]) * inv);
    if (r < rows) *reinterpret_cast<V*>(y + r * D + li * VN) = out;
  }
}

template <typename T, int LPR>
__global__ __launch_bounds__(256) void l2norm_bwd_vec_kernel(const T* x, const T* dy, T* dx, int64_t rows) {
  typedef typename Vec16<T>::V V;
  constexpr int VN = Vec16<T>::N, RPW = 64 / LPR, UNR = 4, D = LPR * VN;
  const int lane = threadIdx.x & 63, sub = lane / LPR, li = lane % LPR;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t r0 = wave * (RPW * UNR) + sub;
  V xv[UNR], gv[UNR];
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t r = r0 + u * RPW;
    xv[u] = vec_zero<T>();
    gv[u] = vec_zero<T>();
    if (r < rows) {
      xv[u] = *reinterpret_cast<const V*>(x + r * D + li * VN);
      gv[u] = *reinterpret_cast<const V*>(dy + r * D + li * VN);
    }
  }
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t r = r0 + u * RPW;
    float ss = 0.f, dot = 0.f;
#pragma unroll
    for (int e = 0; e < VN; ++e) {
      const float t = to_f32(xv[u][e]);
      ss += t * t;
      dot += t * to_f32(gv[u][e]);
    }
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) {
      ss += __shfl_xor(ss, m, LNX_WAVE);
      dot += __shfl_xor(dot, m, LNX_WAVE);
    }
    const float n = sqrtf(ss), sd = n + LNX_L2_EPS;
    const float c = dot / (fmaxf(n, 1e-30f) * sd * sd);
    V out;
#pragma unroll
    for (int e = 0; e < VN; ++e) out[e] = from_f32<T>(to_f32(gv[u][e]) / sd - to_f32(xv[u][e]) * c);
    if (r < rows) *reinterpret_cast<V*>(dx + r * D + li * VN) = out;
  }
}

// lanes per row for the vector kernels, or 0 when the row length does not fit them
template <typename T> int norm_lanes(int d) {
  constexpr int VN = 16 / sizeof(T);
  if (d % VN != 0) return 0;
  const int l = d / VN;
  return (l == 4 || l == 8 || l == 16 || l == 32 || l == 64) ? l : 0;
}

template <typename T>
bool launch_norm_fwd(const T* x, T* y, int64_t rows, int d, hipStream_t st) {
  const int l = norm_lanes<T>(d);
  if (!l) return false;
  const int64_t waves = (rows + (64 / l) * 4 - 1) / ((64 / l) * 4);
  dim3 grid((unsigned)((waves + 3) / 4));
  switch (l) {
    case 4: hipLaunchKernelGGL((l2norm_fwd_vec_kernel<T, 4>), grid, dim3(256), 0, st, x, y, rows); break;
    case 8: hipLaunchKernelGGL((l2norm_fwd_vec_kernel<T, 8>), grid, dim3(256), 0, st, x, y, rows); break;
    case 16: hipLaunchKernelGGL((l2norm_fwd_vec_kernel<T, 16>), grid, dim3(256), 0, st, x, y, rows); break;
    case 32: hipLaunchKernelGGL((l2norm_fwd_vec_kernel<T, 32>), grid, dim3(256), 0, st, x, y, rows); break;
    default: hipLaunchKernelGGL((l2norm_fwd_vec_kernel<T, 64>), grid, dim3(256), 0, st, x, y, rows); break;
  }
  return true;
}

template <typename T>
bool launch_norm_bwd(const T* x, const T* dy, T* dx, int64_t rows, int d, hipStream_t st) {
  const int l = norm_lanes<T>(d);
  if (!l) return false;
  const int64_t waves = (rows + (64 / l) * 4 - 1) / ((64 / l) * 4);
  dim3 grid((unsigned)((waves + 3) / 4));
  switch (l) {
    case 4: hipLaunchKernelGGL((l2norm_bwd_vec_kernel<T, 4>), grid, dim3(256), 0, st, x, dy, dx, rows); break;
    case 8: hipLaunchKernelGGL((l2norm_bwd_vec_kernel<T, 8>), grid, dim3(256), 0, st, x, dy, dx, rows); break;
    case 16: hipLaunchKernelGGL((l2norm_bwd_vec_kernel<T, 16>), grid, dim3(256), 0, st, x, dy, dx, rows); break;
    case 32: hipLaunchKernelGGL((l2norm_bwd_vec_kernel<T, 32>), grid, dim3(256), 0, st, x, dy, dx, rows); break;
    default: hipLaunchKernelGGL((l2norm_bwd_vec_kernel<T, 64>), grid, dim3(256), 0, st, x, dy, dx, rows); break;
  }
  return true;
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
  hipStream_t st = (hipStream_t)stream;
  const bool vec = (dtype == LNX_BF16) ? launch_norm_fwd<bf16_t>((const bf16_t*)x, (bf16_t*)y, rows, d, st)
                                       : launch_norm_fwd<float>((const float*)x, (float*)y, rows, d, st);
  if (!vec) {  // row lengths the vector kernels do not cover
    dim3 grid((unsigned)((rows + 3) / 4));
    if (dtype == LNX_BF16)
      hipLaunchKernelGGL(l2norm_fwd_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)x, (bf16_t*)y, rows, d);
    else
      hipLaunchKernelGGL(l2norm_fwd_kernel<float>, grid, dim3(256), 0, st, (const float*)x, (float*)y, rows, d);
  }
  return finish("l2norm_fwd");
}

extern "C" int lnx_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t d, int32_t dtype,
                              void* stream) {
  int rc = check_norm_args(x, dy, rows, d, dtype);
  if (rc != LNX_OK) return rc;
  if (rows == 0) return LNX_OK;
  if (!dx) return lnx_set_error(LNX_ERR_NULL, "l2norm_bwd: dx is NULL");
  hipStream_t st = (hipStream_t)stream;
  const bool vec = (dtype == LNX_BF16)
                       ? launch_norm_bwd<bf16_t>((const bf16_t*)x, (const bf16_t*)dy, (bf16_t*)dx, rows, d, st)
                       : launch_norm_bwd<float>((const float*)x, (const float*)dy, (float*)dx, rows, d, st);
  if (!vec) {
    dim3 grid((unsigned)((rows + 3) / 4));
    if (dtype == LNX_BF16)
      hipLaunchKernelGGL(l2norm_bwd_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)x, (const bf16_t*)dy, (bf16_t*)dx, rows, d);
    else
      hipLaunchKernelGGL(l2norm_bwd_kernel<float>, grid, dim3(256), 0, st, (const float*)x, (const float*)dy, (float*)dx, rows, d);
  }
  return finish("l2norm_bwd");
}
