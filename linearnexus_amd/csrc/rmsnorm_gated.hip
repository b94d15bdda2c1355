// RMSNorm with an optional sigmoid gate over the rows of a [rows, d] matrix, forward and backward: the
// output epilogue of the reference's blocks (FusedRMSNormGated, linearnexus/modules/linear_attn/kda.py:664-700,
// used as o_norm(o) * sigmoid(gate) in gated_deltanet.py:854-862):
//   y = x * rsqrt(mean(x^2) + eps) * weight * sigmoid(gate)        (gate NULL: no gate)
// Streaming kernels: LPR lanes share a row of LPR 16-byte vectors, a wavefront covers 64 / LPR rows per pass,
// and the loads of four passes are issued together.  The backward also keeps d_weight partial sums in
// registers over all passes of a wavefront and adds them with one atomic per column and workgroup.
#include "lnx_common.h"
#include "mma_tiles.h"
#include "reduce_rows.h"

namespace {

constexpr int UNR = 4;         // passes whose loads are in flight together
constexpr int BWD_STEPS = 8;   // steps (of UNR passes) per wavefront in the backward: rows per d_weight atomic

__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + __expf(-z)); }

template <typename T, int LPR>
__global__ __launch_bounds__(256) void rmsnorm_gated_fwd_kernel(const T* x, const T* gate, const float* w, T* y,
                                                                int64_t rows, float eps) {
  typedef typename Vec16<T>::V V;
  constexpr int VN = Vec16<T>::N, RPW = 64 / LPR, D = LPR * VN;
  const int lane = threadIdx.x & 63, sub = lane / LPR, li = lane % LPR;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t r0 = wave * (RPW * UNR) + sub;
  float wv[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) wv[e] = w[li * VN + e];
  V xv[UNR], gv[UNR];
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t r = r0 + u * RPW;
    xv[u] = vec_zero<T>();
    gv[u] = vec_zero<T>();
    if (r < rows) {
      xv[u] = *reinterpret_cast<const V*>(x + r * D + li * VN);
      if (gate) gv[u] = *reinterpret_cast<const V*>(gate + r * D + li * VN);
    }
  }
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t r = r0 + u * RPW;
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < VN; ++e) { const float t = to_f32(xv[u][e]); ss += t * t; }
#pragma unroll
    for (int m = LPR / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, LNX_WAVE);
    const float rstd = rsqrtf(ss * (1.f / D) + eps);
    V out;
#pragma unroll
    for (int e = 0; e < VN; ++e) {
      const float s = gate ? sigmoidf(to_f32(gv[u][e])) : 1.f;
      out[e] = from_f32<T>(to_f32(xv[u][e]) * rstd * wv[e] * s);
    }
    if (r < rows) *reinterpret_cast<V*>(y + r * D + li * VN) = out;
  }
}

// With xn = x rstd, s = sigmoid(gate), u = dy s w:
//   dx = rstd (u - xn mean(u xn));  dgate = dy xn w s (1 - s);  dweight = sum over rows of dy xn s.
template <typename T, int LPR>
__global__ __launch_bounds__(256) void rmsnorm_gated_bwd_kernel(const T* x, const T* gate, const float* w, const T* dy,
                                                                T* dx, T* dgate, float* dw, int64_t rows, float eps) {
  typedef typename Vec16<T>::V V;
  constexpr int VN = Vec16<T>::N, RPW = 64 / LPR, D = LPR * VN;
  const int lane = threadIdx.x & 63, sub = lane / LPR, li = lane % LPR;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  float wv[VN], dwv[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) wv[e] = w[li * VN + e], dwv[e] = 0.f;
  for (int step = 0; step < BWD_STEPS; ++step) {
    const int64_t r0 = (wave * BWD_STEPS + step) * (RPW * UNR) + sub;
    if (r0 - sub >= rows) break;
    V xv[UNR], gv[UNR], yv[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int64_t r = r0 + u * RPW;
      xv[u] = vec_zero<T>();
      gv[u] = vec_zero<T>();
      yv[u] = vec_zero<T>();
      if (r < rows) {
        xv[u] = *reinterpret_cast<const V*>(x + r * D + li * VN);
        yv[u] = *reinterpret_cast<const V*>(dy + r * D + li * VN);
        if (gate) gv[u] = *reinterpret_cast<const V*>(gate + r * D + li * VN);
      }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int64_t r = r0 + u * RPW;
      float ss = 0.f, dot = 0.f, uu[VN], sg[VN];
#pragma unroll
      for (int e = 0; e < VN; ++e) {
        const float t = to_f32(xv[u][e]);
        sg[e] = gate ? sigmoidf(to_f32(gv[u][e])) : 1.f;
        uu[e] = to_f32(yv[u][e]) * sg[e] * wv[e];
        ss += t * t;
        dot += uu[e] * t;
      }
#pragma unroll
      for (int m = LPR / 2; m >= 1; m >>= 1) {
        ss += __shfl_xor(ss, m, LNX_WAVE);
        dot += __shfl_xor(dot, m, LNX_WAVE);
      }
      const float rstd = rsqrtf(ss * (1.f / D) + eps);
      const float c = dot * rstd * rstd * (1.f / D);  // mean(u xn) rstd / rstd: applied to x below
      V ox, og;
#pragma unroll
      for (int e = 0; e < VN; ++e) {
        const float t = to_f32(xv[u][e]), xn = t * rstd, g = to_f32(yv[u][e]);
        ox[e] = from_f32<T>(rstd * (uu[e] - t * c));
        og[e] = from_f32<T>(g * xn * wv[e] * sg[e] * (1.f - sg[e]));
        dwv[e] += g * xn * sg[e];  // rows past the end contribute zeros (x, dy loaded as zeros)
      }
      if (r < rows) {
        *reinterpret_cast<V*>(dx + r * D + li * VN) = ox;
        if (gate) *reinterpret_cast<V*>(dgate + r * D + li * VN) = og;
      }
    }
  }
  if (!dw) return;
  // d_weight: over the rows of a pass by shuffles, over the four wavefronts in LDS, then one row of partial sums
  // per workgroup in the workspace (a second kernel adds the rows: no atomics, the result is deterministic)
  __shared__ float red[3][D];
  const int wv_i = threadIdx.x >> 6;
#pragma unroll
  for (int e = 0; e < VN; ++e) {
    float t = dwv[e];
#pragma unroll
    for (int m = LPR; m < 64; m <<= 1) t += __shfl_xor(t, m, LNX_WAVE);
    dwv[e] = t;
    if (sub == 0 && wv_i > 0) red[wv_i - 1][li * VN + e] = t;
  }
  __syncthreads();
  if (wv_i == 0 && sub == 0) {
#pragma unroll
    for (int e = 0; e < VN; ++e)
      dw[(size_t)blockIdx.x * D + li * VN + e] = dwv[e] + red[0][li * VN + e] + red[1][li * VN + e] + red[2][li * VN + e];
  }
}

// Rows of any other width (a multiple of one 16-byte vector, at most 256 vectors -- e.g. the 512-wide value heads of
// the reference's Gated DeltaNet presets in fp32): one row per wavefront and pass, lane l holds vectors l, l + 64, ...
// (NV of them, those past the row masked), two passes in flight.
constexpr int UNRW = 2;

template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_gated_fwd_wide_kernel(const T* x, const T* gate, const float* w, T* y,
                                                                     int64_t rows, int d, float eps) {
  typedef typename Vec16<T>::V V;
  constexpr int VN = Vec16<T>::N;
  const int lane = threadIdx.x & 63, nvec = d / VN;
  const int64_t r0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * UNRW;
  float wv[NV][VN];
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int e = 0; e < VN; ++e) wv[j][e] = (lane + 64 * j < nvec) ? w[(lane + 64 * j) * VN + e] : 0.f;
  V xv[UNRW][NV], gv[UNRW][NV];
#pragma unroll
  for (int u = 0; u < UNRW; ++u)
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t r = r0 + u;
      const int c = (lane + 64 * j) * VN;
      xv[u][j] = vec_zero<T>();
      gv[u][j] = vec_zero<T>();
      if (r < rows && c < d) {
        xv[u][j] = *reinterpret_cast<const V*>(x + r * d + c);
        if (gate) gv[u][j] = *reinterpret_cast<const V*>(gate + r * d + c);
      }
    }
#pragma unroll
  for (int u = 0; u < UNRW; ++u) {
    const int64_t r = r0 + u;
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < VN; ++e) { const float t = to_f32(xv[u][j][e]); ss += t * t; }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, LNX_WAVE);
    const float rstd = rsqrtf(ss / d + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int c = (lane + 64 * j) * VN;
      V out;
#pragma unroll
      for (int e = 0; e < VN; ++e) {
        const float sg = gate ? sigmoidf(to_f32(gv[u][j][e])) : 1.f;
        out[e] = from_f32<T>(to_f32(xv[u][j][e]) * rstd * wv[j][e] * sg);
      }
      if (r < rows && c < d) *reinterpret_cast<V*>(y + r * d + c) = out;
    }
  }
}

template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_gated_bwd_wide_kernel(const T* x, const T* gate, const float* w, const T* dy,
                                                                     T* dx, T* dgate, float* dw, int64_t rows, int d, float eps) {
  typedef typename Vec16<T>::V V;
  constexpr int VN = Vec16<T>::N;
  const int lane = threadIdx.x & 63, wv_i = threadIdx.x >> 6;
  const int64_t wave = (int64_t)blockIdx.x * 4 + wv_i;
  float wv[NV][VN], dwv[NV][VN];
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int e = 0; e < VN; ++e) {
      wv[j][e] = ((lane + 64 * j) * VN < d) ? w[(lane + 64 * j) * VN + e] : 0.f;
      dwv[j][e] = 0.f;
    }
  for (int step = 0; step < BWD_STEPS; ++step) {
    const int64_t r0 = (wave * BWD_STEPS + step) * UNRW;
    if (r0 >= rows) break;
    V xv[UNRW][NV], gv[UNRW][NV], yv[UNRW][NV];
#pragma unroll
    for (int u = 0; u < UNRW; ++u)
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int64_t r = r0 + u;
        const int c = (lane + 64 * j) * VN;
        xv[u][j] = vec_zero<T>();
        gv[u][j] = vec_zero<T>();
        yv[u][j] = vec_zero<T>();
        if (r < rows && c < d) {
          xv[u][j] = *reinterpret_cast<const V*>(x + r * d + c);
          yv[u][j] = *reinterpret_cast<const V*>(dy + r * d + c);
          if (gate) gv[u][j] = *reinterpret_cast<const V*>(gate + r * d + c);
        }
      }
#pragma unroll
    for (int u = 0; u < UNRW; ++u) {
      const int64_t r = r0 + u;
      float ss = 0.f, dot = 0.f, uu[NV][VN], sg[NV][VN];
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int e = 0; e < VN; ++e) {
          const float t = to_f32(xv[u][j][e]);
          sg[j][e] = gate ? sigmoidf(to_f32(gv[u][j][e])) : 1.f;
          uu[j][e] = to_f32(yv[u][j][e]) * sg[j][e] * wv[j][e];
          ss += t * t;
          dot += uu[j][e] * t;
        }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) {
        ss += __shfl_xor(ss, m, LNX_WAVE);
        dot += __shfl_xor(dot, m, LNX_WAVE);
      }
      const float rstd = rsqrtf(ss / d + eps);
      const float c = dot * rstd * rstd / d;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int col = (lane + 64 * j) * VN;
        V ox, og;
#pragma unroll
        for (int e = 0; e < VN; ++e) {
          const float t = to_f32(xv[u][j][e]), xn = t * rstd, g = to_f32(yv[u][j][e]);
          ox[e] = from_f32<T>(rstd * (uu[j][e] - t * c));
          og[e] = from_f32<T>(g * xn * wv[j][e] * sg[j][e] * (1.f - sg[j][e]));
          dwv[j][e] += g * xn * sg[j][e];
        }
        if (r < rows && col < d) {
          *reinterpret_cast<V*>(dx + r * d + col) = ox;
          if (gate) *reinterpret_cast<V*>(dgate + r * d + col) = og;
        }
      }
    }
  }
  if (!dw) return;
  // every lane owns its columns: only the four wavefronts of the workgroup are left to add
  __shared__ float red[3][NV * 64 * VN];
  if (wv_i > 0) {
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < VN; ++e) red[wv_i - 1][(lane + 64 * j) * VN + e] = dwv[j][e];
  }
  __syncthreads();
  if (wv_i == 0) {
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < VN; ++e) {
        const int col = (lane + 64 * j) * VN + e;
        if (col < d) dw[(size_t)blockIdx.x * d + col] = dwv[j][e] + red[0][col] + red[1][col] + red[2][col];
      }
  }
}

// Lanes per row of the specialised kernels (rows of 4 .. 64 vectors, a power of two), or 0.
template <typename T> int lanes_for(int d) {
  constexpr int VN = 16 / sizeof(T);
  if (d % VN != 0) return 0;
  const int l = d / VN;
  return (l == 4 || l == 8 || l == 16 || l == 32 || l == 64) ? l : 0;
}

// Vectors per lane of the wide kernels (1, 2 or 4), or 0 when the row is no whole number of vectors or too wide.
template <typename T> int wide_vectors(int d) {
  constexpr int VN = 16 / sizeof(T);
  if (d % VN != 0 || d / VN > 256) return 0;
  const int l = d / VN;
  return l <= 64 ? 1 : l <= 128 ? 2 : 4;
}

#define LNX_LPR_SWITCH(KERNEL, ...)                                                              \
  switch (l) {                                                                                   \
    case 4: hipLaunchKernelGGL((KERNEL<T, 4>), grid, dim3(256), 0, st, __VA_ARGS__); break;      \
    case 8: hipLaunchKernelGGL((KERNEL<T, 8>), grid, dim3(256), 0, st, __VA_ARGS__); break;      \
    case 16: hipLaunchKernelGGL((KERNEL<T, 16>), grid, dim3(256), 0, st, __VA_ARGS__); break;    \
    case 32: hipLaunchKernelGGL((KERNEL<T, 32>), grid, dim3(256), 0, st, __VA_ARGS__); break;    \
    default: hipLaunchKernelGGL((KERNEL<T, 64>), grid, dim3(256), 0, st, __VA_ARGS__); break;    \
  }

#define LNX_NV_SWITCH(KERNEL, ...)                                                               \
  switch (nv) {                                                                                  \
    case 1: hipLaunchKernelGGL((KERNEL<T, 1>), grid, dim3(256), 0, st, __VA_ARGS__); break;      \
    case 2: hipLaunchKernelGGL((KERNEL<T, 2>), grid, dim3(256), 0, st, __VA_ARGS__); break;      \
    default: hipLaunchKernelGGL((KERNEL<T, 4>), grid, dim3(256), 0, st, __VA_ARGS__); break;     \
  }

// l: lanes per row of the specialised kernels, or 0 for the wide ones
template <typename T>
void launch_fwd(int l, int d, const void* x, const void* gate, const float* w, void* y, int64_t rows, float eps, hipStream_t st) {
  if (l) {
    const int64_t waves = (rows + (64 / l) * UNR - 1) / ((64 / l) * UNR);
    dim3 grid((unsigned)((waves + 3) / 4));
    LNX_LPR_SWITCH(rmsnorm_gated_fwd_kernel, (const T*)x, (const T*)gate, w, (T*)y, rows, eps)
  } else {
    const int nv = wide_vectors<T>(d);
    dim3 grid((unsigned)(((rows + UNRW - 1) / UNRW + 3) / 4));
    LNX_NV_SWITCH(rmsnorm_gated_fwd_wide_kernel, (const T*)x, (const T*)gate, w, (T*)y, rows, d, eps)
  }
}

int64_t bwd_blocks(int l, int64_t rows) {
  const int64_t per_wave = l ? (int64_t)(64 / l) * UNR * BWD_STEPS : (int64_t)UNRW * BWD_STEPS;
  return ((rows + per_wave - 1) / per_wave + 3) / 4;
}

template <typename T>
void launch_bwd(int l, int d, const void* x, const void* gate, const float* w, const void* dy, void* dx, void* dgate, float* dw,
                int64_t rows, float eps, hipStream_t st) {
  dim3 grid((unsigned)bwd_blocks(l, rows));
  if (l) {
    LNX_LPR_SWITCH(rmsnorm_gated_bwd_kernel, (const T*)x, (const T*)gate, w, (const T*)dy, (T*)dx, (T*)dgate, dw, rows, eps)
  } else {
    const int nv = wide_vectors<T>(d);
    LNX_NV_SWITCH(rmsnorm_gated_bwd_wide_kernel, (const T*)x, (const T*)gate, w, (const T*)dy, (T*)dx, (T*)dgate, dw, rows, d, eps)
  }
}

int check(const void* x, const float* w, int64_t rows, int d, int dtype) {
  if (rows < 0 || d <= 0) return lnx_set_error(LNX_ERR_SHAPE, "rmsnorm_gated: rows=%lld d=%d", (long long)rows, d);
  if (dtype != LNX_F32 && dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "rmsnorm_gated: dtype %d", dtype);
  const int nv = dtype == LNX_BF16 ? wide_vectors<bf16_t>(d) : wide_vectors<float>(d);
  if (!nv)
    return lnx_set_error(LNX_ERR_SHAPE, "rmsnorm_gated: d=%d must be a whole number of 16-byte vectors, at most 256", d);
  if (!w || (rows > 0 && !x)) return lnx_set_error(LNX_ERR_NULL, "rmsnorm_gated: x and weight are required");
  return LNX_OK;
}

}  // namespace

extern "C" int lnx_rmsnorm_gated_fwd(const void* x, const void* gate, const float* weight, void* y, int64_t rows, int32_t d,
                                     float eps, int32_t dtype, void* hip_stream) {
  if (int rc = check(x, weight, rows, d, dtype)) return rc;
  if (rows == 0) return LNX_OK;
  if (!y) return lnx_set_error(LNX_ERR_NULL, "rmsnorm_gated_fwd: y is NULL");
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  lnx_profile_mark("rmsnorm_gated_fwd", st);
  if (dtype == LNX_BF16) launch_fwd<bf16_t>(lanes_for<bf16_t>(d), d, x, gate, weight, y, rows, eps, st);
  else launch_fwd<float>(lanes_for<float>(d), d, x, gate, weight, y, rows, eps, st);
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "rmsnorm_gated_fwd: %s", hipGetErrorString(e));
}

extern "C" uint64_t lnx_rmsnorm_gated_bwd_workspace_bytes(int64_t rows, int32_t d, int32_t dtype) {
  const int l = dtype == LNX_BF16 ? lanes_for<bf16_t>(d) : lanes_for<float>(d);
  const int nv = dtype == LNX_BF16 ? wide_vectors<bf16_t>(d) : wide_vectors<float>(d);
  if (!nv || rows <= 0) return 0;
  return lnx_sum_rows_bytes(bwd_blocks(l, rows), d);
}

extern "C" int lnx_rmsnorm_gated_bwd(const void* x, const void* gate, const float* weight, const void* dy, void* dx,
                                     void* d_gate, float* d_weight, int64_t rows, int32_t d, float eps, int32_t dtype,
                                     void* workspace, uint64_t workspace_bytes, void* hip_stream) {
  if (int rc = check(x, weight, rows, d, dtype)) return rc;
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int l = dtype == LNX_BF16 ? lanes_for<bf16_t>(d) : lanes_for<float>(d);
  float* part = nullptr;
  if (rows > 0) {
    if (!dy || !dx || (gate && !d_gate)) return lnx_set_error(LNX_ERR_NULL, "rmsnorm_gated_bwd: dy, dx (and d_gate) are required");
    if (d_weight) {
      const uint64_t need = lnx_rmsnorm_gated_bwd_workspace_bytes(rows, d, dtype);
      if (!workspace || workspace_bytes < need)
        return lnx_set_error(LNX_ERR_WORKSPACE, "rmsnorm_gated_bwd: d_weight needs a workspace of %llu bytes", (unsigned long long)need);
      part = static_cast<float*>(workspace);
    }
    lnx_profile_mark("rmsnorm_gated_bwd", st);
    if (dtype == LNX_BF16) launch_bwd<bf16_t>(l, d, x, gate, weight, dy, dx, d_gate, part, rows, eps, st);
    else launch_bwd<float>(l, d, x, gate, weight, dy, dx, d_gate, part, rows, eps, st);
  }
  if (d_weight) {
    lnx_profile_mark("rmsnorm_dweight", st);
    lnx_sum_rows(part, rows > 0 ? bwd_blocks(l, rows) : 0, d, d_weight, st);
  }
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "rmsnorm_gated_bwd: %s", hipGetErrorString(e));
}
