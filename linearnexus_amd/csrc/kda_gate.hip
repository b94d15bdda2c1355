// KDA's gate activation and its gradient (linearnexus/modules/linear_attn/kda.py:120-172):
//   g_out[r, h, c] = -exp(A_log[h]) * softplus(g[r, h*dk + c] + g_bias[h*dk + c]),  softplus(x) = x for x > threshold,
//   beta_out = sigmoid(beta)
// Elementwise streaming kernels over [rows, H*dk]; the output can be written in fp32 directly, which is what the
// KDA scan reads (the reference casts to the input dtype, kda.py:172, and the scan casts back to fp32, kda.py:393).
// The backward keeps per-channel sums of d_bias and of d_out * out in registers over a run of rows, writes them as
// partial rows to a workspace and finishes them with the shared column-sum kernel: no atomics.
#include "lnx_common.h"
#include "reduce_rows.h"

namespace {

constexpr int RUN = 8;       // rows whose loads are in flight together, per thread (all of a forward thread's rows)
constexpr int BWD_RUN = 32;  // rows per thread in the backward: one partial row of parameter sums per BWD_RUN rows

struct GateParams {
  const void* g; const float* A_log; const float* bias; void* out;
  const void* d_out; void* d_g; float* part;  // part: [2][nruns][D]
  int64_t rows; int D, dk; float threshold; int nruns;
};

template <typename T, int N> struct VecT { typedef T raw __attribute__((ext_vector_type(N))); };

template <typename T, int N> __device__ __forceinline__ void ldv(const T* p, float (&o)[N]) {
  typename VecT<T, N>::raw r = *reinterpret_cast<const typename VecT<T, N>::raw*>(p);
#pragma unroll
  for (int i = 0; i < N; ++i) o[i] = (float)r[i];
}
template <typename T, int N> __device__ __forceinline__ void stv(T* p, const float (&v)[N]) {
  typename VecT<T, N>::raw r;
#pragma unroll
  for (int i = 0; i < N; ++i) r[i] = from_f32<T>(v[i]);
  *reinterpret_cast<typename VecT<T, N>::raw*>(p) = r;
}

// log(1 + e^x) in the overflow-free form max(x, 0) + log1p(e^-|x|); x itself above the threshold (kda.py:157-163)
__device__ __forceinline__ float softplus_thr(float x, float thr) {
  return x > thr ? x : fmaxf(x, 0.f) + __logf(1.f + __expf(-fabsf(x)));
}

// thread = (4 channels, run of RUN rows); 4 loads in flight per thread
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void kda_gate_fwd_kernel(GateParams p) {
  constexpr int N = 4;
  const int c = (blockIdx.x * 256 + threadIdx.x) * N;
  if (c >= p.D) return;
  const int64_t r0 = (int64_t)blockIdx.y * RUN, r1 = min(r0 + RUN, p.rows);
  const float na = -__expf(p.A_log[c / p.dk]);
  float b[N];
#pragma unroll
  for (int i = 0; i < N; ++i) b[i] = p.bias ? p.bias[c + i] : 0.f;
  const TI* gp = static_cast<const TI*>(p.g) + r0 * p.D + c;
  TO* op = static_cast<TO*>(p.out) + r0 * p.D + c;
  if (r1 - r0 == RUN) {
    float x[RUN][N];
#pragma unroll
    for (int u = 0; u < RUN; ++u) ldv<TI, N>(gp + (int64_t)u * p.D, x[u]);
#pragma unroll
    for (int u = 0; u < RUN; ++u) {
#pragma unroll
      for (int i = 0; i < N; ++i) x[u][i] = na * softplus_thr(x[u][i] + b[i], p.threshold);
      stv<TO, N>(op + (int64_t)u * p.D, x[u]);
    }
    return;
  }
  for (int64_t r = r0; r < r1; ++r, gp += p.D, op += p.D) {
    float x[N];
    ldv<TI, N>(gp, x);
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] = na * softplus_thr(x[i] + b[i], p.threshold);
    stv<TO, N>(op, x);
  }
}

// d_g = d_out * (-e^A) * softplus'(x);  per channel: sum d_g (d_bias) and sum d_out * out (d_A_log before the sum
// over the head's channels)
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void kda_gate_bwd_kernel(GateParams p) {
  constexpr int N = 4;
  const int c = (blockIdx.x * 256 + threadIdx.x) * N;
  if (c >= p.D) return;
  const int64_t r0 = (int64_t)blockIdx.y * BWD_RUN, r1 = min(r0 + BWD_RUN, p.rows);
  const float na = -__expf(p.A_log[c / p.dk]);
  float b[N], sb[N], sa[N];
#pragma unroll
  for (int i = 0; i < N; ++i) b[i] = p.bias ? p.bias[c + i] : 0.f, sb[i] = 0.f, sa[i] = 0.f;
  const TI* gp = static_cast<const TI*>(p.g) + r0 * p.D + c;
  const TO* dp = static_cast<const TO*>(p.d_out) + r0 * p.D + c;
  TI* op = static_cast<TI*>(p.d_g) + r0 * p.D + c;
  auto row = [&](float (&x)[N], float (&d)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      // one exponential serves both: softplus(t) = max(t, 0) + log(1 + e), sigmoid(t) = (t >= 0 ? 1 : e) / (1 + e), e = e^-|t|
      const float t = x[i] + b[i];
      const bool lin = t > p.threshold;
      const float e = __expf(-fabsf(t)), rc = __builtin_amdgcn_rcpf(1.f + e);
      const float sp = lin ? t : fmaxf(t, 0.f) + __logf(1.f + e), ds = lin ? 1.f : (t >= 0.f ? rc : e * rc);
      sa[i] += d[i] * na * sp;
      x[i] = d[i] * na * ds;
      sb[i] += x[i];
    }
  };
  int64_t r = r0;
  for (; r + RUN <= r1; r += RUN) {
    float x[RUN][N], d[RUN][N];
#pragma unroll
    for (int u = 0; u < RUN; ++u) {
      ldv<TI, N>(gp + (int64_t)u * p.D, x[u]);
      ldv<TO, N>(dp + (int64_t)u * p.D, d[u]);
    }
#pragma unroll
    for (int u = 0; u < RUN; ++u) {
      row(x[u], d[u]);
      stv<TI, N>(op + (int64_t)u * p.D, x[u]);
    }
    gp += (int64_t)RUN * p.D, dp += (int64_t)RUN * p.D, op += (int64_t)RUN * p.D;
  }
  for (; r < r1; ++r, gp += p.D, dp += p.D, op += p.D) {
    float x[N], d[N];
    ldv<TI, N>(gp, x);
    ldv<TO, N>(dp, d);
    row(x, d);
    stv<TI, N>(op, x);
  }
  if (p.part) {
    store4(p.part + (int64_t)blockIdx.y * p.D + c, floatx4{sb[0], sb[1], sb[2], sb[3]});
    store4(p.part + ((int64_t)p.nruns + LNX_SUM_SLICES + blockIdx.y) * p.D + c, floatx4{sa[0], sa[1], sa[2], sa[3]});
  }
}

// out[h] = sum of in[h * dk .. h * dk + dk - 1]; one wavefront per head
__global__ __launch_bounds__(64) void sum_heads_kernel(const float* in, int dk, float* out) {
  float t = 0.f;
  for (int i = threadIdx.x; i < dk; i += 64) t += in[(int64_t)blockIdx.x * dk + i];
  t = wave_sum(t);
  if (threadIdx.x == 0) out[blockIdx.x] = t;
}

__global__ void zero_kernel(float* a, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) a[i] = 0.f;
}

__global__ void sigmoid_fwd_kernel(const float* x, float* y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = 1.f / (1.f + __expf(-x[i]));
}

__global__ void sigmoid_bwd_kernel(const float* y, const float* dy, float* dx, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dx[i] = dy[i] * y[i] * (1.f - y[i]);
}

int check(int64_t rows, int H, int dk, int dtype, int out_dtype) {
  if (rows < 0 || H <= 0 || dk <= 0 || dk % 4 != 0)
    return lnx_set_error(LNX_ERR_SHAPE, "kda_gate: rows=%lld H=%d dk=%d (dk must be a multiple of 4)", (long long)rows, H, dk);
  if ((dtype != LNX_F32 && dtype != LNX_BF16) || (out_dtype != LNX_F32 && out_dtype != LNX_BF16))
    return lnx_set_error(LNX_ERR_DTYPE, "kda_gate: dtype %d / out dtype %d", dtype, out_dtype);
  return LNX_OK;
}

#define LNX_GATE_DISPATCH(KERNEL)                                                                  \
  if (dtype == LNX_BF16 && out_dtype == LNX_BF16) KERNEL<bf16_t, bf16_t><<<grid, 256, 0, st>>>(p); \
  else if (dtype == LNX_BF16) KERNEL<bf16_t, float><<<grid, 256, 0, st>>>(p);                      \
  else if (out_dtype == LNX_BF16) KERNEL<float, bf16_t><<<grid, 256, 0, st>>>(p);                  \
  else KERNEL<float, float><<<grid, 256, 0, st>>>(p)

}  // namespace

extern "C" int lnx_kda_gate_fwd(const void* g, const float* A_log, const float* g_bias, void* g_out, int64_t rows, int32_t H,
                                int32_t dk, float threshold, int32_t dtype, int32_t out_dtype, void* hip_stream) {
  if (int rc = check(rows, H, dk, dtype, out_dtype)) return rc;
  if (rows == 0) return LNX_OK;
  if (!g || !A_log || !g_out) return lnx_set_error(LNX_ERR_NULL, "kda_gate_fwd: g, A_log and g_out are required");
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int D = H * dk, nruns = (int)((rows + RUN - 1) / RUN);
  GateParams p{g, A_log, g_bias, g_out, nullptr, nullptr, nullptr, rows, D, dk, threshold, nruns};
  dim3 grid((D / 4 + 255) / 256, nruns);
  lnx_profile_mark("kda_gate_fwd", st);
  LNX_GATE_DISPATCH(kda_gate_fwd_kernel);
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "kda_gate_fwd: %s", hipGetErrorString(e));
}

extern "C" uint64_t lnx_kda_gate_bwd_workspace_bytes(int64_t rows, int32_t H, int32_t dk) {
  if (rows <= 0 || H <= 0 || dk <= 0) return 0;
  const int64_t nruns = (rows + BWD_RUN - 1) / BWD_RUN;
  return 2 * lnx_sum_rows_bytes(nruns, H * dk) + (uint64_t)H * dk * sizeof(float);
}

extern "C" int lnx_kda_gate_bwd(const void* g, const float* A_log, const float* g_bias, const void* d_out, void* d_g,
                                float* d_A_log, float* d_bias, int64_t rows, int32_t H, int32_t dk, float threshold,
                                int32_t dtype, int32_t out_dtype, void* workspace, uint64_t workspace_bytes, void* hip_stream) {
  if (int rc = check(rows, H, dk, dtype, out_dtype)) return rc;
  if (!A_log) return lnx_set_error(LNX_ERR_NULL, "kda_gate_bwd: A_log is required");
  if (rows > 0 && (!g || !d_out || !d_g)) return lnx_set_error(LNX_ERR_NULL, "kda_gate_bwd: g, d_out and d_g are required");
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int D = H * dk, nruns = (int)((rows + BWD_RUN - 1) / BWD_RUN);
  const bool sums = d_A_log || d_bias;
  float* part = nullptr;
  if (sums && rows > 0) {
    const uint64_t need = lnx_kda_gate_bwd_workspace_bytes(rows, H, dk);
    if (!workspace || workspace_bytes < need)
      return lnx_set_error(LNX_ERR_WORKSPACE, "kda_gate_bwd: parameter gradients need a workspace of %llu bytes", (unsigned long long)need);
    part = static_cast<float*>(workspace);
  }
  if (rows > 0) {
    GateParams p{g, A_log, g_bias, nullptr, d_out, d_g, part, rows, D, dk, threshold, nruns};
    dim3 grid((D / 4 + 255) / 256, nruns);
    lnx_profile_mark("kda_gate_bwd", st);
    LNX_GATE_DISPATCH(kda_gate_bwd_kernel);
  }
  if (sums) {
    lnx_profile_mark("kda_gate_sums", st);
    if (rows > 0) {
      float* part_a = part + ((int64_t)nruns + LNX_SUM_SLICES) * D;
      float* chan = part_a + ((int64_t)nruns + LNX_SUM_SLICES) * D;  // [D] per-channel sum of d_out * out
      if (d_bias) lnx_sum_rows(part, nruns, D, d_bias, st);
      if (d_A_log) {
        lnx_sum_rows(part_a, nruns, D, chan, st);
        sum_heads_kernel<<<H, 64, 0, st>>>(chan, dk, d_A_log);
      }
    } else {  // no rows: the sums are zero
      if (d_bias) zero_kernel<<<(D + 255) / 256, 256, 0, st>>>(d_bias, D);
      if (d_A_log) zero_kernel<<<(H + 255) / 256, 256, 0, st>>>(d_A_log, H);
    }
  }
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "kda_gate_bwd: %s", hipGetErrorString(e));
}

// Parameter gradients of the gate activation fused into the chunk kernels: `part` holds two [nrows x H*dk] matrices of
// per-chunk partial sums (d_bias parts, then d_out * out parts), each followed by its first-level sums, and H*dk floats
// of per-channel scratch -- lnx_gate_part_bytes(nrows, H * dk) bytes in all.
uint64_t lnx_gate_part_bytes(int64_t nrows, int D) { return 2 * lnx_sum_rows_bytes(nrows, D) + (uint64_t)D * sizeof(float); }

void lnx_gate_finish_sums(float* part, int64_t nrows, int H, int dk, float* d_A_log, float* d_bias, hipStream_t st) {
  const int D = H * dk;
  float* part_a = part + (nrows + LNX_SUM_SLICES) * D;
  float* chan = part_a + (nrows + LNX_SUM_SLICES) * D;
  lnx_profile_mark("kda_gate_sums", st);
  if (d_bias) lnx_sum_rows(part, nrows, D, d_bias, st);
  if (d_A_log) {
    lnx_sum_rows(part_a, nrows, D, chan, st);
    sum_heads_kernel<<<H, 64, 0, st>>>(chan, dk, d_A_log);
  }
}

extern "C" int lnx_sigmoid_fwd(const float* x, float* y, int64_t n, void* hip_stream) {
  if (n < 0) return lnx_set_error(LNX_ERR_SHAPE, "sigmoid: n=%lld", (long long)n);
  if (n == 0) return LNX_OK;
  if (!x || !y) return lnx_set_error(LNX_ERR_NULL, "sigmoid_fwd: NULL tensor");
  sigmoid_fwd_kernel<<<(unsigned)((n + 255) / 256), 256, 0, static_cast<hipStream_t>(hip_stream)>>>(x, y, n);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "sigmoid_fwd: %s", hipGetErrorString(e));
}

extern "C" int lnx_sigmoid_bwd(const float* y, const float* dy, float* dx, int64_t n, void* hip_stream) {
  if (n < 0) return lnx_set_error(LNX_ERR_SHAPE, "sigmoid: n=%lld", (long long)n);
  if (n == 0) return LNX_OK;
  if (!y || !dy || !dx) return lnx_set_error(LNX_ERR_NULL, "sigmoid_bwd: NULL tensor");
  sigmoid_bwd_kernel<<<(unsigned)((n + 255) / 256), 256, 0, static_cast<hipStream_t>(hip_stream)>>>(y, dy, dx, n);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "sigmoid_bwd: %s", hipGetErrorString(e));
}
