// Gated DeltaNet's gate and learning-rate activations and their gradient
// (linearnexus/modules/linear_attn/gated_deltanet.py:804-815):
//   g[r, h]    = -exp(A_log[h]) * softplus(a[r, h] + dt_bias[h])        fp32 log-decay per token and head
//   beta[r, h] = beta_scale * sigmoid(b[r, h])                          beta_scale = 2 with allow_neg_eigval, else 1
// a and b are the [rows, H] outputs of the block's a_proj / b_proj in the activation dtype; g and beta leave in fp32,
// the type the scan kernels read.  Two megabytes at the benchmark shapes: one streaming kernel each way.  The
// backward keeps the per-head sums for d_A_log and d_dt_bias in registers over a run of rows, writes them as partial
// rows to a caller-owned workspace and finishes them with the shared column-sum kernel (no atomics, deterministic).
#include "lnx_common.h"
#include "reduce_rows.h"

namespace {

constexpr int RUN = 64;  // rows per thread

struct GdnGateParams {
  const void* a; const void* b; const float* A_log; const float* dt_bias;
  float* g; float* beta;
  const float* d_g; const float* d_beta; void* d_a; void* d_b; float* part;  // part: [2][nruns + slices][Hp]
  int64_t rows; int H, Hp, nruns; float beta_scale;
};

// log(1 + e^x) in the overflow-free form max(x, 0) + log1p(e^-|x|) (what jax.nn.softplus evaluates)
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(__expf(-fabsf(x))); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + __expf(-x)); }

// thread = (head, run of RUN rows): consecutive lanes take consecutive heads of a row, so a wavefront reads whole rows
template <typename T>
__global__ __launch_bounds__(256) void gdn_gate_fwd_kernel(GdnGateParams p) {
  const int h = blockIdx.x * 256 + threadIdx.x;
  if (h >= p.H) return;
  const int64_t r0 = (int64_t)blockIdx.y * RUN, r1 = min(r0 + RUN, p.rows);
  const float na = -__expf(p.A_log[h]), bias = p.dt_bias ? p.dt_bias[h] : 0.f;
  const T* a = static_cast<const T*>(p.a);
  const T* b = static_cast<const T*>(p.b);
  for (int64_t r = r0; r < r1; ++r) {
    const int64_t i = r * p.H + h;
    p.g[i] = na * softplus_f(to_f32(a[i]) + bias);
    if (b) p.beta[i] = p.beta_scale * sigmoid_f(to_f32(b[i]));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gdn_gate_bwd_kernel(GdnGateParams p) {
  const int h = blockIdx.x * 256 + threadIdx.x;
  if (h >= p.Hp) return;
  float sb = 0.f, sa = 0.f;
  if (h < p.H) {
    const int64_t r0 = (int64_t)blockIdx.y * RUN, r1 = min(r0 + RUN, p.rows);
    const float na = -__expf(p.A_log[h]), bias = p.dt_bias ? p.dt_bias[h] : 0.f;
    const T* a = static_cast<const T*>(p.a);
    const T* b = static_cast<const T*>(p.b);
    T* da = static_cast<T*>(p.d_a);
    T* db = static_cast<T*>(p.d_b);
    for (int64_t r = r0; r < r1; ++r) {
      const int64_t i = r * p.H + h;
      const float x = to_f32(a[i]) + bias, dg = p.d_g ? p.d_g[i] : 0.f;
      const float dx = dg * na * sigmoid_f(x);  // softplus' = sigmoid
      sa += dg * na * softplus_f(x);            // d g / d A_log = g
      sb += dx;
      da[i] = from_f32<T>(dx);
      if (b) {
        const float s = sigmoid_f(to_f32(b[i]));
        db[i] = from_f32<T>((p.d_beta ? p.d_beta[i] : 0.f) * p.beta_scale * s * (1.f - s));
      }
    }
  }
  if (p.part) {  // columns H .. Hp - 1 pad the partial rows to whole 16-byte vectors
    p.part[(int64_t)blockIdx.y * p.Hp + h] = sb;
    p.part[((int64_t)p.nruns + LNX_SUM_SLICES + blockIdx.y) * p.Hp + h] = sa;
  }
}

__global__ void copy_heads_kernel(const float* in, float* out, int H) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < H) out[i] = in[i];
}

__global__ void zero_heads_kernel(float* a, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) a[i] = 0.f;
}

int check(int64_t rows, int H, int dtype) {
  if (rows < 0 || H <= 0) return lnx_set_error(LNX_ERR_SHAPE, "gdn_gate: rows=%lld H=%d", (long long)rows, H);
  if (dtype != LNX_F32 && dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "gdn_gate: dtype %d", dtype);
  return LNX_OK;
}

}  // namespace

extern "C" int lnx_gdn_gate_fwd(const void* a, const void* b, const float* A_log, const float* dt_bias, float* g, float* beta,
                                int64_t rows, int32_t H, float beta_scale, int32_t dtype, void* hip_stream) {
  if (int rc = check(rows, H, dtype)) return rc;
  if (rows == 0) return LNX_OK;
  if (!a || !A_log || !g || (b && !beta)) return lnx_set_error(LNX_ERR_NULL, "gdn_gate_fwd: a, A_log and g are required (beta with b)");
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int nruns = (int)((rows + RUN - 1) / RUN);
  GdnGateParams p{a, b, A_log, dt_bias, g, beta, nullptr, nullptr, nullptr, nullptr, nullptr, rows, H, H, nruns, beta_scale};
  dim3 grid((H + 255) / 256, nruns);
  lnx_profile_mark("gdn_gate_fwd", st);
  if (dtype == LNX_BF16) gdn_gate_fwd_kernel<bf16_t><<<grid, 256, 0, st>>>(p);
  else gdn_gate_fwd_kernel<float><<<grid, 256, 0, st>>>(p);
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "gdn_gate_fwd: %s", hipGetErrorString(e));
}

extern "C" uint64_t lnx_gdn_gate_bwd_workspace_bytes(int64_t rows, int32_t H) {
  if (rows <= 0 || H <= 0) return 0;
  const int Hp = (H + 3) & ~3;
  return 2 * lnx_sum_rows_bytes((rows + RUN - 1) / RUN, Hp) + 2 * (uint64_t)Hp * sizeof(float);
}

extern "C" int lnx_gdn_gate_bwd(const void* a, const void* b, const float* A_log, const float* dt_bias, const float* d_g,
                                const float* d_beta, void* d_a, void* d_b, float* d_A_log, float* d_dt_bias, int64_t rows,
                                int32_t H, float beta_scale, int32_t dtype, void* workspace, uint64_t workspace_bytes,
                                void* hip_stream) {
  if (int rc = check(rows, H, dtype)) return rc;
  if (!A_log) return lnx_set_error(LNX_ERR_NULL, "gdn_gate_bwd: A_log is required");
  if (rows > 0 && (!a || !d_a || (b && !d_b))) return lnx_set_error(LNX_ERR_NULL, "gdn_gate_bwd: a and d_a are required (d_b with b)");
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int Hp = (H + 3) & ~3, nruns = (int)((rows + RUN - 1) / RUN);
  const bool sums = d_A_log || d_dt_bias;
  float* part = nullptr;
  if (sums && rows > 0) {
    const uint64_t need = lnx_gdn_gate_bwd_workspace_bytes(rows, H);
    if (!workspace || workspace_bytes < need)
      return lnx_set_error(LNX_ERR_WORKSPACE, "gdn_gate_bwd: parameter gradients need a workspace of %llu bytes", (unsigned long long)need);
    part = static_cast<float*>(workspace);
  }
  lnx_profile_mark("gdn_gate_bwd", st);
  if (rows > 0) {
    GdnGateParams p{a, b, A_log, dt_bias, nullptr, nullptr, d_g, d_beta, d_a, d_b, part, rows, H, Hp, nruns, beta_scale};
    dim3 grid((Hp + 255) / 256, nruns);
    if (dtype == LNX_BF16) gdn_gate_bwd_kernel<bf16_t><<<grid, 256, 0, st>>>(p);
    else gdn_gate_bwd_kernel<float><<<grid, 256, 0, st>>>(p);
    if (sums) {
      float* part_a = part + ((int64_t)nruns + LNX_SUM_SLICES) * Hp;
      float* tot = part_a + ((int64_t)nruns + LNX_SUM_SLICES) * Hp;  // [2][Hp]
      if (d_dt_bias) {
        lnx_sum_rows(part, nruns, Hp, tot, st);
        copy_heads_kernel<<<(H + 255) / 256, 256, 0, st>>>(tot, d_dt_bias, H);
      }
      if (d_A_log) {
        lnx_sum_rows(part_a, nruns, Hp, tot + Hp, st);
        copy_heads_kernel<<<(H + 255) / 256, 256, 0, st>>>(tot + Hp, d_A_log, H);
      }
    }
  } else if (sums) {  // no rows: the sums are zero
    if (d_dt_bias) zero_heads_kernel<<<(H + 255) / 256, 256, 0, st>>>(d_dt_bias, H);
    if (d_A_log) zero_heads_kernel<<<(H + 255) / 256, 256, 0, st>>>(d_A_log, H);
  }
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LNX_OK : lnx_set_error(LNX_ERR_LAUNCH, "gdn_gate_bwd: %s", hipGetErrorString(e));
}
