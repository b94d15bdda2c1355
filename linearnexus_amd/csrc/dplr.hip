// RWKV-7's diagonal-plus-low-rank delta rule, token by token in fp32, with the same register-slab design as
// the delta-rule token kernels: one wavefront keeps a [dk x 32]-column slab of the state in registers
// (lane = (row group, 4 columns)) and finishes the two column reductions with three xor-shuffles.
//
// Per token (w = exp(gk), q~ = scale * q), restating linearnexus/modules/linear_attn/rwkv7.py:171-196:
//   u = h^T a;   h <- w (.) h + b u^T + k v^T;   o = h^T q~ = (w (.) h_old)^T q~ + <b,q~> u + <k,q~> v
// so both reductions run over the old state in one pass.
#include "lnx_common.h"

namespace {

struct DplrParams {
  const void *q, *k, *v, *a, *b;
  const float* gk;
  const float* s_in;
  float* s_out;
  void* o;
  int H, T, dv;
  float scale;
  int o_dtype;
};

__device__ __forceinline__ floatx4 rowgroup_sum(floatx4 x) {
#pragma unroll
  for (int m = 8; m <= 32; m <<= 1) {
    x[0] += __shfl_xor(x[0], m, LNX_WAVE);
    x[1] += __shfl_xor(x[1], m, LNX_WAVE);
    x[2] += __shfl_xor(x[2], m, LNX_WAVE);
    x[3] += __shfl_xor(x[3], m, LNX_WAVE);
  }
  return x;
}

// Loads the five dk-vectors of one token with a full wavefront into sm ([5][DK]: q~, k, a, b, w) and returns
// (<b,q~>, <k,q~>).
template <typename T, int DK>
__device__ __forceinline__ floatx2 stage_token(const T* qp, const T* kp, const T* ap, const T* bp, const float* gp,
                                               float* sm, int lane, float scale) {
  float bq = 0.f, kq = 0.f;
#pragma unroll
  for (int e = 0; e < (DK + 63) / 64; ++e) {
    const int idx = lane + 64 * e;
    if (idx < DK) {
      const float qv = to_f32(qp[idx]) * scale, kv = to_f32(kp[idx]), bv = to_f32(bp[idx]);
      sm[idx] = qv;
      sm[DK + idx] = kv;
      sm[2 * DK + idx] = to_f32(ap[idx]);
      sm[3 * DK + idx] = bv;
      sm[4 * DK + idx] = expf(gp[idx]);
      bq += bv * qv;
      kq += kv * qv;
    }
  }
  floatx2 r = {wave_sum(bq), wave_sum(kq)};
  return r;
}

template <int DK>
__device__ __forceinline__ floatx4 apply_token(floatx4 (&S)[DK / 8], const float* sm, int row0, floatx4 v4, floatx2 dots) {
  constexpr int RPL = DK / 8;
  floatx4 u = {0.f, 0.f, 0.f, 0.f}, pq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    u += S[i] * sm[2 * DK + row0 + i];
    S[i] *= sm[4 * DK + row0 + i];
    pq += S[i] * sm[row0 + i];
  }
  u = rowgroup_sum(u);
  pq = rowgroup_sum(pq);
#pragma unroll
  for (int i = 0; i < RPL; ++i) S[i] += u * sm[3 * DK + row0 + i] + v4 * sm[DK + row0 + i];
  return pq + u * dots[0] + v4 * dots[1];
}

__device__ __forceinline__ void store_o4(void* o, int64_t idx, floatx4 x, int o_dtype) {
  if (o_dtype == LNX_BF16) store4(reinterpret_cast<bf16_t*>(o) + idx, x);
  else store4(reinterpret_cast<float*>(o) + idx, x);
}

// Single token.  grid (B*H, ceil(dv/128)), block 256: wave w owns columns [32*(4*blockIdx.y+w), +32).
template <typename T, int DK>
__global__ __launch_bounds__(256) void dplr_step_kernel(DplrParams p) {
  constexpr int RPL = DK / 8;
  __shared__ float sm_all[4][5 * DK];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t bh = blockIdx.x;
  float* sm = sm_all[wave];
  const T *q = static_cast<const T*>(p.q), *k = static_cast<const T*>(p.k), *a = static_cast<const T*>(p.a),
          *b = static_cast<const T*>(p.b);
  const floatx2 dots = stage_token<T, DK>(q + bh * DK, k + bh * DK, a + bh * DK, b + bh * DK, p.gk + bh * DK, sm, lane, p.scale);
  __syncthreads();
  const int col0 = (blockIdx.y * 4 + wave) * 32 + (lane & 7) * 4;
  if (col0 >= p.dv) return;
  const int row0 = (lane >> 3) * RPL;
  const int64_t sbase = (bh * DK + row0) * p.dv + col0;
  floatx4 S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i)
    S[i] = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(p.s_in + sbase + (int64_t)i * p.dv));
  const floatx4 v4 = load4(static_cast<const T*>(p.v) + bh * p.dv + col0);
  const floatx4 o4 = apply_token<DK>(S, sm, row0, v4, dots);
#pragma unroll
  for (int i = 0; i < RPL; ++i)
    __builtin_nontemporal_store(S[i], reinterpret_cast<floatx4*>(p.s_out + sbase + (int64_t)i * p.dv));
  if ((lane >> 3) == 0) store_o4(p.o, bh * p.dv + col0, o4, p.o_dtype);
}

// Scan over T.  grid (B*H, ceil(dv/32)), block 64: one wavefront per 32-column slab.
template <typename T, int DK>
__global__ __launch_bounds__(64) void dplr_recurrent_kernel(DplrParams p) {
  constexpr int RPL = DK / 8;
  __shared__ float sm[5 * DK];
  const int lane = threadIdx.x;
  const int64_t bh = blockIdx.x;
  const int col0 = blockIdx.y * 32 + (lane & 7) * 4;
  const bool active = col0 < p.dv;
  const int ccol = active ? col0 : 0;
  const int row0 = (lane >> 3) * RPL;
  const int64_t sbase = (bh * DK + row0) * p.dv + ccol;
  floatx4 S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    if (p.s_in && active) S[i] = load4(p.s_in + sbase + (int64_t)i * p.dv);
    else S[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const int64_t tok0 = bh * p.T;
  const T *q = static_cast<const T*>(p.q) + tok0 * DK, *k = static_cast<const T*>(p.k) + tok0 * DK,
          *a = static_cast<const T*>(p.a) + tok0 * DK, *b = static_cast<const T*>(p.b) + tok0 * DK;
  const T* v = static_cast<const T*>(p.v) + tok0 * p.dv + ccol;
  const float* gk = p.gk + tok0 * DK;
  for (int t = 0; t < p.T; ++t) {
    const int64_t r = (int64_t)t * DK;
    const floatx4 v4 = load4(v + (int64_t)t * p.dv);
    __syncthreads();  // the previous token's reads of sm are done
    const floatx2 dots = stage_token<T, DK>(q + r, k + r, a + r, b + r, gk + r, sm, lane, p.scale);
    __syncthreads();
    const floatx4 o4 = apply_token<DK>(S, sm, row0, v4, dots);
    if ((lane >> 3) == 0 && active) store_o4(p.o, (tok0 + t) * p.dv + col0, o4, p.o_dtype);
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) store4(p.s_out + sbase + (int64_t)i * p.dv, S[i]);
  }
}

template <typename T>
int launch(bool step, int dk, const DplrParams& p, dim3 grid, hipStream_t st) {
#define LNX_DPLR(D)                                                                     \
  case D:                                                                               \
    if (step) hipLaunchKernelGGL((dplr_step_kernel<T, D>), grid, dim3(256), 0, st, p);  \
    else hipLaunchKernelGGL((dplr_recurrent_kernel<T, D>), grid, dim3(64), 0, st, p);   \
    return LNX_OK
  switch (dk) {
    LNX_DPLR(8); LNX_DPLR(16); LNX_DPLR(32); LNX_DPLR(64); LNX_DPLR(128);
    default: return lnx_set_error(LNX_ERR_SHAPE, "dplr kernels need dk in {8,16,32,64,128}, got %d", dk);
  }
#undef LNX_DPLR
}

int entry(bool step, const lnx_dplr_args* a, void* stream) {
  if (!a) return lnx_set_error(LNX_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->H <= 0 || a->dk <= 0 || a->dv <= 0 || (!step && a->T < 0))
    return lnx_set_error(LNX_ERR_SHAPE, "bad dimensions B=%d H=%d T=%d dk=%d dv=%d", a->B, a->H, a->T, a->dk, a->dv);
  const bool tokens = a->B > 0 && (step || a->T > 0);
  if ((tokens && (!a->q || !a->k || !a->v || !a->a || !a->b || !a->gk || !a->o)) || (a->B > 0 && !a->final_state))
    return lnx_set_error(LNX_ERR_NULL, "q, k, v, a, b, gk, o and final_state are required");
  if (step && a->B > 0 && !a->initial_state) return lnx_set_error(LNX_ERR_NULL, "the step needs the current state");
  if (a->dv % 4 != 0) return lnx_set_error(LNX_ERR_SHAPE, "dv must be a multiple of 4, got %d", a->dv);
  if (a->dtype != LNX_F32 && a->dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "dtype %d", a->dtype);
  if (a->o_dtype != LNX_F32 && a->o_dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "o_dtype %d", a->o_dtype);
  if (a->B == 0) return LNX_OK;
  DplrParams p{a->q, a->k, a->v, a->a, a->b, a->gk, a->initial_state, a->final_state, a->o,
               a->H, a->T, a->dv, a->scale, a->o_dtype};
  dim3 grid((unsigned)((int64_t)a->B * a->H), (unsigned)((a->dv + (step ? 127 : 31)) / (step ? 128 : 32)));
  hipStream_t st = static_cast<hipStream_t>(stream);
  lnx_profile_mark(step ? "dplr_step" : "dplr_recurrent", st);
  const int rc = a->dtype == LNX_BF16 ? launch<bf16_t>(step, a->dk, p, grid, st) : launch<float>(step, a->dk, p, grid, st);
  lnx_profile_mark(nullptr, st);
  if (rc != LNX_OK) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "dplr kernel launch: %s", hipGetErrorString(e));
  return LNX_OK;
}

}  // namespace

extern "C" int lnx_dplr_step(const lnx_dplr_args* a, void* hip_stream) { return entry(true, a, hip_stream); }
extern "C" int lnx_dplr_recurrent_fwd(const lnx_dplr_args* a, void* hip_stream) { return entry(false, a, hip_stream); }
