// Token-level delta-rule kernels in fp32: the single-token decode step and the
// token-by-token scan.  Both keep a [dk x 32]-column slab of the state in the registers
// of one wavefront: lane = (row group, 4 columns), so a state row segment is read and
// written as 128 contiguous bytes and the two column reductions (S'^T k and S'^T q) are
// finished with three xor-shuffles inside the wavefront -- no LDS traffic for the state.
//
// Arithmetic per token (alpha = exp(g): 1, a scalar, or a dk-vector):
//   S' = alpha * S;  d = beta (v - S'^T k);  S = S' + k d^T;  o = S^T q~ = S'^T q~ + <q~,k> d
// which restates linearnexus/modules/linear_attn/delta_net.py:189-198,
// gated_deltanet.py:200-213 and kda.py:251-267 (KDA's beta-on-k form is the same product).

#include "lnx_common.h"

namespace {

struct TokenParams {
  const void* q;
  const void* k;
  const void* v;
  const float* beta;
  const float* g;
  const float* s_in;
  float* s_out;
  void* o;
  const int32_t* cu_seqlens;
  int H, T, dv;
  int ts;  // distance between consecutive tokens of a (batch, head) row, in tokens: 1 ([B,H,T,.]) or H ([B,T,H,.])
  float scale;
  int l2norm;
  int o_dtype;
};

template <int DK> struct Lanes {
  static constexpr int RPL = DK / 8;            // state rows per lane
  static constexpr int EPL = (DK + 63) / 64;    // q/k elements per lane when a wave loads a row
};

// Reduces over the 8 row groups (lane bits 3..5); all lanes get the column totals.
__device__ __forceinline__ floatx4 rowgroup_sum(floatx4 x) {
#pragma unroll
  for (int c = 0; c < 4; ++c)
    x[c] += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x[c]), 0x128, 0xF, 0xF, true));  // row_ror:8 = lane ^ 8
#pragma unroll
  for (int m = 16; m <= 32; m <<= 1) {
    x[0] += __shfl_xor(x[0], m, LNX_WAVE);
    x[1] += __shfl_xor(x[1], m, LNX_WAVE);
    x[2] += __shfl_xor(x[2], m, LNX_WAVE);
    x[3] += __shfl_xor(x[3], m, LNX_WAVE);
  }
  return x;
}

__device__ __forceinline__ void store_o4(void* o, int64_t idx, floatx4 x, int o_dtype) {
  if (o_dtype == LNX_BF16) store4(reinterpret_cast<bf16_t*>(o) + idx, x);
  else store4(reinterpret_cast<float*>(o) + idx, x);
}

// One q/k row pair (and the gate row of a vector gate) in the registers of a wavefront, as loaded: the scan fetches a
// token's rows one token ahead, and a conversion here would make the fetch wait for its own loads.
template <typename T, int DK, int GATE> struct QkRegs {
  static constexpr int EPL = Lanes<DK>::EPL;
  T k[EPL], q[EPL];
  float g[EPL];
  __device__ __forceinline__ void fetch(const T* qp, const T* kp, const float* gp, int lane) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int idx = min(lane + 64 * e, DK - 1);  // lanes past the row repeat its last element and drop it in commit
      k[e] = kp[idx];
      q[e] = qp[idx];
      if (GATE == LNX_GATE_VECTOR) g[e] = gp[idx];
    }
  }
  // Normalises / scales the rows and leaves k^, q~ (and exp(g) for a vector gate) in `sm` ([3][DK] floats).  Returns <q~, k^>.
  __device__ __forceinline__ float commit(float* sm, int lane, float scale, int l2norm) const {
    float kv[EPL], qv[EPL];
    float ksq = 0.f, qsq = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const bool ok = lane + 64 * e < DK;
      kv[e] = ok ? to_f32(k[e]) : 0.f;
      qv[e] = ok ? to_f32(q[e]) : 0.f;
      ksq += kv[e] * kv[e];
      qsq += qv[e] * qv[e];
    }
    float kmul = 1.f, qmul = scale;
    if (l2norm) {
      kmul = 1.f / (sqrtf(wave_sum(ksq)) + LNX_L2_EPS);
      qmul = scale / (sqrtf(wave_sum(qsq)) + LNX_L2_EPS);
    }
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int idx = lane + 64 * e;
      kv[e] *= kmul;
      qv[e] *= qmul;
      dot += kv[e] * qv[e];
      if (idx < DK) {
        sm[idx] = kv[e];
        sm[DK + idx] = qv[e];
        if (GATE == LNX_GATE_VECTOR) sm[2 * DK + idx] = expf(g[e]);
      }
    }
    return wave_sum(dot);
  }
};

// Loads one q/k row pair with a full wavefront, normalises/scales it and leaves
// k^, q~ (and exp(g) for a vector gate) in `sm` ([3][DK] floats).  Returns <q~, k^>.
template <typename T, int DK, int GATE>
__device__ __forceinline__ float stage_qk(const T* qp, const T* kp, const float* gp, float* sm,
                                          int lane, float scale, int l2norm) {
  QkRegs<T, DK, GATE> r;
  r.fetch(qp, kp, gp, lane);
  return r.commit(sm, lane, scale, l2norm);
}

// One token applied to the register slab S[RPL] (rows row0.., columns of this lane).
template <int DK, int GATE>
__device__ __forceinline__ floatx4 apply_token(floatx4 (&S)[Lanes<DK>::RPL], const float* sm, int row0,
                                               float alpha_s, float beta, floatx4 v4, float qk) {
  constexpr int RPL = Lanes<DK>::RPL;
  floatx4 a1 = {0.f, 0.f, 0.f, 0.f}, a2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const float kk = sm[row0 + i], qq = sm[DK + row0 + i];
    if (GATE == LNX_GATE_VECTOR) S[i] *= sm[2 * DK + row0 + i];
    else if (GATE == LNX_GATE_SCALAR) S[i] *= alpha_s;
    a1 += S[i] * kk;
    a2 += S[i] * qq;
  }
  a1 = rowgroup_sum(a1);
  a2 = rowgroup_sum(a2);
  const floatx4 d = (v4 - a1) * beta;
#pragma unroll
  for (int i = 0; i < RPL; ++i) S[i] += d * sm[row0 + i];
  return a2 + d * qk;
}

// grid (B*H, ceil(dv/128)), block 256: wave w owns columns [32*(4*blockIdx.y+w), +32).
template <typename T, int DK, int GATE>
__global__ __launch_bounds__(256) void decode_step_kernel(TokenParams p) {
  constexpr int RPL = Lanes<DK>::RPL;
  __shared__ float sm_all[4][3 * DK];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t bh = blockIdx.x;
  float* sm = sm_all[wave];
  const int col0 = (blockIdx.y * 4 + wave) * 32 + (lane & 7) * 4;
  const bool active = col0 < p.dv;
  const int row0 = (lane >> 3) * RPL;
  const int64_t sbase = (bh * DK + row0) * p.dv + (active ? col0 : 0);
  // The state loads go out first: they do not depend on the q / k staging below, whose loads, reductions and barrier
  // would otherwise sit in front of the only traffic that matters.
  floatx4 S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    // streamed once: non-temporal, so the 512 MiB state does not churn L2 / the memory-side cache
    S[i] = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(p.s_in + sbase + (int64_t)i * p.dv));
  }
  const floatx4 v4 = load4(reinterpret_cast<const T*>(p.v) + bh * p.dv + (active ? col0 : 0));
  const float beta = p.beta[bh];
  const float g_s = (GATE == LNX_GATE_SCALAR) ? p.g[bh] : 0.f;
  const float* gp = (GATE == LNX_GATE_VECTOR) ? p.g + bh * DK : nullptr;
  const float qk = stage_qk<T, DK, GATE>(reinterpret_cast<const T*>(p.q) + bh * DK,
                                         reinterpret_cast<const T*>(p.k) + bh * DK, gp, sm, lane, p.scale,
                                         p.l2norm);
  __syncthreads();
  if (!active) return;
  const float alpha_s = (GATE == LNX_GATE_SCALAR) ? expf(g_s) : 1.f;
  const floatx4 o4 = apply_token<DK, GATE>(S, sm, row0, alpha_s, beta, v4, qk);
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    __builtin_nontemporal_store(S[i], reinterpret_cast<floatx4*>(p.s_out + sbase + (int64_t)i * p.dv));
  }
  if ((lane >> 3) == 0) store_o4(p.o, bh * p.dv + col0, o4, p.o_dtype);
}

// grid (nstate*H, ceil(dv/32)), block 64: one wavefront scans a 32-column slab over time.
template <typename T, int DK, int GATE>
__global__ __launch_bounds__(64) void recurrent_fwd_kernel(TokenParams p) {
  constexpr int RPL = Lanes<DK>::RPL;
  __shared__ float sm[3 * DK];
  const int lane = threadIdx.x;
  const int64_t sh = blockIdx.x;  // state index: (batch or sequence) * H + head
  const int h = (int)(sh % p.H);
  const int sb = (int)(sh / p.H);
  int t0 = 0, t1 = p.T;
  int64_t bh = sh;  // row of the [B*H, T, .] token tensors
  if (p.cu_seqlens) {
    t0 = seq_first(p.cu_seqlens, sb, p.T);
    t1 = seq_end(p.cu_seqlens, sb, p.T);
    bh = h;
  }
  const int col0 = blockIdx.y * 32 + (lane & 7) * 4;
  const bool active = col0 < p.dv;
  const int ccol = active ? col0 : 0;
  const int row0 = (lane >> 3) * RPL;
  const int64_t sbase = (sh * DK + row0) * p.dv + ccol;
  floatx4 S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    if (p.s_in && active) S[i] = load4(p.s_in + sbase + (int64_t)i * p.dv);
    else S[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // position of token 0 of this row in units of one token's vector; token t is t * ts further on
  const int64_t ts = p.ts, tok0 = (ts == 1) ? bh * p.T : (bh / p.H) * p.T * p.H + bh % p.H;
  const T* qb = reinterpret_cast<const T*>(p.q) + tok0 * DK;
  const T* kb = reinterpret_cast<const T*>(p.k) + tok0 * DK;
  const T* vb = reinterpret_cast<const T*>(p.v) + tok0 * p.dv + ccol;
  const float* betab = p.beta + tok0;
  const float* gb = nullptr;
  if (GATE == LNX_GATE_SCALAR) gb = p.g + tok0;
  if (GATE == LNX_GATE_VECTOR) gb = p.g + tok0 * DK;
  // The rows of token t + 1 are fetched (raw, nothing converted) while token t is applied, and the barriers order LDS
  // only: with __syncthreads() or a conversion at the fetch every token would wait for a round trip to memory.
  struct Ahead {
    QkRegs<T, DK, GATE> qk;
    typename Vec4<T>::V v;
    float beta, g;
  };
  auto fetch = [&](Ahead& r, int t) {
    const int64_t tt = (int64_t)min(t, t1 - 1) * ts;  // past the end: the last token again, never used
    r.qk.fetch(qb + tt * DK, kb + tt * DK, (GATE == LNX_GATE_VECTOR) ? gb + tt * DK : nullptr, lane);
    r.v = *reinterpret_cast<const typename Vec4<T>::V*>(vb + tt * p.dv);
    r.beta = betab[tt];
    r.g = (GATE == LNX_GATE_SCALAR) ? gb[tt] : 0.f;
  };
  Ahead cur, nxt;
  if (t0 < t1) fetch(cur, t0);
  for (int t = t0; t < t1; ++t) {
    fetch(nxt, t + 1);
    lds_barrier();  // previous token's reads of sm are done
    const float qk = cur.qk.commit(sm, lane, p.scale, p.l2norm);
    lds_barrier();
    const float alpha_s = (GATE == LNX_GATE_SCALAR) ? expf(cur.g) : 1.f;
    const floatx4 v4 = {to_f32(cur.v[0]), to_f32(cur.v[1]), to_f32(cur.v[2]), to_f32(cur.v[3])};
    const floatx4 o4 = apply_token<DK, GATE>(S, sm, row0, alpha_s, cur.beta, v4, qk);
    if ((lane >> 3) == 0 && active) store_o4(p.o, (tok0 + (int64_t)t * ts) * p.dv + col0, o4, p.o_dtype);
    cur = nxt;
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) store4(p.s_out + sbase + (int64_t)i * p.dv, S[i]);
  }
}

template <typename T, int DK>
int launch_gate(bool decode, int gate, const TokenParams& p, dim3 grid, hipStream_t st) {
#define LNX_LAUNCH(G)                                                                          \
  if (decode) hipLaunchKernelGGL((decode_step_kernel<T, DK, G>), grid, dim3(256), 0, st, p);   \
  else hipLaunchKernelGGL((recurrent_fwd_kernel<T, DK, G>), grid, dim3(64), 0, st, p)
  switch (gate) {
    case LNX_GATE_NONE: LNX_LAUNCH(LNX_GATE_NONE); break;
    case LNX_GATE_SCALAR: LNX_LAUNCH(LNX_GATE_SCALAR); break;
    case LNX_GATE_VECTOR: LNX_LAUNCH(LNX_GATE_VECTOR); break;
    default: return lnx_set_error(LNX_ERR_SHAPE, "unknown gate kind %d", gate);
  }
#undef LNX_LAUNCH
  return LNX_OK;
}

template <typename T>
int launch_dk(bool decode, int dk, int gate, const TokenParams& p, dim3 grid, hipStream_t st) {
  switch (dk) {
    case 8: return launch_gate<T, 8>(decode, gate, p, grid, st);
    case 16: return launch_gate<T, 16>(decode, gate, p, grid, st);
    case 32: return launch_gate<T, 32>(decode, gate, p, grid, st);
    case 64: return launch_gate<T, 64>(decode, gate, p, grid, st);
    case 128: return launch_gate<T, 128>(decode, gate, p, grid, st);
    case 256: return launch_gate<T, 256>(decode, gate, p, grid, st);
    default:
      return lnx_set_error(LNX_ERR_SHAPE, "token kernels need dk in {8,16,32,64,128,256}, got %d", dk);
  }
}

int token_entry(bool decode, const lnx_scan_args* a, void* stream) {
  if (!a) return lnx_set_error(LNX_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->H <= 0 || a->dk <= 0 || a->dv <= 0 || (!decode && a->T < 0))
    return lnx_set_error(LNX_ERR_SHAPE, "bad dimensions B=%d H=%d T=%d dk=%d dv=%d", a->B, a->H, a->T, a->dk, a->dv);
  // tensors without elements (no batch rows, or no tokens in a scan) may come with null pointers
  const bool tokens = a->B > 0 && (decode || a->T > 0);
  if ((tokens && (!a->q || !a->k || !a->v || !a->beta || !a->o)) || (a->B > 0 && !a->final_state))
    return lnx_set_error(LNX_ERR_NULL, "q, k, v, beta, o and final_state are required");
  if (tokens && a->gate != LNX_GATE_NONE && !a->g) return lnx_set_error(LNX_ERR_NULL, "gate kind %d needs g", a->gate);
  if (decode && a->B > 0 && !a->initial_state) return lnx_set_error(LNX_ERR_NULL, "decode step needs the current state");
  if (a->dv % 4 != 0) return lnx_set_error(LNX_ERR_SHAPE, "dv must be a multiple of 4, got %d", a->dv);
  if (a->dtype != LNX_F32 && a->dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "dtype %d", a->dtype);
  if (a->o_dtype != LNX_F32 && a->o_dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "o_dtype %d", a->o_dtype);
  const bool packed = !decode && a->cu_seqlens != nullptr;
  if (packed && (a->B != 1 || a->nseq <= 0))
    return lnx_set_error(LNX_ERR_SHAPE, "packed batches need B == 1 and nseq > 0 (B=%d nseq=%d)", a->B, a->nseq);
  const int64_t nstate = packed ? a->nseq : a->B;
  if (nstate == 0) return LNX_OK;  // empty batch: nothing to launch (T == 0 still copies the state)
  TokenParams p;
  p.q = a->q; p.k = a->k; p.v = a->v; p.beta = a->beta; p.g = a->g;
  p.s_in = a->initial_state; p.s_out = a->final_state; p.o = a->o;
  p.cu_seqlens = packed ? a->cu_seqlens : nullptr;
  p.H = a->H; p.T = a->T; p.dv = a->dv; p.ts = (!decode && a->token_first) ? a->H : 1; p.scale = a->scale; p.l2norm = a->use_qk_l2norm; p.o_dtype = a->o_dtype;
  dim3 grid((unsigned)(nstate * a->H), (unsigned)((a->dv + (decode ? 127 : 31)) / (decode ? 128 : 32)));
  hipStream_t st = (hipStream_t)stream;
  lnx_profile_mark(decode ? "decode_step" : "recurrent_fwd", st);
  int rc = (a->dtype == LNX_BF16) ? launch_dk<bf16_t>(decode, a->dk, a->gate, p, grid, st)
                                  : launch_dk<float>(decode, a->dk, a->gate, p, grid, st);
  lnx_profile_mark(nullptr, st);
  if (rc != LNX_OK) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "token kernel launch: %s", hipGetErrorString(e));
  return LNX_OK;
}

}  // namespace

extern "C" int lnx_decode_step(const lnx_scan_args* a, void* hip_stream) { return token_entry(true, a, hip_stream); }
extern "C" int lnx_recurrent_fwd(const lnx_scan_args* a, void* hip_stream) { return token_entry(false, a, hip_stream); }
