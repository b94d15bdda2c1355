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

__device__ __forceinline__ floatx4 rowgroup_sum(floatx4 x) {  // over the eight row groups (lanes 8 apart), in every lane
#pragma unroll
  for (int c = 0; c < 4; ++c)
    x[c] += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x[c]), 0x128, 0xF, 0xF, true));  // row_ror:8 = lane ^ 8
#pragma unroll
  for (int c = 0; c < 4; ++c) x[c] = xor32_sum(xor16_sum(x[c]));
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

// The five dk-vectors of a token in the registers of one wavefront, so that a token's loads are issued one token ahead
// of their use and only the LDS write sits between the two barriers of a token.
// Four consecutive elements as loaded (converted where they are used, not where they are fetched)
template <typename T> struct Raw4;
template <> struct Raw4<float> {
  floatx4 x;
  __device__ __forceinline__ void load(const float* p) { x = *reinterpret_cast<const floatx4*>(p); }
  __device__ __forceinline__ floatx4 f32() const { return x; }
};
template <> struct Raw4<bf16_t> {
  bf16x4 x;
  __device__ __forceinline__ void load(const bf16_t* p) { x = *reinterpret_cast<const bf16x4*>(p); }
  __device__ __forceinline__ floatx4 f32() const { return floatx4{(float)x[0], (float)x[1], (float)x[2], (float)x[3]}; }
};

template <typename T, int DK> struct TokenRegs {
  static constexpr int E = (DK + 63) / 64;
  T q[E], k[E], a[E], b[E];  // as loaded: converting here would make the fetch wait for its own loads
  float g[E];
  __device__ __forceinline__ void fetch(const T* qp, const T* kp, const T* ap, const T* bp, const float* gp, int lane) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int idx = min(lane + 64 * e, DK - 1);
      q[e] = qp[idx];
      k[e] = kp[idx];
      a[e] = ap[idx];
      b[e] = bp[idx];
      g[e] = gp[idx];
    }
  }
  // sm: q~, k, a, b, w.  DOTS: returns (<b, q~>, <k, q~>), which the outputs of the forward scan need.
  template <bool DOTS = true>
  __device__ __forceinline__ floatx2 commit(float* sm, int lane, float scale) const {
    float bq = 0.f, kq = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int idx = lane + 64 * e;
      if (idx < DK) {
        const float qv = to_f32(q[e]) * scale, kv = to_f32(k[e]), bv = to_f32(b[e]);
        sm[idx] = qv;
        sm[DK + idx] = kv;
        sm[2 * DK + idx] = to_f32(a[e]);
        sm[3 * DK + idx] = bv;
        sm[4 * DK + idx] = expf(g[e]);
        bq += bv * qv;
        kq += kv * qv;
      }
    }
    if (!DOTS) return floatx2{0.f, 0.f};
    return floatx2{wave_sum(bq), wave_sum(kq)};
  }
};

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
  // A token's compute time is a fraction of a memory round trip, so its vectors are requested four tokens before their
  // use: four register sets in rotation, each refilled as soon as its token has been written to LDS.  The barriers order
  // LDS only (see TokenRegs).
  TokenRegs<T, DK> s0, s1, s2, s3;
  Raw4<T> w0, w1, w2, w3;
  auto fetch = [&](TokenRegs<T, DK>& s, Raw4<T>& w, int t) {
    const int64_t tc = min(t, p.T - 1);
    s.fetch(q + tc * DK, k + tc * DK, a + tc * DK, b + tc * DK, gk + tc * DK, lane);
    w.load(v + tc * p.dv);
  };
  auto step = [&](TokenRegs<T, DK>& s, Raw4<T>& w, int t) {
    if (t >= p.T) return;
    lds_barrier();  // the previous token's reads of sm are done
    const floatx2 dots = s.commit(sm, lane, p.scale);
    const floatx4 v4 = w.f32();
    lds_barrier();
    fetch(s, w, t + 4);
    const floatx4 o4 = apply_token<DK>(S, sm, row0, v4, dots);
    if ((lane >> 3) == 0 && active) store_o4(p.o, (tok0 + t) * p.dv + col0, o4, p.o_dtype);
  };
  if (p.T > 0) {
    fetch(s0, w0, 0);
    fetch(s1, w1, 1);
    fetch(s2, w2, 2);
    fetch(s3, w3, 3);
  }
  for (int t = 0; t < p.T; t += 4) {
    step(s0, w0, t);
    step(s1, w1, t + 1);
    step(s2, w2, t + 2);
    step(s3, w3, t + 3);
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) store4(p.s_out + sbase + (int64_t)i * p.dv, S[i]);
  }
}

// ---------------------------------------------------------------------------------------
// Backward pass of the scan: the gradients of <o, d_o> + <final state, d_final_state> (the reference differentiates its
// lax.scan with jax.grad, rwkv7.py:148-213).  Per token, with h' the state before it, u = h'^T a and D the gradient of
// the state after it (the later tokens' share plus q~ d_o^T):
//   dq = scale h d_o;  dv = D^T k;  dk = D v;  db = D u;  du = D^T b;  da = h' du;  dgk = w (.) rowsum(D (.) h');
//   gradient of h' = w (.) D + a du^T.
// Every token needs the state it started from.  The recurrence cannot be run backwards (its inverse divides by the
// decays), so one workgroup per (batch, head) first sweeps forward and keeps the state at the start of every SEG-token
// segment (checkpoints), then takes the segments last to first: a forward sweep through the segment that writes each
// token's starting state to a tape, and the reverse sweep reading it back.  Wave w owns value columns [32 w, 32 w + 32)
// with the register layout of the forward kernels; checkpoints and tape are read by the lane that wrote them.  The five
// dk-vector gradients are sums over all value columns: per token the waves leave their shares in LDS and the
// workgroup adds them up -- no atomics, the result does not depend on the order of anything.
// ---------------------------------------------------------------------------------------
constexpr int DPLR_SEG = 64;

struct DplrBwdParams {
  const void *q, *k, *v, *a, *b;
  const float* gk;
  const float* s_in;
  const void* d_o;
  const float* d_sT;
  float *dq, *dk, *da, *db, *dgk, *dv_out, *ds0;
  float *ckpt, *tape;  // [B*H][nseg][dk][dv], [B*H][DPLR_SEG][dk][dv]
  int H, T, dv, nseg;
  float scale;
  int o_dtype;
};

__device__ __forceinline__ float dot4(floatx4 x, floatx4 y) { return x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3]; }
__device__ __forceinline__ float colgroup_sum(float x) {  // over the eight lanes that hold the columns of one row group
  x = quad_sum(x);                                                                         // two DPP quad permutes
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xF, 0xF, true));  // row_half_mirror: lane i <-> 7 - i
  return x;
}

template <typename T, int DK>
__global__ __launch_bounds__(512) void dplr_bwd_kernel(DplrBwdParams p) {
  constexpr int RPL = DK / 8;
  __shared__ float sm[5 * DK];          // q~, k, a, b, w of the current token
  __shared__ float red[8][5][DK];       // per wave: its share of dq / scale, dk, db, dgk / w, da
  constexpr int NB = 8;                 // tokens whose five gradient rows wait in LDS for one coalesced write
  __shared__ __align__(16) float outb[5][NB][DK];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nthr = blockDim.x;
  const int64_t bh = blockIdx.x;
  const int col0 = wave * 32 + (lane & 7) * 4;
  const bool active = col0 < p.dv;
  const int ccol = active ? col0 : 0;
  const int row0 = (lane >> 3) * RPL;
  const int64_t sbase = (bh * DK + row0) * p.dv + ccol;            // this lane's piece of a [dk][dv] state of this (b, h)
  const int64_t slab = (int64_t)row0 * p.dv + ccol;                // the same inside one state
  const int64_t ssz = (int64_t)DK * p.dv;
  float* ckpt = p.ckpt + bh * p.nseg * ssz;
  float* tape = p.tape + bh * DPLR_SEG * ssz;
  const int64_t tok0 = bh * p.T;
  const T *q = static_cast<const T*>(p.q) + tok0 * DK, *k = static_cast<const T*>(p.k) + tok0 * DK,
          *a = static_cast<const T*>(p.a) + tok0 * DK, *b = static_cast<const T*>(p.b) + tok0 * DK;
  const T* v = static_cast<const T*>(p.v) + tok0 * p.dv + ccol;
  const float* gk = p.gk + tok0 * DK;

  // Token t's vectors are fetched (by every wave, wave 0 writes them to LDS) while token t -/+ 1 is being worked on (`ahead`: the token after this one in
  // sweep order, or -1); between a token's two barriers there is only the LDS write.  The barriers order LDS only:
  // __syncthreads() would also wait for the loads just issued for the next token, i.e. for a memory round trip per token.
  TokenRegs<T, DK> tr;
  auto fetch_tok = [&](int t) {  // every wave, no branch: behind one the compiler cannot count the loads in flight
    const int64_t r = (int64_t)min(max(t, 0), p.T - 1) * DK;
    tr.fetch(q + r, k + r, a + r, b + r, gk + r, lane);
  };
  const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
  auto load_state = [&](const float* ptr) -> floatx4 {  // inactive lanes read a valid address and drop what they read
    const floatx4 x = load4(ptr);
    return active ? x : zero4;
  };
  auto stage = [&](int ahead) {
    lds_barrier();  // the previous token's reads of sm (and of the sums over the waves) are done
    if (wave == 0) tr.template commit<false>(sm, lane, p.scale);
    fetch_tok(ahead);
    lds_barrier();
  };
  floatx4 S[RPL];

  // ---- checkpoints ----
#pragma unroll
  for (int i = 0; i < RPL; ++i) S[i] = p.s_in ? load_state(p.s_in + sbase + (int64_t)i * p.dv) : zero4;
  {
    const int tend = (p.nseg - 1) * DPLR_SEG;  // the last segment is swept below
    fetch_tok(0);
    Raw4<T> v4, vn;
    v4.load(v);
    for (int t = 0; t < tend; ++t) {
      if (t % DPLR_SEG == 0 && active) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) store4(ckpt + (t / DPLR_SEG) * ssz + slab + (int64_t)i * p.dv, S[i]);
      }
      stage(t + 1 < tend ? t + 1 : -1);
      vn.load(v + (int64_t)min(t + 1, p.T - 1) * p.dv);
      apply_token<DK>(S, sm, row0, v4.f32(), floatx2{0.f, 0.f});
      v4 = vn;
    }
    if (active) {
#pragma unroll
      for (int i = 0; i < RPL; ++i) store4(ckpt + (p.nseg - 1) * ssz + slab + (int64_t)i * p.dv, S[i]);
    }
  }

  floatx4 D[RPL];  // gradient of the state after the current token
#pragma unroll
  for (int i = 0; i < RPL; ++i) D[i] = p.d_sT ? load_state(p.d_sT + sbase + (int64_t)i * p.dv) : zero4;

  // d_o may be fp32 or bf16 whatever the inputs are: both raw forms travel, the one that was loaded is converted at use
  struct RawDo {
    floatx4 f;
    bf16x4 h;
  };
  auto load_do = [&](RawDo& r, int t) {
    if (p.o_dtype == LNX_BF16) r.h = *reinterpret_cast<const bf16x4*>(static_cast<const bf16_t*>(p.d_o) + (tok0 + t) * p.dv + ccol);
    else r.f = *reinterpret_cast<const floatx4*>(static_cast<const float*>(p.d_o) + (tok0 + t) * p.dv + ccol);
  };
  auto do_f32 = [&](const RawDo& r) -> floatx4 {
    if (!active) return floatx4{0.f, 0.f, 0.f, 0.f};
    if (p.o_dtype == LNX_BF16) return floatx4{(float)r.h[0], (float)r.h[1], (float)r.h[2], (float)r.h[3]};
    return r.f;
  };

  for (int seg = p.nseg - 1; seg >= 0; --seg) {
    const int t0 = seg * DPLR_SEG, len = min(DPLR_SEG, p.T - t0);
    // ---- forward through the segment, every token's starting state onto the tape ----
#pragma unroll
    for (int i = 0; i < RPL; ++i) S[i] = load_state(ckpt + seg * ssz + slab + (int64_t)i * p.dv);
    {
      fetch_tok(t0);
      Raw4<T> v4, vn;
      v4.load(v + (int64_t)t0 * p.dv);
      for (int tl = 0; tl < len; ++tl) {
        const bool last = tl + 1 == len;
        if (!last) {
          stage(tl + 2 < len ? t0 + tl + 1 : -1);
          vn.load(v + (int64_t)(t0 + tl + 1) * p.dv);
        }
        // after this token's loads: the memory counter runs in order, so a store issued before a load is waited for
        // with that load, one token later
        if (active) {
#pragma unroll
          for (int i = 0; i < RPL; ++i) store4(tape + tl * ssz + slab + (int64_t)i * p.dv, S[i]);
        }
        if (last) break;
        apply_token<DK>(S, sm, row0, v4.f32(), floatx2{0.f, 0.f});
        v4 = vn;
      }
    }
    // ---- reverse: the next token's tape entry, v and d_o are in flight while this one is worked on ----
    fetch_tok(t0 + len - 1);
    floatx4 hp[RPL];
    Raw4<T> vr, vnr;
    RawDo dr{}, dnr{};
    vr.load(v + (int64_t)(t0 + len - 1) * p.dv);
    load_do(dr, t0 + len - 1);
#pragma unroll
    for (int i = 0; i < RPL; ++i) hp[i] = load_state(tape + (len - 1) * ssz + slab + (int64_t)i * p.dv);
    // Two barriers per token.  Between them: the sums over the waves of the token before (its shares are complete at the
    // first barrier) go to the output buffer while wave 0 writes this token's vectors.
    int pend = -1;  // position in the segment of the token whose shares wait in `red`
    auto reduce_pending = [&]() {
      if (pend < 0) return;
      const int nw = nthr >> 6, slot = (len - 1 - pend) % NB;
      for (int idx = tid; idx < 5 * DK; idx += nthr) {
        const int x = idx / DK, kk = idx - x * DK;
        float sum = 0.f;
        for (int w_ = 0; w_ < nw; ++w_) sum += red[w_][x][kk];
        outb[x][NB - 1 - slot][kk] = x == 0 ? sum * p.scale : sum;  // rows in increasing token order
      }
    };
    auto flush = [&](int tfirst, int rows) {  // tokens tfirst .. tfirst + rows - 1 lie in buffer rows NB - rows .. NB - 1
      for (int idx = tid; idx < 5 * rows * (DK / 4); idx += nthr) {
        const int x = idx / (rows * (DK / 4)), rem = idx - x * rows * (DK / 4), j = rem / (DK / 4), c4 = (rem - j * (DK / 4)) * 4;
        float* dst = x == 0 ? p.dq : x == 1 ? p.dk : x == 2 ? p.db : x == 3 ? p.dgk : p.da;
        store4(dst + (tok0 + tfirst + j) * DK + c4, load4(&outb[x][NB - rows + j][c4]));
      }
    };
    for (int tl = len - 1; tl >= 0; --tl) {
      const int t = t0 + tl;
      lds_barrier();
      reduce_pending();
      if (wave == 0) tr.template commit<false>(sm, lane, p.scale);
      fetch_tok(tl > 0 ? t - 1 : -1);
      lds_barrier();
      if (pend >= 0 && (len - 1 - pend) % NB == NB - 1) flush(t0 + pend, NB);
      const int tn = max(tl - 1, 0);
      constexpr int NPRE = DK <= 64 ? RPL : 1;  // at dk = 128 a second set of state registers would spill: the tape is read in place
      floatx4 hn[NPRE];
      if (DK <= 64) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) hn[i] = load_state(tape + tn * ssz + slab + (int64_t)i * p.dv);
      }
      vnr.load(v + (int64_t)(t0 + tn) * p.dv);
      load_do(dnr, t0 + tn);
      const floatx4 v4 = vr.f32(), do4 = do_f32(dr);
      floatx4 u = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < RPL; ++i) u += hp[i] * sm[2 * DK + row0 + i];
      u = rowgroup_sum(u);
      floatx4 dv4 = {0.f, 0.f, 0.f, 0.f}, du4 = {0.f, 0.f, 0.f, 0.f};
      float pq[RPL], pk[RPL], pb[RPL], pw[RPL];
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const float qv = sm[row0 + i], kv = sm[DK + row0 + i], bv = sm[3 * DK + row0 + i], wv = sm[4 * DK + row0 + i];
        const floatx4 h = hp[i] * wv + u * bv + v4 * kv;  // the state after the token
        pq[i] = dot4(h, do4);
        D[i] += do4 * qv;
        pk[i] = dot4(D[i], v4);
        pb[i] = dot4(D[i], u);
        pw[i] = dot4(D[i], hp[i]);
        dv4 += D[i] * kv;
        du4 += D[i] * bv;
      }
      dv4 = rowgroup_sum(dv4);
      const floatx4 du = rowgroup_sum(du4);
      if ((lane >> 3) == 0 && active) store4(p.dv_out + (tok0 + t) * p.dv + col0, dv4);
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const float pa = colgroup_sum(dot4(hp[i], du));
        const float sq = colgroup_sum(pq[i]), sk = colgroup_sum(pk[i]), sb = colgroup_sum(pb[i]), sw = colgroup_sum(pw[i]);
        if ((lane & 7) == 0) {
          red[wave][0][row0 + i] = sq;
          red[wave][1][row0 + i] = sk;
          red[wave][2][row0 + i] = sb;
          red[wave][3][row0 + i] = sw * sm[4 * DK + row0 + i];
          red[wave][4][row0 + i] = pa;
        }
        D[i] = D[i] * sm[4 * DK + row0 + i] + du * sm[2 * DK + row0 + i];  // gradient of the state before the token
      }
      pend = tl;
#pragma unroll
      for (int i = 0; i < RPL; ++i) hp[i] = DK <= 64 ? hn[DK <= 64 ? i : 0] : (load_state(tape + tn * ssz + slab + (int64_t)i * p.dv));
      vr = vnr;
      dr = dnr;
    }
    lds_barrier();
    reduce_pending();
    lds_barrier();
    flush(t0, (len - 1) % NB + 1);
  }
  if (p.ds0 && active) {
#pragma unroll
    for (int i = 0; i < RPL; ++i) store4(p.ds0 + sbase + (int64_t)i * p.dv, D[i]);
  }
}

__global__ void dplr_pass_state_kernel(const float* src, float* dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src ? src[i] : 0.f;
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

extern "C" uint64_t lnx_dplr_recurrent_bwd_workspace_bytes(int32_t B, int32_t H, int32_t T, int32_t dk, int32_t dv) {
  if (B <= 0 || H <= 0 || T <= 0 || dk <= 0 || dv <= 0) return 0;
  const uint64_t nseg = (uint64_t)(T + DPLR_SEG - 1) / DPLR_SEG;
  return (uint64_t)B * H * (nseg + DPLR_SEG) * dk * dv * sizeof(float);
}

extern "C" int lnx_dplr_recurrent_bwd(const lnx_dplr_bwd_args* g, void* hip_stream) {
  if (!g) return lnx_set_error(LNX_ERR_NULL, "args is NULL");
  const lnx_dplr_args* a = &g->fwd;
  if (a->B < 0 || a->H <= 0 || a->T < 0 || a->dk <= 0 || a->dv <= 0)
    return lnx_set_error(LNX_ERR_SHAPE, "bad dimensions B=%d H=%d T=%d dk=%d dv=%d", a->B, a->H, a->T, a->dk, a->dv);
  if (a->dv % 4 != 0 || a->dv > 256) return lnx_set_error(LNX_ERR_SHAPE, "the backward pass needs dv a multiple of 4, at most 256; got %d", a->dv);
  if (a->dtype != LNX_F32 && a->dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "dtype %d", a->dtype);
  if (a->o_dtype != LNX_F32 && a->o_dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "o_dtype %d", a->o_dtype);
  if (a->B == 0) return LNX_OK;
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int64_t state = (int64_t)a->B * a->H * a->dk * a->dv;
  if (a->T == 0) {  // no token: the state passes through (a kernel, not a memset: callers may be capturing a graph)
    if (g->d_initial_state) {
      hipLaunchKernelGGL(dplr_pass_state_kernel, dim3((unsigned)((state + 255) / 256)), dim3(256), 0, st, g->d_final_state, g->d_initial_state, state);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "state gradient copy: %s", hipGetErrorString(e));
    }
    return LNX_OK;
  }
  if (!a->q || !a->k || !a->v || !a->a || !a->b || !a->gk || !g->d_o || !g->dq || !g->dk || !g->dv || !g->da || !g->db || !g->dgk)
    return lnx_set_error(LNX_ERR_NULL, "q, k, v, a, b, gk, d_o and the six token gradients are required");
  const uint64_t need = lnx_dplr_recurrent_bwd_workspace_bytes(a->B, a->H, a->T, a->dk, a->dv);
  if (!g->workspace || g->workspace_bytes < need)
    return lnx_set_error(LNX_ERR_WORKSPACE, "workspace of %llu bytes needed, %llu given", (unsigned long long)need, (unsigned long long)g->workspace_bytes);
  const int nseg = (a->T + DPLR_SEG - 1) / DPLR_SEG;
  DplrBwdParams p{a->q, a->k, a->v, a->a, a->b, a->gk, a->initial_state, g->d_o, g->d_final_state,
                  g->dq, g->dk, g->da, g->db, g->dgk, g->dv, g->d_initial_state,
                  static_cast<float*>(g->workspace), static_cast<float*>(g->workspace) + (int64_t)a->B * a->H * nseg * a->dk * a->dv,
                  a->H, a->T, a->dv, nseg, a->scale, a->o_dtype};
  const dim3 grid((unsigned)((int64_t)a->B * a->H)), block(64 * ((a->dv + 31) / 32));
  lnx_profile_mark("dplr_bwd", st);
#define LNX_DPLR_BWD(D)                                                                                        \
  case D:                                                                                                      \
    if (a->dtype == LNX_BF16) hipLaunchKernelGGL((dplr_bwd_kernel<bf16_t, D>), grid, block, 0, st, p);         \
    else hipLaunchKernelGGL((dplr_bwd_kernel<float, D>), grid, block, 0, st, p);                               \
    break
  switch (a->dk) {
    LNX_DPLR_BWD(8); LNX_DPLR_BWD(16); LNX_DPLR_BWD(32); LNX_DPLR_BWD(64); LNX_DPLR_BWD(128);
    default: lnx_profile_mark(nullptr, st); return lnx_set_error(LNX_ERR_SHAPE, "dplr kernels need dk in {8,16,32,64,128}, got %d", a->dk);
  }
#undef LNX_DPLR_BWD
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "dplr backward launch: %s", hipGetErrorString(e));
  return LNX_OK;
}

extern "C" int lnx_dplr_step(const lnx_dplr_args* a, void* hip_stream) { return entry(true, a, hip_stream); }
extern "C" int lnx_dplr_recurrent_fwd(const lnx_dplr_args* a, void* hip_stream) { return entry(false, a, hip_stream); }
