// Short causal depthwise convolution (kernel width <= 4) with an optional fused SiLU, forward and
// backward, for [B, T, D] activations with a [B, K-1, D] carry-in cache -- the step that precedes
// the delta-rule ops in the reference's blocks (linearnexus/core/conv.py:13-68 followed by
// jax.nn.silu, gated_deltanet.py:765-779).
//
//   xin = concat(cache, x) along T;   z[t] = bias + sum_j w[j] * xin[t + j]  (j = 0..K-1: w[K-1] meets the
//   current token);   y = z or silu(z);   new_cache = last K-1 rows of xin.
//
// Streaming kernels: one thread owns 16 bytes of channels and a run of consecutive tokens, keeps the
// K-1 previous tokens in registers and touches every element of x (and dy) once apart from a K-1 halo.
#include "lnx_common.h"

namespace {

constexpr int KMAX = 4;
constexpr int SEG_FWD = 32;   // tokens per thread, forward
constexpr int SEG_BWD = 64;   // tokens per thread, backward
constexpr int BWD_RUNS = 4;   // token runs per workgroup, backward
constexpr int BATCH = 8;      // tokens whose loads are in flight together, per thread
// A workgroup's 256 threads cover `gx` adjacent channel groups (64, 128 or 256: as many as the row has, so that
// the workgroup reads long contiguous pieces of each token row) times 256/gx token runs.

struct ConvParams {
  const void* x; const float* w; const float* bias; const void* cache;
  void* y; void* new_cache;
  const void* dy; void* dx; float* dw; float* dbias;
  int B, T, D, K, act, gx;
  const int32_t* cu; int nseq;  // packed batch (B = 1): the taps stop at the start of each token's sequence
  void* dcache;                 // conv1d_dcache_kernel only
};

// Packed batches: [lo, hi) is the sequence that holds token t (bisection over the table; entries clamped to [0, T]).
// A token the table does not cover is treated as part of the sequence before it.
__device__ __forceinline__ void seq_of(const ConvParams& p, int t, int& s, int& lo, int& hi) {
  int a = 0, b = p.nseq - 1;
  while (a < b) {
    const int m = (a + b + 1) >> 1;
    if (seq_first(p.cu, m, p.T) <= t) a = m; else b = m - 1;
  }
  s = a;
  lo = seq_first(p.cu, s, p.T);
  hi = seq_end(p.cu, s, p.T);
}
// Moves (s, lo, hi) on to the sequence that holds token t >= hi (empty sequences are stepped over).
__device__ __forceinline__ void seq_advance(const ConvParams& p, int t, int& s, int& lo, int& hi) {
  while (t >= hi && s + 1 < p.nseq) {
    ++s;
    lo = seq_first(p.cu, s, p.T);
    hi = seq_end(p.cu, s, p.T);
  }
  if (t >= hi) hi = p.T + KMAX;  // past the table: no further boundary
}

// N consecutive channels of one token as one vector access (16 bytes forward, 8 or 16 bytes backward: the
// backward keeps five sums per channel in registers, and the narrower group doubles its occupancy).
template <typename T, int N> struct Vec { typedef T raw __attribute__((ext_vector_type(N))); };

template <typename T, int N> __device__ __forceinline__ void load_vec(const T* p, float (&o)[N]) {
  typename Vec<T, N>::raw r = *reinterpret_cast<const typename Vec<T, N>::raw*>(p);
#pragma unroll
  for (int i = 0; i < N; ++i) o[i] = (float)r[i];
}
template <typename T, int N> __device__ __forceinline__ void store_vec(T* p, const float (&v)[N]) {
  typename Vec<T, N>::raw r;
#pragma unroll
  for (int i = 0; i < N; ++i) r[i] = from_f32<T>(v[i]);
  *reinterpret_cast<typename Vec<T, N>::raw*>(p) = r;
}

__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + __expf(-z)); }

// Row `s` of xin for one channel group: s >= 0 is x[s]; -(K-1) <= s < 0 is the cache (zeros without one).
template <typename T, int N>
__device__ __forceinline__ void load_xin(const ConvParams& p, int b, int s, int c, float (&o)[N], int lo = 0) {
  if (s >= lo && s >= 0 && s < p.T) {
    load_vec<T, N>(static_cast<const T*>(p.x) + ((size_t)b * p.T + s) * p.D + c, o);
  } else if (s < 0 && s >= -(p.K - 1) && p.cache) {
    load_vec<T, N>(static_cast<const T*>(p.cache) + ((size_t)b * (p.K - 1) + (p.K - 1 + s)) * p.D + c, o);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) o[i] = 0.f;
  }
}

// Weights of one channel group, right-aligned in a width-4 window (taps the kernel does not have are zero).
template <int N>
__device__ __forceinline__ void load_taps(const ConvParams& p, int c, float (&w)[KMAX][N], float (&bias)[N]) {
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    const int jr = j - (KMAX - p.K);
#pragma unroll
    for (int i = 0; i < N; ++i) w[j][i] = jr >= 0 ? (p.K == 1 ? 1.f : p.w[(size_t)jr * p.D + c + i]) : 0.f;  // conv.py:39-44
  }
#pragma unroll
  for (int i = 0; i < N; ++i) bias[i] = p.bias ? p.bias[c + i] : 0.f;
}

template <typename T, int N, bool PACKED>
__global__ __launch_bounds__(256) void conv1d_fwd_kernel(ConvParams p) {
  const int c = (blockIdx.x * p.gx + (threadIdx.x & (p.gx - 1))) * N;
  const int seg = blockIdx.y * (256 / p.gx) + threadIdx.x / p.gx;
  const int b = blockIdx.z;
  const int t0 = seg * SEG_FWD;
  if (c >= p.D || t0 >= p.T) return;
  const int t1 = min(t0 + SEG_FWD, p.T);
  float w[KMAX][N], bias[N], win[KMAX][N];
  load_taps<N>(p, c, w, bias);
  int sq = 0, lo = 0, hi = p.T + KMAX;
  if (PACKED) seq_of(p, t0, sq, lo, hi);
#pragma unroll
  for (int j = 0; j < KMAX - 1; ++j) load_xin<T, N>(p, b, t0 - (KMAX - 1) + j, c, win[j], lo);
  const T* xp = static_cast<const T*>(p.x) + ((size_t)b * p.T + t0) * p.D + c;
  T* yp = static_cast<T*>(p.y) + ((size_t)b * p.T + t0) * p.D + c;
  int tcur = t0;
  auto token = [&]() {
    if (PACKED) {
      if (tcur >= hi) {  // first token of the next sequence: nothing carries over
        seq_advance(p, tcur, sq, lo, hi);
#pragma unroll
        for (int j = 0; j < KMAX - 1; ++j)
#pragma unroll
          for (int i = 0; i < N; ++i) win[j][i] = 0.f;
      }
      ++tcur;
    }
    float z[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float a = bias[i];
#pragma unroll
      for (int j = 0; j < KMAX; ++j) a = fmaf(w[j][i], win[j][i], a);
      z[i] = p.act ? a * sigmoidf(a) : a;
    }
    store_vec<T, N>(yp, z);
    yp += p.D;
#pragma unroll
    for (int j = 0; j < KMAX - 1; ++j)
#pragma unroll
      for (int i = 0; i < N; ++i) win[j][i] = win[j + 1][i];
  };
  typedef typename Vec<T, N>::raw raw_t;
  int t = t0;
  for (; t + BATCH <= t1; t += BATCH) {  // the loads of BATCH tokens go out together
    raw_t xr[BATCH];
#pragma unroll
    for (int e = 0; e < BATCH; ++e) xr[e] = *reinterpret_cast<const raw_t*>(xp + (size_t)e * p.D);
    xp += (size_t)BATCH * p.D;
#pragma unroll
    for (int e = 0; e < BATCH; ++e) {
#pragma unroll
      for (int i = 0; i < N; ++i) win[KMAX - 1][i] = (float)xr[e][i];
      token();
    }
  }
  for (; t < t1; ++t, xp += p.D) {
    load_vec<T, N>(xp, win[KMAX - 1]);
    token();
  }
  if (p.new_cache && t1 == p.T) {  // this thread saw the end of the (last) sequence: the window holds its last 3 rows
    const int keep = p.K - 1;
    T* cp = static_cast<T*>(p.new_cache) + (size_t)b * keep * p.D + c;
    if (PACKED && seq_end(p.cu, p.nseq - 1, p.T) <= seq_first(p.cu, p.nseq - 1, p.T)) {
      // the last sequence has no tokens: the window still holds the tail of the one before it, the carry is zero
#pragma unroll
      for (int j = 0; j < KMAX; ++j)
#pragma unroll
        for (int i = 0; i < N; ++i) win[j][i] = 0.f;
    }
    for (int i = 0; i < keep; ++i) store_vec<T, N>(cp + (size_t)i * p.D, win[KMAX - 1 - keep + i]);
  }
}

// Backward of one run [t0, t1): sweeps u = t0 .. t1+2, recomputes z[u] from the window of x, forms
// dz[u] = dy[u] * act'(z[u]) and emits dx[u-3] = sum_j w[j] dz[u-j] once its four terms are known.
// dw, dbias: per-thread sums over the run's own tokens, reduced over the workgroup's four runs in LDS and
// added to the fp32 outputs with one hardware fp32 atomic (not a compare-and-swap loop) per (tap, channel) and workgroup.  The workgroup is 64 channel
// groups x 4 runs here whatever the row length.
template <typename T, int N, bool PACKED>
__global__ __launch_bounds__(256) void conv1d_bwd_kernel(ConvParams p) {
  __shared__ float red[BWD_RUNS - 1][KMAX + 1][64 * N];
  const int lane = threadIdx.x & 63, run = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) * N;
  const int seg = blockIdx.y * BWD_RUNS + run;
  const int b = blockIdx.z;
  const int t0 = seg * SEG_BWD;
  const bool live = c < p.D && t0 < p.T;
  float gw[KMAX][N], gb[N];
#pragma unroll
  for (int i = 0; i < N; ++i) {
    gb[i] = 0.f;
#pragma unroll
    for (int j = 0; j < KMAX; ++j) gw[j][i] = 0.f;
  }
  if (live) {
    const int t1 = min(t0 + SEG_BWD, p.T);
    float w[KMAX][N], bias[N], win[KMAX][N], dz[KMAX][N];
    load_taps<N>(p, c, w, bias);
    int sq = 0, lo = 0, hi = p.T + KMAX;
    int sst[KMAX];  // packed: first token of the sequence each dz slot's token belongs to
    if (PACKED) seq_of(p, t0, sq, lo, hi);
#pragma unroll
    for (int j = 0; j < KMAX - 1; ++j) {
      load_xin<T, N>(p, b, t0 - (KMAX - 1) + j, c, win[j], lo);
      sst[j] = lo;
#pragma unroll
      for (int i = 0; i < N; ++i) dz[j][i] = 0.f;
    }
    const T* xp = static_cast<const T*>(p.x) + ((size_t)b * p.T + t0) * p.D + c;
    const T* gp = static_cast<const T*>(p.dy) + ((size_t)b * p.T + t0) * p.D + c;
    T* dp = static_cast<T*>(p.dx) + ((size_t)b * p.T + t0) * p.D + c;
    // one token: win[3] and g hold x[u] and dy[u] (zeros past the end of the sequence)
    auto token = [&](int u, float (&g)[N]) {
      const bool own = u < t1;
      if (PACKED) {
        if (u >= hi) {  // first token of the next sequence: its window starts empty
          seq_advance(p, u, sq, lo, hi);
#pragma unroll
          for (int j = 0; j < KMAX - 1; ++j)
#pragma unroll
            for (int i = 0; i < N; ++i) win[j][i] = 0.f;
        }
        sst[KMAX - 1] = lo;
      }
#pragma unroll
      for (int i = 0; i < N; ++i) {
        float d = g[i];
        if (p.act) {
          float a = bias[i];
#pragma unroll
          for (int j = 0; j < KMAX; ++j) a = fmaf(w[j][i], win[j][i], a);
          const float s = sigmoidf(a);
          d *= s * (1.f + a * (1.f - s));
        }
        dz[KMAX - 1][i] = d;
        if (own) {
          gb[i] += d;
#pragma unroll
          for (int j = 0; j < KMAX; ++j) gw[j][i] = fmaf(d, win[j][i], gw[j][i]);
        }
      }
      if (u - (KMAX - 1) >= t0) {
        float r[N];
#pragma unroll
        for (int i = 0; i < N; ++i) {
          float a = 0.f;
#pragma unroll
          for (int j = 0; j < KMAX; ++j)  // packed: only tokens of the same sequence reach back to token u - 3
            a = fmaf(w[j][i], (PACKED && sst[KMAX - 1 - j] > u - (KMAX - 1)) ? 0.f : dz[KMAX - 1 - j][i], a);
          r[i] = a;
        }
        store_vec<T, N>(dp, r);
        dp += p.D;
      }
#pragma unroll
      for (int j = 0; j < KMAX - 1; ++j) {
        if (PACKED) sst[j] = sst[j + 1];
#pragma unroll
        for (int i = 0; i < N; ++i) win[j][i] = win[j + 1][i], dz[j][i] = dz[j + 1][i];
      }
    };
    // Tokens with data, BATCH at a time: all their loads are issued before the first is used (loads behind a
    // per-token bounds test would go out one token at a time).
    typedef typename Vec<T, N>::raw raw_t;
    const int uend = min(t1 + KMAX - 1, p.T);
    int u = t0;
    for (; u + BATCH <= uend; u += BATCH) {
      raw_t xr[BATCH], gr[BATCH];
#pragma unroll
      for (int e = 0; e < BATCH; ++e) {
        xr[e] = *reinterpret_cast<const raw_t*>(xp + (size_t)e * p.D);
        gr[e] = *reinterpret_cast<const raw_t*>(gp + (size_t)e * p.D);
      }
      xp += (size_t)BATCH * p.D, gp += (size_t)BATCH * p.D;
#pragma unroll
      for (int e = 0; e < BATCH; ++e) {
        float g[N];
#pragma unroll
        for (int i = 0; i < N; ++i) win[KMAX - 1][i] = (float)xr[e][i], g[i] = (float)gr[e][i];
        token(u + e, g);
      }
    }
    for (; u < t1 + KMAX - 1; ++u, xp += p.D, gp += p.D) {
      float g[N];
      if (u < uend) {
        load_vec<T, N>(xp, win[KMAX - 1]);
        load_vec<T, N>(gp, g);
      } else {
#pragma unroll
        for (int i = 0; i < N; ++i) win[KMAX - 1][i] = 0.f, g[i] = 0.f;
      }
      token(u, g);
    }
  }
  if (!p.dw) return;
  if (run > 0) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      red[run - 1][KMAX][lane * N + i] = gb[i];
#pragma unroll
      for (int j = 0; j < KMAX; ++j) red[run - 1][j][lane * N + i] = gw[j][i];
    }
  }
  __syncthreads();
  if (run == 0 && c < p.D) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float sb = gb[i];
      for (int r = 0; r < BWD_RUNS - 1; ++r) sb += red[r][KMAX][lane * N + i];
      if (p.dbias) unsafeAtomicAdd(p.dbias + c + i, sb);
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        const int jr = j - (KMAX - p.K);
        if (jr < 0 || p.K == 1) continue;  // a width-1 kernel ignores its weight (conv.py:39-44)
        float s = gw[j][i];
        for (int r = 0; r < BWD_RUNS - 1; ++r) s += red[r][j][lane * N + i];
        unsafeAtomicAdd(p.dw + (size_t)jr * p.D + c + i, s);
      }
    }
  }
}

// Gradient with respect to the carry-in cache: row i of the cache is xin[i - (K-1)], which only the first K-1 outputs
// see.  One thread per (batch row, 16-byte channel group); recomputes z for those outputs.
template <typename T, int N>
__global__ __launch_bounds__(256) void conv1d_dcache_kernel(ConvParams p) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * N;
  const int b = blockIdx.y;
  if (c >= p.D) return;
  float w[KMAX][N], bias[N], win[KMAX][N], dzv[KMAX - 1][N];
  load_taps<N>(p, c, w, bias);
#pragma unroll
  for (int j = 0; j < KMAX - 1; ++j) load_xin<T, N>(p, b, j - (KMAX - 1), c, win[j]);
#pragma unroll
  for (int t = 0; t < KMAX - 1; ++t) {  // outputs 0 .. K-2 (those past the end of a short sequence contribute nothing)
    load_xin<T, N>(p, b, t, c, win[KMAX - 1]);
    float g[N];
    if (t < p.T) load_vec<T, N>(static_cast<const T*>(p.dy) + ((size_t)b * p.T + t) * p.D + c, g);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float d = t < p.T ? g[i] : 0.f;
      if (p.act) {
        float a = bias[i];
#pragma unroll
        for (int j = 0; j < KMAX; ++j) a = fmaf(w[j][i], win[j][i], a);
        const float sg = sigmoidf(a);
        d *= sg * (1.f + a * (1.f - sg));
      }
      dzv[t][i] = d;
    }
#pragma unroll
    for (int j = 0; j < KMAX - 1; ++j)
#pragma unroll
      for (int i = 0; i < N; ++i) win[j][i] = win[j + 1][i];
  }
  // cache row i sits at position s = i - (K-1); output t reads it through tap (KMAX-1) - (t - s)
  T* dp = static_cast<T*>(p.dcache) + (size_t)b * (p.K - 1) * p.D + c;
  for (int i = 0; i < p.K - 1; ++i) {
    const int sp = i - (p.K - 1);
    float r[N];
#pragma unroll
    for (int e = 0; e < N; ++e) r[e] = 0.f;
#pragma unroll
    for (int t = 0; t < KMAX - 1; ++t) {
      const int j = (KMAX - 1) - (t - sp);
      if (j >= 0 && j < KMAX) {
#pragma unroll
        for (int e = 0; e < N; ++e) r[e] = fmaf(w[j][e], dzv[t][e], r[e]);
      }
    }
    store_vec<T, N>(dp + (size_t)i * p.D, r);
  }
}

__global__ void fill_zero_kernel(float* a, int na, float* b, int nb) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < na) a[i] = 0.f;
  if (b && i < nb) b[i] = 0.f;
}

int group_span(int groups) { return groups > 128 ? 256 : groups > 64 ? 128 : 64; }

int check(const ConvParams& p, int dtype, bool bwd) {
  if (p.B < 0 || p.T < 0 || p.D <= 0 || p.K < 1 || p.K > KMAX)
    return lnx_set_error(LNX_ERR_SHAPE, "conv1d: dimensions B=%d T=%d D=%d K=%d (K must be 1..4)", p.B, p.T, p.D, p.K);
  if (dtype != LNX_F32 && dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "conv1d: dtype %d", dtype);
  const int n = dtype == LNX_BF16 ? 8 : 4;
  if (p.D % n) return lnx_set_error(LNX_ERR_SHAPE, "conv1d: D=%d must be a multiple of %d (16-byte channel groups)", p.D, n);
  if (p.act != 0 && p.act != 1) return lnx_set_error(LNX_ERR_SHAPE, "conv1d: activation %d (0 = none, 1 = SiLU)", p.act);
  if (!p.w) return lnx_set_error(LNX_ERR_NULL, "conv1d: weight is required");
  const bool elems = (size_t)p.B * p.T > 0;
  if (elems && !p.x) return lnx_set_error(LNX_ERR_NULL, "conv1d: x is required");
  if (!bwd && elems && !p.y) return lnx_set_error(LNX_ERR_NULL, "conv1d: y is required");
  if (bwd && elems && (!p.dy || !p.dx)) return lnx_set_error(LNX_ERR_NULL, "conv1d: dy and dx are required");
  if (!bwd && p.new_cache && p.new_cache == p.cache && p.T > SEG_FWD)
    return lnx_set_error(LNX_ERR_SHAPE, "conv1d: the cache can be updated in place for T <= %d only", SEG_FWD);
  return 0;
}

}  // namespace

namespace {

int conv_fwd(ConvParams p, int dtype, hipStream_t st) {
  if (int rc = check(p, dtype, false)) return rc;
  const int B = p.B, T = p.T, D = p.D, K = p.K;
  if (K == 1) p.new_cache = nullptr, p.cache = nullptr;  // a width-1 kernel carries nothing
  const int n = dtype == LNX_BF16 ? 8 : 4;
  if ((size_t)B * T == 0) {
    // nothing to convolve: the carry passes through unchanged (zeros without one, like the reference's zero cache)
    if (p.new_cache && p.new_cache != p.cache && B > 0) {
      const size_t bytes = (size_t)B * (K - 1) * D * (dtype == LNX_BF16 ? 2 : 4);
      hipError_t e = p.cache ? hipMemcpyAsync(p.new_cache, p.cache, bytes, hipMemcpyDeviceToDevice, st) : hipSuccess;
      if (!p.cache) fill_zero_kernel<<<(unsigned)((bytes / 4 + 255) / 256), 256, 0, st>>>(static_cast<float*>(p.new_cache), (int)(bytes / 4), nullptr, 0);
      if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "conv1d: cache copy failed");
    }
    return 0;
  }
  const int nseg = (T + SEG_FWD - 1) / SEG_FWD;
  p.gx = group_span(D / n);
  dim3 grid((D / n + p.gx - 1) / p.gx, (nseg * p.gx + 255) / 256, B);
  lnx_profile_mark("conv1d_fwd", st);
  if (p.cu) {
    if (dtype == LNX_BF16) conv1d_fwd_kernel<bf16_t, 8, true><<<grid, 256, 0, st>>>(p);
    else conv1d_fwd_kernel<float, 4, true><<<grid, 256, 0, st>>>(p);
  } else {
    if (dtype == LNX_BF16) conv1d_fwd_kernel<bf16_t, 8, false><<<grid, 256, 0, st>>>(p);
    else conv1d_fwd_kernel<float, 4, false><<<grid, 256, 0, st>>>(p);
  }
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "conv1d_fwd launch: %s", hipGetErrorString(e));
  return 0;
}

int conv_bwd(ConvParams p, int dtype, hipStream_t st) {
  if (int rc = check(p, dtype, true)) return rc;
  if (p.dbias && !p.dw) return lnx_set_error(LNX_ERR_NULL, "conv1d_bwd: d_bias needs d_weight");
  const int B = p.B, T = p.T, D = p.D, K = p.K;
  if (p.dw) {
    lnx_profile_mark("conv1d_fill", st);
    fill_zero_kernel<<<(K * D + 255) / 256, 256, 0, st>>>(p.dw, K * D, p.dbias, D);
  }
  if ((size_t)B * T > 0) {
    const int nseg = (T + SEG_BWD - 1) / SEG_BWD;
    dim3 grid((D / 4 + 63) / 64, (nseg + BWD_RUNS - 1) / BWD_RUNS, B);
    lnx_profile_mark("conv1d_bwd", st);
    if (p.cu) {
      if (dtype == LNX_BF16) conv1d_bwd_kernel<bf16_t, 4, true><<<grid, 256, 0, st>>>(p);
      else conv1d_bwd_kernel<float, 4, true><<<grid, 256, 0, st>>>(p);
    } else {
      if (dtype == LNX_BF16) conv1d_bwd_kernel<bf16_t, 4, false><<<grid, 256, 0, st>>>(p);
      else conv1d_bwd_kernel<float, 4, false><<<grid, 256, 0, st>>>(p);
    }
  }
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "conv1d_bwd launch: %s", hipGetErrorString(e));
  return 0;
}

int check_packed(const int32_t* cu, int nseq) {
  if (!cu || nseq <= 0) return lnx_set_error(LNX_ERR_SHAPE, "conv1d: a packed batch needs cu_seqlens and nseq > 0 (nseq=%d)", nseq);
  return 0;
}

}  // namespace

extern "C" int lnx_conv1d_fwd(const void* x, const float* weight, const float* bias, const void* cache, void* y,
                              void* new_cache, int32_t B, int32_t T, int32_t D, int32_t K, int32_t dtype,
                              int32_t activation, void* hip_stream) {
  ConvParams p{x, weight, bias, cache, y, new_cache, nullptr, nullptr, nullptr, nullptr, B, T, D, K, activation, 64, nullptr, 0, nullptr};
  return conv_fwd(p, dtype, static_cast<hipStream_t>(hip_stream));
}

extern "C" int lnx_conv1d_bwd(const void* x, const float* weight, const float* bias, const void* cache, const void* dy,
                              void* dx, float* d_weight, float* d_bias, int32_t B, int32_t T, int32_t D, int32_t K,
                              int32_t dtype, int32_t activation, void* hip_stream) {
  ConvParams p{x, weight, bias, cache, nullptr, nullptr, dy, dx, d_weight, d_bias, B, T, D, K, activation, 64, nullptr, 0, nullptr};
  return conv_bwd(p, dtype, static_cast<hipStream_t>(hip_stream));
}

extern "C" int lnx_conv1d_packed_fwd(const void* x, const float* weight, const float* bias, const int32_t* cu_seqlens,
                                     int32_t nseq, void* y, void* new_cache, int32_t T, int32_t D, int32_t K, int32_t dtype,
                                     int32_t activation, void* hip_stream) {
  if (int rc = check_packed(cu_seqlens, nseq)) return rc;
  ConvParams p{x, weight, bias, nullptr, y, new_cache, nullptr, nullptr, nullptr, nullptr, 1, T, D, K, activation, 64, cu_seqlens, nseq, nullptr};
  return conv_fwd(p, dtype, static_cast<hipStream_t>(hip_stream));
}

extern "C" int lnx_conv1d_packed_bwd(const void* x, const float* weight, const float* bias, const int32_t* cu_seqlens,
                                     int32_t nseq, const void* dy, void* dx, float* d_weight, float* d_bias, int32_t T,
                                     int32_t D, int32_t K, int32_t dtype, int32_t activation, void* hip_stream) {
  if (int rc = check_packed(cu_seqlens, nseq)) return rc;
  ConvParams p{x, weight, bias, nullptr, nullptr, nullptr, dy, dx, d_weight, d_bias, 1, T, D, K, activation, 64, cu_seqlens, nseq, nullptr};
  return conv_bwd(p, dtype, static_cast<hipStream_t>(hip_stream));
}

extern "C" int lnx_conv1d_cache_bwd(const void* x, const float* weight, const float* bias, const void* cache, const void* dy,
                                    void* d_cache, int32_t B, int32_t T, int32_t D, int32_t K, int32_t dtype,
                                    int32_t activation, void* hip_stream) {
  ConvParams p{x, weight, bias, cache, nullptr, nullptr, dy, d_cache, nullptr, nullptr, B, T, D, K, activation, 64, nullptr, 0, d_cache};
  if (int rc = check(p, dtype, true)) return rc;
  if (K == 1 || B == 0) return 0;  // no carry to differentiate
  if (!d_cache) return lnx_set_error(LNX_ERR_NULL, "conv1d_cache_bwd: d_cache is required");
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const int n = dtype == LNX_BF16 ? 8 : 4;
  dim3 grid((D / n + 255) / 256, B);
  lnx_profile_mark("conv1d_dcache", st);
  if (dtype == LNX_BF16) conv1d_dcache_kernel<bf16_t, 8><<<grid, 256, 0, st>>>(p);
  else conv1d_dcache_kernel<float, 4><<<grid, 256, 0, st>>>(p);
  lnx_profile_mark(nullptr, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "conv1d_cache_bwd launch: %s", hipGetErrorString(e));
  return 0;
}
