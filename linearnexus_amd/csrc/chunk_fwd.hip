// Chunked (WY) delta-rule forward on gfx950 MFMA, three kernels per call:
//
//   chunk_prepare2 (one workgroup per 64-token chunk, all chunks in parallel; kda_prepare for a vector gate)
//       A = tril(diag(beta) K K^T * E, -1);  Tm = (I + A)^-1 (fp32, block forward substitution +
//       MFMA block merges);  W = Tm diag(beta e^G) K;  U = Tm diag(beta) V;
//       P = scale * tril(Q K^T * E);  also Tm^T for the backward pass.
//   chunk_scan     (one workgroup per (state, 64-column slab of dv), sequential over chunks)
//       D = U - W S;  S <- e^{G_last} S + (K e^{G_last - G})^T D, with the fp32 state held in
//       MFMA accumulators across the whole sequence; stores D and the entering state.
//   chunk_output   (one workgroup per (chunk, 64-column slab), all in parallel)
//       O = scale (Q e^G) S_n + P D.
//
// This is the algorithm of linearnexus/modules/linear_attn/gated_deltanet.py:444-523
// (delta_net.py:296-330 without a gate, kda.py:569-648 with a vector gate); E_ij =
// exp(G_i - G_j) with G the cumulative log-decay inside the chunk.

#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "chunk_common.h"

namespace {

struct FwdParams {
  ChunkGeom geom;
  const void* q;
  const void* k;
  const void* v;
  const float* beta;
  const float* g;
  const float* s0;
  float* sT_out;
  void* o;
  int dv, o_dtype;
  int save;  // write the per-chunk tensors the backward pass (or the separate output kernel) reads
  int out_spw;  // chunk_output: value slabs per workgroup
  int vcols;    // leading value columns present in v (its row length); the rest of the dv columns are zero
  int l2norm;   // chunk_prepare2<LITE>: q and k rows are normalised as x / (|x| + 1e-6) inside the kernels
  int slab;     // lnx_scan_args.test_scan_slab
  // per-channel gate formed inside kda_prepare from the raw projection (lnx_scan_args.gate_raw): element type of q
  const void* graw;
  const float* gA;
  const float* gbias;
  float gthr;
  float scale;
  char* ws;
  ChunkWs off;
};

template <typename T> __device__ __forceinline__ T* ws_ptr(const FwdParams& p, uint64_t off) {
  return reinterpret_cast<T*>(p.ws + off);
}

// Inclusive prefix sum over the 64 lanes of a wavefront.
__device__ __forceinline__ float wave_cumsum(float x, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const float y = __shfl_up(x, d, LNX_WAVE);
    if (lane >= d) x += y;
  }
  return x;
}

// ---------------------------------------------------------------------------------------
// chunk_prepare2 (no gate / scalar gate), organised as slab loops with register prefetch so
// that three workgroups fit a CU: K K^T and Q K^T over
// 64-channel slabs, the fp32 inverse, then one 64-column slab of [dk | dv] at a time for
// W and U, every result leaving through LDS with 16-byte stores.
// ---------------------------------------------------------------------------------------
template <typename T, int DK> struct Prep2Cfg {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int LDC = LNX_C + PAD;
  static constexpr int kTile = 64 * LDC;
  static constexpr size_t cmax(size_t a, size_t b) { return a > b ? a : b; }
  static constexpr size_t mat = sizeof(float) * 64 * LNX_LDA;  // one fp32 64x64 matrix
  static constexpr size_t scr = sizeof(float) * 32 * 36;       // scratch of the inverse's block merges
  // Two regions, each used by one thing at a time (2-byte inputs: 18 + 0.5 + 21.5 KB = 40 KB, four workgroups per CU):
  //   region 0: A (fp32)                      -> after the inverse: Tw, Tu tiles
  //   region 2: K, Q slab tiles, then P       -> Tm (fp32) + merge scratch -> loop-2 slab and result tiles
  static constexpr size_t r0 = cmax(mat, 2 * kTile * sizeof(T));
  static constexpr size_t r1 = sizeof(float) * 128;  // beta, G
  static constexpr size_t r2 = cmax(mat + scr, 2 * kTile * sizeof(T));
  static constexpr size_t bytes = r0 + r1 + r2;
  // LITE: the slab tiles, then A inverted in place + merge scratch | beta, G, row factors | P   (31.5 KB, five per CU)
  static constexpr size_t lite_bytes = mat + scr + sizeof(float) * 256 + kTile * sizeof(T);
};

// LITE: stop after the inverse and leave Tm itself (row-major) next to Pm and G -- all that the kernels of
// chunk_direct.hip read; V is not touched.
template <typename T, int DK, int GATE, bool LITE = false>
__global__ __launch_bounds__(256, LITE ? 5 : 1) void chunk_prepare2_kernel(FwdParams p) {
  typedef Prep2Cfg<T, DK> L;
  constexpr int LDC = L::LDC, NKS = DK / 64;
  extern __shared__ __align__(16) char smem[];
  float* sA = reinterpret_cast<float*>(smem);      // region 0 (LITE: over the slab tiles)
  T* sTw = reinterpret_cast<T*>(smem);             //   Tw, Tu once the inverse is done with A
  T* sTu = sTw + L::kTile;
  float* sBeta = reinterpret_cast<float*>(smem + (LITE ? L::mat + L::scr : L::r0));
  float* sG = sBeta + 64;
  char* reg2 = LITE ? smem : smem + L::r0 + L::r1;  // region 2
  T* sKa = reinterpret_cast<T*>(reg2);             //   K slab of the first loop, then P
  T* sQa = sKa + L::kTile;                         //   Q slab
  float* sT = reinterpret_cast<float*>(reg2);      //   Tm
  float* sX = reinterpret_cast<float*>(reg2 + L::mat);
  T* sIn = sKa;                                    //   second loop: slab in, result out
  T* sOut = sQa;
  T* sPt = LITE ? reinterpret_cast<T*>(smem + L::mat + L::scr + sizeof(float) * 256) : sKa;  // P on its way out

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  const int64_t slot = blockIdx.x;
  const int row = (int)(slot / N), n = (int)(slot % N);
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  if (len <= 0) return;
  const int64_t tbase = tok_index(p.geom, row, tok0);
  const int64_t tsk = (int64_t)p.geom.ts * DK, tsv = (int64_t)p.geom.ts * p.vcols;  // row strides of the token tiles
  const T* qg = reinterpret_cast<const T*>(p.q) + tbase * DK;
  const T* kg = reinterpret_cast<const T*>(p.k) + tbase * DK;
  const T* vg = reinterpret_cast<const T*>(p.v) + tbase * p.vcols;
  const int wi = wave >> 1, wj = wave & 1;

  // LITE with two slabs: all four tiles are requested at once, so the latency of the loads is waited out once
  constexpr bool AHEAD = LITE && NKS == 2;
  TileRegs<T, 64, 64> rK, rQ, rK1, rQ1;
  rK.load(kg, tsk, len, tid);
  rQ.load(qg, tsk, len, tid);
  if (AHEAD) {
    rK1.load(kg + 64, tsk, len, tid);
    rQ1.load(qg + 64, tsk, len, tid);
  }
  if (wave == 0) {
    const bool ok = lane < len;
    sBeta[lane] = ok ? p.beta[tbase + (int64_t)lane * p.geom.ts] : 0.f;
    float gv = 0.f;
    if (GATE == LNX_GATE_SCALAR && ok) gv = p.g[tbase + (int64_t)lane * p.geom.ts];
    gv = wave_cumsum(gv, lane);
    sG[lane] = gv;
    ws_ptr<float>(p, p.off.G)[slot * 64 + lane] = gv;
  }
  floatx16 ax[1][1], ap[1][1];
  frag_zero(ax);
  frag_zero(ap);
  float nk2 = 0.f, nq2 = 0.f;  // LITE: squared row norms, thread = (row tid / 4, 16 columns of the slab)
#pragma unroll(AHEAD ? 2 : 1)
  for (int s_ = 0; s_ < NKS; ++s_) {
    lds_barrier();
    if (AHEAD && s_ == 1) {
      rK1.store(sKa, LDC, tid);
      rQ1.store(sQa, LDC, tid);
    } else {
      rK.store(sKa, LDC, tid);
      rQ.store(sQa, LDC, tid);
    }
    lds_barrier();
    if (!AHEAD && s_ + 1 < NKS) {
      rK.load(kg + 64 * (s_ + 1), tsk, len, tid);
      rQ.load(qg + 64 * (s_ + 1), tsk, len, tid);
    }
    if (!(wi == 0 && wj == 1)) {
      mma_nt<T, 1, 1>(ax, sKa + 32 * wi * LDC, LDC, sKa + 32 * wj * LDC, LDC, 64, lane);
      mma_nt<T, 1, 1>(ap, sQa + 32 * wi * LDC, LDC, sKa + 32 * wj * LDC, LDC, 64, lane);
    }
    if (LITE && p.l2norm) {
      const int r = tid >> 2, c0 = (tid & 3) * 16;
#pragma unroll
      for (int u = 0; u < 16; u += 4) {
        const floatx4 k4 = load4(sKa + r * LDC + c0 + u), q4 = load4(sQa + r * LDC + c0 + u);
#pragma unroll
        for (int e = 0; e < 4; ++e) nk2 += k4[e] * k4[e], nq2 += q4[e] * q4[e];
      }
    }
  }
  // LITE: per-row factors 1 / (|x| + eps) (1 without the normalisation), kept behind the slab tiles and written to the
  // workspace for the scans and the chunk-local backward, which scale the rows as they stage them
  float* sNk = sBeta + 128;
  float* sNq = sNk + 64;
  if constexpr (LITE) {
    nk2 = quad_sum(nk2);
    nq2 = quad_sum(nq2);
    if ((tid & 3) == 0) {
      const int r = tid >> 2;
      const float fk = p.l2norm ? 1.f / (sqrtf(nk2) + LNX_L2_EPS) : 1.f, fq = p.l2norm ? 1.f / (sqrtf(nq2) + LNX_L2_EPS) : 1.f;
      sNk[r] = fk;
      sNq[r] = fq;
      ws_ptr<float>(p, p.off.Nk)[slot * 64 + r] = fk;
      ws_ptr<float>(p, p.off.Nq)[slot * 64 + r] = fq;
      ws_ptr<float>(p, p.off.Fq)[slot * 64 + r] = p.scale * fq * ((GATE == LNX_GATE_SCALAR) ? __expf(sG[r]) : 1.f);
    }
  }
  // first slab of the second loop, in flight during the inverse
  TileRegs<T, 64, 64> rIn;
  auto fetch = [&](int s_) {
    if (s_ < NKS) rIn.load(kg + 64 * s_, tsk, len, tid);
    else if (64 * (s_ - NKS) < p.vcols) rIn.load(vg + 64 * (s_ - NKS), tsv, len, tid);
    else rIn.zero();  // value columns that v does not hold
  };
  if (!LITE) fetch(0);
  lds_barrier();  // slab tiles dead
  {
    // the per-row scalars of this lane's sixteen fragment rows (four runs of four) first, as vectors: read one by one
    // between the stores below, each read waited for its own round trip to LDS (the stores might alias them)
    floatx4 gi[4], bi[4], nki[4], nqi[4];
    const int j = 32 * wj + frag_col(lane);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i0 = 32 * wi + 8 * q + 4 * (lane >> 5);
      gi[q] = load4(sG + i0);
      bi[q] = load4(sBeta + i0);
      if (LITE) nki[q] = load4(sNk + i0), nqi[q] = load4(sNq + i0);
    }
    const float gj = sG[j], nkj = LITE ? sNk[j] : 1.f;
    floatx16 pe[1][1];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = 32 * wi + frag_row(e, lane), q = e >> 2, u = e & 3;
      const float dec = (GATE == LNX_GATE_NONE) ? 1.f : __expf(fminf(gi[q][u] - gj, 0.f));
      const float fx = LITE ? nki[q][u] * nkj : 1.f, fp = LITE ? nqi[q][u] * nkj : 1.f;
      sA[i * LNX_LDA + j] = (i > j) ? bi[q][u] * dec * fx * ax[0][0][e] : 0.f;
      pe[0][0][e] = (i >= j) ? p.scale * dec * fp * ap[0][0][e] : 0.f;
    }
    frag_store<T, 1, 1>(pe, sPt + 32 * wi * LDC + 32 * wj, LDC, lane);
  }
  lds_barrier();
  // LITE, 2-byte inputs: Pm and Tm leave packed (TriRegs in mma_tiles.h), only the vectors at or below the diagonal;
  // this thread's vector tid and, for tid < 32, vector 256 + tid
  int tr0 = 0, tc0 = 0, tr1 = 0, tc1 = 0;
  const bool tri2 = tid < LNX_TRI_VECS - 256;
  if constexpr (LITE && sizeof(T) == 2) {
    tri_vec_pos(tid, tr0, tc0);
    tri_vec_pos(tri2 ? 256 + tid : 0, tr1, tc1);
    T* Pg = ws_ptr<T>(p, p.off.P) + slot * 64 * 64;
    typedef typename Vec16<T>::V V;
    *reinterpret_cast<V*>(Pg + 8 * tid) = *reinterpret_cast<const V*>(sPt + tr0 * LDC + 8 * tc0);
    if (tri2) *reinterpret_cast<V*>(Pg + 8 * (256 + tid)) = *reinterpret_cast<const V*>(sPt + tr1 * LDC + 8 * tc1);
  } else {
    unstage_tile<T, 64, 64>(ws_ptr<T>(p, p.off.P) + slot * 64 * 64, 64, sPt, LDC, 64, tid);
  }
  if constexpr (LITE) {
    tri_inverse_64<true>(sA, sA, sX, tid);
  } else {
    lds_barrier();  // Tm is built over the P tile
    tri_inverse_64(sA, sT, sX, tid);
  }
  if constexpr (LITE) {
    T* Tm = ws_ptr<T>(p, p.off.Tm) + slot * 64 * 64;
    if constexpr (sizeof(T) == 2) {
      typedef unsigned uint2_ __attribute__((ext_vector_type(2)));
      typedef unsigned uint4_ __attribute__((ext_vector_type(4)));
      auto put = [&](int idx, int r, int c) {
        const float* src = sA + r * LNX_LDA + 8 * c;
        const uint2_ lo = __builtin_bit_cast(uint2_, pack_bf16x4(load4(src))), hi = __builtin_bit_cast(uint2_, pack_bf16x4(load4(src + 4)));
        *reinterpret_cast<uint4_*>(Tm + 8 * idx) = uint4_{lo[0], lo[1], hi[0], hi[1]};
      };
      put(tid, tr0, tc0);
      if (tri2) put(256 + tid, tr1, tc1);
    } else {
      for (int idx = tid; idx < 64 * 16; idx += 256) {
        const int r = idx >> 4, c = (idx & 15) * 4;
        store4(Tm + r * 64 + c, load4(sA + r * LNX_LDA + c));
      }
    }
    return;
  }
  {
    T* TmT = ws_ptr<T>(p, p.off.TmT) + slot * 64 * 64;
    // one 4x4 block of Tm per thread: four-element row reads, the transpose taken in registers
    const int r0 = (tid >> 4) * 4, c0 = (tid & 15) * 4;
    floatx4 t[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = load4(sT + (r0 + i) * LNX_LDA + c0);
    const floatx4 bu = load4(sBeta + c0);
    floatx4 bw = bu;
    if (GATE != LNX_GATE_NONE) {
      const floatx4 g4 = load4(sG + c0);
#pragma unroll
      for (int e = 0; e < 4; ++e) bw[e] = bu[e] * __expf(g4[e]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      store4(sTu + (r0 + i) * LDC + c0, t[i] * bu);
      store4(sTw + (r0 + i) * LDC + c0, t[i] * bw);
      if (p.save) store4(TmT + (c0 + i) * 64 + r0, floatx4{t[0][i], t[1][i], t[2][i], t[3][i]});
    }
  }
  const int nslab = NKS + p.dv / 64;
#pragma unroll 1
  for (int s_ = 0; s_ < nslab; ++s_) {
    const bool is_k = s_ < NKS;
    lds_barrier();  // fp32 matrices / previous slab's tiles are dead
    rIn.store(sIn, LDC, tid);
    lds_barrier();
    if (s_ + 1 < nslab) fetch(s_ + 1);
    floatx16 acc[1][1];
    frag_zero(acc);
    // W = Tw K, U = Tu V: the slab is [token][column], contracted along its rows
    mma_x<T, 1, 1, false, true>(acc, (is_k ? sTw : sTu) + 32 * wi * LDC, LDC, sIn + 32 * wj, LDC, 64, lane);
    frag_store<T, 1, 1>(acc, sOut + 32 * wi * LDC + 32 * wj, LDC, lane);
    lds_barrier();
    if (is_k)
      unstage_tile<T, 64, 64>(ws_ptr<T>(p, p.off.W) + slot * 64 * DK + 64 * s_, DK, sOut, LDC, 64, tid);
    else
      unstage_tile<T, 64, 64>(ws_ptr<T>(p, p.off.U) + slot * 64 * p.dv + 64 * (s_ - NKS), p.dv, sOut, LDC, 64, tid);
  }
}

// ---------------------------------------------------------------------------------------
// One 64-channel half of the forward pair products X_ij = sum_c k_i k_j E_ij and <q_i, k_j>_E for 2-byte inputs, on
// v_mfma_f32_16x16x32_bf16.  Level H (32 .. 1) pairs a row token i (bit H set) with a column token j (bit H clear) of
// the same 2H-token segment through the reference m = segment start + H:  E_ij = exp(G_i - G_m) exp(G_m - G_j), both
// factors <= 1; each operand row is a token's K (or Q) times its factor, rounded to bf16.  Lane = (token l16 of a
// 16-token block, kq): channels 8 kq .. 8 kq + 7 of each 32-channel step.  Nothing is shared between waves, so there is
// no barrier: wave w forms block (2 + w / 2, w % 2) of both products (level 32), one product of block (1, 0) or (3, 2)
// (level 16) and the diagonal block w (levels 8 .. 1 and the plain diagonal <q_i, k_i>).
// K, Q [64][ldc] bf16, G [64][ldf] fp32 (cumulative gate), all in LDS.
// ---------------------------------------------------------------------------------------
struct PairOp {
  bf16x8 lo, hi;  // channels 8 kq + 0..7 and 32 + 8 kq + 0..7 of this lane's token
};
__device__ __forceinline__ void pair_row_f32(float (&v)[16], const float* __restrict__ rowp) {  // rowp: row + 8 kq
  const floatx4 a = load4(rowp), b = load4(rowp + 4), c = load4(rowp + 32), d = load4(rowp + 36);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[e] = a[e];
    v[4 + e] = b[e];
    v[8 + e] = c[e];
    v[12 + e] = d[e];
  }
}
__device__ __forceinline__ PairOp pair_row_raw(const bf16_t* __restrict__ rowp) {
  return PairOp{*reinterpret_cast<const bf16x8*>(rowp), *reinterpret_cast<const bf16x8*>(rowp + 32)};
}
__device__ __forceinline__ PairOp pair_scaled(const PairOp& x, const float (&F)[16]) {  // F x, rounded to bf16
  typedef unsigned uint4_ __attribute__((ext_vector_type(4)));
  typedef float floatx2_ __attribute__((ext_vector_type(2)));
  uint4_ lo, hi;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const floatx2_ a = {F[2 * w] * (float)x.lo[2 * w], F[2 * w + 1] * (float)x.lo[2 * w + 1]};
    const floatx2_ b = {F[8 + 2 * w] * (float)x.hi[2 * w], F[8 + 2 * w + 1] * (float)x.hi[2 * w + 1]};
    lo[w] = __builtin_bit_cast(unsigned, __builtin_convertvector(a, bf16x2));
    hi[w] = __builtin_bit_cast(unsigned, __builtin_convertvector(b, bf16x2));
  }
  return PairOp{__builtin_bit_cast(bf16x8, lo), __builtin_bit_cast(bf16x8, hi)};
}
__device__ __forceinline__ PairOp pair_masked(const PairOp& x, unsigned m) {
  typedef unsigned uint4_ __attribute__((ext_vector_type(4)));
  return PairOp{__builtin_bit_cast(bf16x8, __builtin_bit_cast(uint4_, x.lo) & m), __builtin_bit_cast(bf16x8, __builtin_bit_cast(uint4_, x.hi) & m)};
}
__device__ __forceinline__ void pair_mma(floatx4& acc, const PairOp& a, const PairOp& b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.lo, b.lo, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.hi, b.hi, acc, 0, 0, 0);
}
// factors exp(-(ga - gb)) clamped to <= 1 (ga >= gb up to rounding: the cumulative gate does not increase)
__device__ __forceinline__ void pair_factors(float (&F)[16], const float (&ga)[16], const float (&gb)[16]) {
#pragma unroll
  for (int x = 0; x < 16; ++x) F[x] = __expf(fminf(gb[x] - ga[x], 0.f));
}

__device__ __forceinline__ void kda_pair_half(floatx4 (&a32)[2], floatx4& a16, floatx4 (&aD)[5][2], const bf16_t* __restrict__ K,
                                              const bf16_t* __restrict__ Q, int ldc, const float* __restrict__ G, int ldf,
                                              int wave, int lane) {
  const int l16 = lane & 15, kq = lane >> 4;
  const bf16_t* Kc = K + 8 * kq;
  const bf16_t* Qc = Q + 8 * kq;
  const float* Gc = G + 8 * kq;
  float gi[16], gj[16], gm[16], F[16];
  {  // level 32: rows 16 ti + l16 against columns 16 tj + l16, reference token 32
    const int i = 16 * (2 + (wave >> 1)) + l16, j = 16 * (wave & 1) + l16;
    pair_row_f32(gm, Gc + 32 * ldf);
    pair_row_f32(gi, Gc + i * ldf);
    pair_row_f32(gj, Gc + j * ldf);
    pair_factors(F, gm, gi);  // exp(G_i - G_32)
    const PairOp kr = pair_scaled(pair_row_raw(Kc + i * ldc), F), qr = pair_scaled(pair_row_raw(Qc + i * ldc), F);
    pair_factors(F, gj, gm);  // exp(G_32 - G_j)
    const PairOp kc = pair_scaled(pair_row_raw(Kc + j * ldc), F);
    pair_mma(a32[0], kr, kc);
    pair_mma(a32[1], qr, kc);
  }
  __builtin_amdgcn_sched_barrier(0);  // one level at a time keeps the live operands few
  {  // level 16: block (1, 0) or (3, 2), reference its first row token; waves 0, 2: K rows, waves 1, 3: Q rows
    const int m = (wave < 2) ? 16 : 48, i = m + l16, j = m - 16 + l16;
    pair_row_f32(gm, Gc + m * ldf);
    pair_row_f32(gi, Gc + i * ldf);
    pair_row_f32(gj, Gc + j * ldf);
    pair_factors(F, gm, gi);
    const PairOp r = pair_scaled(pair_row_raw(((wave & 1) ? Qc : Kc) + i * ldc), F);
    pair_factors(F, gj, gm);
    const PairOp kc = pair_scaled(pair_row_raw(Kc + j * ldc), F);
    pair_mma(a16, r, kc);
  }
  __builtin_amdgcn_sched_barrier(0);
  {  // diagonal block `wave`: token i = 16 wave + l16 is a row token of level H when bit H of l16 is set
    const int i = 16 * wave + l16;
    pair_row_f32(gi, Gc + i * ldf);
    const PairOp kraw = pair_row_raw(Kc + i * ldc), qraw = pair_row_raw(Qc + i * ldc);
    pair_mma(aD[4][1], qraw, kraw);  // only its diagonal is kept
#pragma unroll
    for (int lv = 0; lv < 4; ++lv) {
      const int H = 8 >> lv;
      const bool up = (l16 & H) != 0;
      const int m = 16 * wave + ((l16 & ~(2 * H - 1)) | H);
      pair_row_f32(gm, Gc + m * ldf);
#pragma unroll
      for (int x = 0; x < 16; ++x) F[x] = __expf(fminf(up ? gi[x] - gm[x] : gm[x] - gi[x], 0.f));
      const PairOp pk = pair_scaled(kraw, F), pq = pair_scaled(qraw, F);
      const unsigned mu = up ? 0xffffffffu : 0u;
      const PairOp kb = pair_masked(pk, ~mu);
      pair_mma(aD[lv][0], pair_masked(pk, mu), kb);
      pair_mma(aD[lv][1], pair_masked(pq, mu), kb);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}


// ---------------------------------------------------------------------------------------
// kda_prepare: chunk_prepare for a per-channel (vector) gate.  The pairwise products carry the
// decay inside the dk sum, X_ij = sum_c k_i[c] k_j[c] exp(G_i[c] - G_j[c]).  The channels are
// taken in 64-wide halves (K, Q and the fp32 gate tile of one half fit LDS twice per CU): per half
// the cumulative gate, K e^{G_last - G} and scale Q e^G go to the workspace and the half's share of
// the pair products is accumulated -- 16x16 blocks below the diagonal on the fp32 MFMA with the
// decay factored through the first row of the row block (kda.py:504-523), diagonal blocks on the
// VALU with exponents of non-positive numbers only (kda.py:483-502).  After the inverse, W and U
// are formed by one loop over 64-column slabs of [K | V] with register prefetch, results leaving
// through LDS with 16-byte stores.
// ---------------------------------------------------------------------------------------
template <typename T, int DK> struct KdaPrepSmem {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int LDC = LNX_C + PAD, LDF = 64 + 4;
  static constexpr int kTile = 64 * LDC;
  // K half (later Tm), Q half (later Tm diag(beta)); gate half (later the staged slab); A (later the
  // output staging); the P accumulator / inverse; inverse scratch; beta
  static constexpr size_t bytes = sizeof(T) * 2 * kTile + sizeof(float) * (64 * LDF + 2 * 64 * LNX_LDA + 32 * 36 + 64);
};

// GRAW: the gate arrives as the block's raw projection and is activated here, g = -exp(A_log[h]) softplus(raw + bias)
// (kda.py:153-165), on its way into LDS: the activated fp32 gate tensor is never written or read.
template <typename T, int DK, bool GRAW>
__global__ __launch_bounds__(256, (sizeof(T) == 2 ? 2 : 1)) void kda_prepare_kernel(FwdParams p) {
  typedef KdaPrepSmem<T, DK> L;
  constexpr int LDC = L::LDC, LDF = L::LDF, NH = DK / 64;
  extern __shared__ __align__(16) char smem[];
  T* sK = reinterpret_cast<T*>(smem);
  T* sQ = sK + L::kTile;
  float* sG = reinterpret_cast<float*>(sQ + L::kTile);  // [64][LDF] cumulative gate of the half
  float* sA = sG + 64 * LDF;
  float* sT = sA + 64 * LNX_LDA;
  float* sX = sT + 64 * LNX_LDA;
  float* sBeta = sX + 32 * 36;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  const int64_t slot = blockIdx.x;
  const int row = (int)(slot / N), n = (int)(slot % N);
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  if (len <= 0) return;
  const int64_t tbase = tok_index(p.geom, row, tok0);
  const int64_t tsk = (int64_t)p.geom.ts * DK, tsv = (int64_t)p.geom.ts * p.vcols;  // row strides of the token tiles
  const T* qg = reinterpret_cast<const T*>(p.q) + tbase * DK;
  const T* kg = reinterpret_cast<const T*>(p.k) + tbase * DK;
  const T* vg = reinterpret_cast<const T*>(p.v) + tbase * p.vcols;
  float* Gg = ws_ptr<float>(p, p.off.G) + slot * 64 * DK;
  const int l16 = lane & 15, kq = lane >> 4;

  // ---- phase A: per 64-channel half ----
  TileRegs<T, 64, 64> rK, rQ;
  TileRegs<typename std::conditional<GRAW, T, float>::type, 64, 64> rG;
  const float gna = GRAW ? -__expf(p.gA[row % p.geom.H]) : 0.f;
  typedef TileRegs<T, 64, 64> GT;
  float gbias[GRAW ? GT::N : 1];  // the bias of this thread's channel group (256 % VPR == 0: the same group in every pass)
  auto fetch_half = [&](int h) {
    rK.load(kg + 64 * h, tsk, len, tid);
    rQ.load(qg + 64 * h, tsk, len, tid);
    if constexpr (GRAW) {
      rG.load(reinterpret_cast<const T*>(p.graw) + tbase * DK + 64 * h, tsk, len, tid);
#pragma unroll
      for (int e = 0; e < GT::N; ++e) gbias[e] = p.gbias ? p.gbias[(row % p.geom.H) * DK + 64 * h + (tid % GT::VPR) * GT::N + e] : 0.f;
    } else {
      rG.load(p.g + tbase * DK + 64 * h, tsk, len, tid);
    }
  };
  // the raw gate tile -> activated fp32 gate in LDS; rows past the chunk's end stay zero (they read as raw zeros,
  // whose activation is not zero)
  auto store_gate = [&](int h) {
    if constexpr (GRAW) {
      const int c = (tid % GT::VPR) * GT::N;
#pragma unroll
      for (int it = 0; it < GT::IT; ++it) {
        const int r = (tid + 256 * it) / GT::VPR;
#pragma unroll
        for (int e0 = 0; e0 < GT::N; e0 += 4) {
          floatx4 g4;
#pragma unroll
          for (int e = 0; e < 4; ++e) g4[e] = r < len ? gna * lnx_softplus_thr(to_f32(rG.x[it][e0 + e]) + gbias[e0 + e], p.gthr) : 0.f;
          store4(sG + r * LDF + c + e0, g4);
        }
      }
    } else {
      rG.store(sG, LDF, tid);
    }
  };
  fetch_half(0);
  if (tid < 64) sBeta[tid] = (tid < len) ? p.beta[tbase + (int64_t)tid * p.geom.ts] : 0.f;
  floatx4 acc[3];  // this wave's three below-diagonal tasks (block, product), summed over the halves
#pragma unroll
  for (int u = 0; u < 3; ++u) acc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
  // 2-byte inputs: the pair products by levels on the bf16 MFMA (see pair_levels in chunk_common.h for the splitting).
  // Wave w holds, summed over the halves: block (2 + w / 2, w % 2) of both products (level 32), one product of block
  // (1, 0) or (3, 2) (level 16), and the diagonal block w of both products, one accumulator per level 8, 4, 2, 1 (each
  // level has its own mask) plus the plain <q_i, k_i> diagonal.
  constexpr bool LEVELS = sizeof(T) == 2;
  floatx4 a32[2], a16, aD[5][2];
  a32[0] = a32[1] = a16 = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 5; ++u) aD[u][0] = aD[u][1] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int idx = tid; idx < 64 * LNX_LDA; idx += 256) {  // the diagonal blocks accumulate here over the halves
    sA[idx] = 0.f;
    sT[idx] = 0.f;
  }

#pragma unroll 1
  for (int h = 0; h < NH; ++h) {
    lds_barrier();  // the previous half's tiles are dead
    rK.store(sK, LDC, tid);
    rQ.store(sQ, LDC, tid);
    store_gate(h);
    lds_barrier();
    if (h + 1 < NH) fetch_half(h + 1);
    {  // cumulative gate along the tokens, per channel: 16-row segments in parallel, then their offsets
      const int c = tid & 63, seg = tid >> 6;
      float gs[16];  // the segment's sixteen values in registers: all loads in flight together, one write each
#pragma unroll
      for (int i = 0; i < 16; ++i) gs[i] = sG[(16 * seg + i) * LDF + c];
#pragma unroll
      for (int i = 1; i < 16; ++i) gs[i] += gs[i - 1];
      float* sSeg = sX;  // segment totals [4][64] (the inverse's scratch is free here)
      sSeg[seg * 64 + c] = gs[15];
      lds_barrier();
      float off = 0.f;
      for (int s_ = 0; s_ < seg; ++s_) off += sSeg[s_ * 64 + c];
#pragma unroll
      for (int i = 0; i < 16; ++i) sG[(16 * seg + i) * LDF + c] = gs[i] + off;
    }
    lds_barrier();
    {  // G, K e^{G_last - G}, scale Q e^G of this half -> workspace
      T* Krg = ws_ptr<T>(p, p.off.Kr) + slot * 64 * DK + 64 * h;
      T* Qgg = ws_ptr<T>(p, p.off.Qg) + slot * 64 * DK + 64 * h;
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
        const floatx4 gr = load4(sG + r * LDF + c), gl = load4(sG + 63 * LDF + c);
        const floatx4 kk = load4(sK + r * LDC + c), qq = load4(sQ + r * LDC + c);
        floatx4 kr, qgv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          kr[e] = kk[e] * __expf(fminf(gl[e] - gr[e], 0.f));
          qgv[e] = qq[e] * p.scale * __expf(gr[e]);
        }
        store4(Gg + r * DK + 64 * h + c, gr);
        store4(Krg + r * DK + c, kr);
        store4(Qgg + r * DK + c, qgv);
      }
    }
    if constexpr (LEVELS) {
      kda_pair_half(a32, a16, aD, reinterpret_cast<const bf16_t*>(sK), reinterpret_cast<const bf16_t*>(sQ), LDC, sG, LDF, wave, lane);
    } else {
    // blocks below the diagonal: six blocks x two products = twelve tasks, three per wave
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const int t = wave + 4 * u;
      const int pr = t % 6, I = (pr < 1) ? 1 : (pr < 3) ? 2 : 3, J = pr - ((I == 1) ? 0 : (I == 2) ? 1 : 3);
      const T* sRow = (t < 6) ? sK : sQ;
      const int i = 16 * I + l16, j = 16 * J + l16;
#pragma unroll 8
      for (int ks = 0; ks < 16; ++ks) {
        const int c = 4 * ks + kq;
        const float gref = sG[16 * I * LDF + c];
        const float fa = __expf(fminf(sG[i * LDF + c] - gref, 0.f));
        const float fb = __expf(fminf(gref - sG[j * LDF + c], 0.f));
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(to_f32(sRow[i * LDC + c]) * fa, to_f32(sK[j * LDC + c]) * fb, acc[u], 0, 0, 0);
      }
    }
    {  // diagonal blocks: wave = block; lane = (row slot, quarter q4 of the half's channels).  Rows rp and 15 - rp
       // together have 17 columns j <= i; the two slots of a row pair take nine and eight of them.  The quarters are
       // summed inside the quad, so the only cross-lane traffic is two DPP permutes per value.
      const int q4 = lane & 3, slot_ = lane >> 2, rp = slot_ & 7, t0 = (slot_ >> 3) * 9, r0 = 16 * wave;
#pragma unroll 3
      for (int u = 0; u < 9; ++u) {
        const int t = min(t0 + u, 16);  // the second slot's ninth pass repeats its eighth and is dropped below
        const bool first = t <= rp;
        const int i = r0 + (first ? rp : 15 - rp), j = r0 + (first ? t : t - rp - 1);
        float x = 0.f, pp = 0.f;
#pragma unroll
        for (int c = 16 * q4; c < 16 * q4 + 16; c += 4) {
          const floatx4 ki = load4(sK + i * LDC + c), qi = load4(sQ + i * LDC + c), gi = load4(sG + i * LDF + c);
          const floatx4 kj = load4(sK + j * LDC + c), gj = load4(sG + j * LDF + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float ee = __expf(fminf(gi[e] - gj[e], 0.f)) * kj[e];
            x += ki[e] * ee;
            pp += qi[e] * ee;
          }
        }
        x = quad_sum(x);
        pp = quad_sum(pp);
        if (q4 == 0 && t0 + u < 17) {  // the same lane owns (i, j) in every half
          sA[i * LNX_LDA + j] += x;
          sT[i * LNX_LDA + j] += pp;
        }
      }
    }
    }
  }
  // From here on every index is derived from a thread id that has passed through an empty asm: what the phases below
  // need would otherwise be formed at the kernel's start, spilled across phase A, and each reload would wait until all
  // earlier stores have been acknowledged (the memory counter retires in order).
  int tid_late = threadIdx.x;
  asm volatile("" : "+v"(tid_late));
  {
  const int tid = tid_late, wave = tid >> 6, lane = tid & 63, l16 = lane & 15, kq = lane >> 4;
  // ---- phase B: assemble X and <q, k>_E in sA / sT, write X and P, A = beta X, inverse ----
  if constexpr (LEVELS) {
    const int ti = 2 + (wave >> 1), tj = wave & 1, t16 = (wave < 2) ? 1 : 3;
    float* d16 = (wave & 1) ? sT : sA;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int il = 4 * kq + e;  // row inside the 16x16 block, column l16
      sA[(16 * ti + il) * LNX_LDA + 16 * tj + l16] = a32[0][e];
      sT[(16 * ti + il) * LNX_LDA + 16 * tj + l16] = a32[1][e];
      d16[(16 * t16 + il) * LNX_LDA + 16 * (t16 - 1) + l16] = a16[e];
      // diagonal block: level H keeps the pairs inside one 2H-token segment (the roles are in the operands already)
      const int x = il ^ l16;
      float va = aD[0][0][e], vp = aD[0][1][e];
      va += (x < 8) ? aD[1][0][e] : 0.f;
      vp += (x < 8) ? aD[1][1][e] : 0.f;
      va += (x < 4) ? aD[2][0][e] : 0.f;
      vp += (x < 4) ? aD[2][1][e] : 0.f;
      va += (x < 2) ? aD[3][0][e] : 0.f;
      vp += (x < 2) ? aD[3][1][e] : 0.f;
      vp += (x == 0) ? aD[4][1][e] : 0.f;
      sA[(16 * wave + il) * LNX_LDA + 16 * wave + l16] = va;
      sT[(16 * wave + il) * LNX_LDA + 16 * wave + l16] = vp;
    }
  } else {
#pragma unroll
  for (int u = 0; u < 3; ++u) {
    const int t = wave + 4 * u;
    const int pr = t % 6, I = (pr < 1) ? 1 : (pr < 3) ? 2 : 3, J = pr - ((I == 1) ? 0 : (I == 2) ? 1 : 3);
    float* dst = (t < 6) ? sA : sT;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[(16 * I + 4 * kq + e) * LNX_LDA + 16 * J + l16] = acc[u][e];
  }
  }
  lds_barrier();
  {
    T* Pg = ws_ptr<T>(p, p.off.P) + slot * 64 * 64;
    T* Xg = ws_ptr<T>(p, p.off.X) + slot * 64 * 64;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + 256 * it, i = idx >> 4, j0 = (idx & 15) * 4;
      floatx4 x = load4(sA + i * LNX_LDA + j0), pp = load4(sT + i * LNX_LDA + j0);
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // entries above the diagonal of the diagonal blocks were never written
        x[e] = (j0 + e < i) ? x[e] : 0.f;
        pp[e] = (j0 + e <= i) ? p.scale * pp[e] : 0.f;
      }
      if (p.save) store4(Xg + i * 64 + j0, x);
      store4(Pg + i * 64 + j0, pp);
      store4(sA + i * LNX_LDA + j0, x * sBeta[i]);
    }
  }
  lds_barrier();
  tri_inverse_64(sA, sT, sX, tid);

  // ---- phase C: Tm^T to the workspace; Tm and Tm diag(beta) as MFMA operands ----
  T* sTm = sK;
  T* sTu = sQ;
  {
    T* TmT = ws_ptr<T>(p, p.off.TmT) + slot * 64 * 64;
    // one 4x4 block of Tm per thread: four-element row reads, the transpose taken in registers
    const int r0 = (tid >> 4) * 4, c0 = (tid & 15) * 4;
    floatx4 t[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = load4(sT + (r0 + i) * LNX_LDA + c0);
    const floatx4 bu = load4(sBeta + c0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      store4(sTm + (r0 + i) * LDC + c0, t[i]);
      store4(sTu + (r0 + i) * LDC + c0, t[i] * bu);
      if (p.save) store4(TmT + (c0 + i) * 64 + r0, floatx4{t[0][i], t[1][i], t[2][i], t[3][i]});
    }
  }
  // ---- phase D: W = Tm (beta e^G K), U = Tu V, one 64-column slab at a time ----
  T* sIn = reinterpret_cast<T*>(sG);    // staged slab [token][col]
  T* sOut = reinterpret_cast<T*>(sA);   // result slab on its way to the workspace
  const int wi = wave >> 1, wj = wave & 1;
  const int nslab = NH + p.dv / 64;
  typedef TileRegs<T, 64, 64> Slab;
  constexpr int VN = Slab::N;
  Slab rIn;
  floatx4 rGs[Slab::IT][VN / 4];  // K slabs: the gate values of exactly the elements this thread holds
  auto fetch_slab = [&](int s_) {
    if (s_ < NH) {
      rIn.load(kg + 64 * s_, tsk, len, tid);
#pragma unroll
      for (int it = 0; it < Slab::IT; ++it) {
        const int idx = tid + 256 * it, r = idx / Slab::VPR, c = (idx - r * Slab::VPR) * VN;
#pragma unroll
        for (int j = 0; j < VN / 4; ++j) rGs[it][j] = load4(Gg + r * DK + 64 * s_ + c + 4 * j);
      }
    } else {
      if (64 * (s_ - NH) < p.vcols) rIn.load(vg + 64 * (s_ - NH), tsv, len, tid);
      else rIn.zero();  // value columns that v does not hold
    }
  };
  __syncthreads();  // G is read back from the workspace by other threads than wrote it: global memory must be ordered too
  fetch_slab(0);
#pragma unroll 1
  for (int s_ = 0; s_ < nslab; ++s_) {
    const bool is_k = s_ < NH;
    lds_barrier();  // the previous slab's tiles (first pass: the inverse, the gate tile) are dead
    if (is_k) {     // K slab scaled by beta_t e^{G_t[c]} on its way into LDS
#pragma unroll
      for (int it = 0; it < Slab::IT; ++it) {
        const int idx = tid + 256 * it, r = idx / Slab::VPR, c = (idx - r * Slab::VPR) * VN;
        typename Vec16<T>::V x = rIn.x[it];
#pragma unroll
        for (int e = 0; e < VN; ++e) x[e] = from_f32<T>(to_f32(x[e]) * sBeta[r] * __expf(rGs[it][e / 4][e % 4]));
        *reinterpret_cast<typename Vec16<T>::V*>(sIn + r * LDC + c) = x;
      }
    } else {
      rIn.store(sIn, LDC, tid);
    }
    lds_barrier();
    if (s_ + 1 < nslab) fetch_slab(s_ + 1);
    floatx16 o[1][1];
    frag_zero(o);
    mma_x<T, 1, 1, false, true>(o, (is_k ? sTm : sTu) + 32 * wi * LDC, LDC, sIn + 32 * wj, LDC, 64, lane);
    frag_store<T, 1, 1>(o, sOut + 32 * wi * LDC + 32 * wj, LDC, lane);
    lds_barrier();
    if (is_k)
      unstage_tile<T, 64, 64>(ws_ptr<T>(p, p.off.W) + slot * 64 * DK + 64 * s_, DK, sOut, LDC, 64, tid);
    else
      unstage_tile<T, 64, 64>(ws_ptr<T>(p, p.off.U) + slot * 64 * p.dv + 64 * (s_ - NH), p.dv, sOut, LDC, 64, tid);
  }
  }
}

// ---------------------------------------------------------------------------------------
// chunk_scan: the sequential pass over the chunks of one (state, 64-column slab of dv).
// Per chunk: D = U - W S, the state update, and -- for 2-byte inputs, where the tiles fit LDS --
// the outputs o = scale e^G (Q S) + P D of the same slab, so the state and D are not read back
// by a separate output kernel.
//
// The pass is one dependent chain per workgroup and only (states x slabs) workgroups exist, so
// nothing hides memory instructions behind another workgroup.  The 512 threads therefore split
// into two roles, one wave of each per SIMD: waves 0-3 do the matrix work on the tiles in LDS,
// waves 4-7 ("movers") only move data -- global loads two chunks ahead into registers, tile
// writes into LDS as soon as the previous chunk's reader is done with a tile, and the
// LDS -> global copies of the state, D and the outputs.  Three barriers per chunk:
//   B1  tiles of chunk n and the entering state S_n (transposed, LDS) are complete
//         compute: D                         movers: loads of chunk n+2, S_n -> workspace
//   B2  D is in LDS (plain in place of U, decay-scaled and transposed for the update)
//         compute: outputs, state update     movers: W of chunk n+1 -> LDS, D -> workspace
//   B3  all reads of chunk n's tiles are done
//         compute: S_{n+1} -> LDS            movers: remaining tiles of chunk n+1 -> LDS, outputs -> global
// ---------------------------------------------------------------------------------------
// BV = columns of dv per workgroup: 64, or 32 (dk = 128, 2-byte inputs) when 64-column slabs would
// leave more than half of the CUs without a workgroup.
template <typename T, int DK, int BVW = 64> struct ScanSmem {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int LDK = DK + PAD;
  static constexpr int LDC = LNX_C + PAD;
  static constexpr int BV = BVW;
  static constexpr bool FUSE_OUT = sizeof(T) == 2;
  static constexpr int LDO = BV + 8;  // staging tile of 2-byte outputs (fp32 outputs go out as 128-byte row segments directly)
  // 4-byte inputs with dk = 256: W (read for D) and K (read for the state update) of a chunk take turns in one tile
  static constexpr bool SHARE = sizeof(T) == 4 && DK > 128;
  // 2-byte inputs with dk = 256 and 64-column slabs: W (read for D) and Q (read for the outputs) take turns in one tile
  static constexpr bool SHAREQ = sizeof(T) == 2 && DK > 128 && BV == 64;
  static constexpr int kW = 64 * LDK, kKT = SHARE ? 0 : 64 * LDK, kU = 64 * (BV + PAD), kST = BV * LDK, kDT = BV * LDC;
  static constexpr int kQ = (FUSE_OUT && !SHAREQ) ? 64 * LDK : 0, kP = FUSE_OUT ? 64 * LDC : 0;
  static constexpr int kG = DK > 128 ? DK : 128;  // gate values: 64 tokens (scalar gate) or dk channels (vector gate)
  // 32-column slabs of 2-byte inputs with dk = 128: every input tile twice, so that the movers write chunk n + 1
  // while chunk n is being read
  static constexpr bool DB = sizeof(T) == 2 && DK == 128 && BV == 32;
  static constexpr int NB = DB ? 2 : 1;
  // staging tile of the outputs: bf16 [64][LDO]; double-buffered form: also fp32 [64][LDOF], so that every global store
  // of the kernel is a mover's
  static constexpr int LDOF = BV + 4;
  static constexpr size_t o_bytes = !FUSE_OUT ? 0 : DB ? sizeof(float) * 64 * LDOF : sizeof(bf16_t) * 64 * LDO;
  static constexpr size_t bytes = sizeof(T) * (NB * (kW + kKT + kU + kQ + kP) + kST + kDT) + o_bytes + sizeof(float) * NB * (kG + 4);
};

template <typename T, int DK, int GATE, int BVW = 64>
__global__ __launch_bounds__(512) void chunk_scan_kernel(FwdParams p) {
  typedef ScanSmem<T, DK, BVW> L;
  constexpr int LDK = L::LDK, LDC = L::LDC, BV = L::BV, LDU = BV + L::PAD, LDO = L::LDO;
  constexpr bool FUSE = L::FUSE_OUT;
  // state tiles: (DK/32) x (BV/32); DK>=128: wave w owns the RT = DK/128 row tiles from RT * w on and all column
  // tiles, DK=64: wave w owns row tile (w & 1) and column tile (w >> 1)
  constexpr int CT = BV / 32;
  constexpr int RT = (DK >= 128) ? DK / 128 : 1;
  constexpr int NT = (DK >= 128) ? CT : 1;
  static_assert(BV == 64 || (BV == 32 && DK >= 128), "32-column slabs: the wave's state tile must be a full row tile");
  extern __shared__ __align__(16) char smem[];
  constexpr int NB = L::NB;  // buffers per input tile (the second of a pair follows the first)
  T* sW = reinterpret_cast<T*>(smem);
  T* sK = L::SHARE ? sW : sW + NB * L::kW;  // K rows [token][dk] (vector gate: K * e^{G_last - G})
  T* sU = sW + NB * (L::kW + L::kKT);       // U rows [token][v], replaced by D
  T* sST = sU + NB * L::kU;
  T* sDT = sST + L::kST;
  T* sQ = L::SHAREQ ? sW : sDT + L::kDT;  // fused output only: Q rows (vector gate: scale Q e^G), P, output staging
  T* sP = sDT + L::kDT + NB * L::kQ;
  bf16_t* sO = reinterpret_cast<bf16_t*>(sP + NB * L::kP);
  float* sOf = reinterpret_cast<float*>(sO);  // double-buffered form with fp32 outputs
  float* sG = reinterpret_cast<float*>(reinterpret_cast<char*>(sO) + L::o_bytes);  // [NB][kG + 4]: gate values, then first token and
                                                                     // length of the chunk whose tiles are in the buffer
  int* sMeta = reinterpret_cast<int*>(sG + L::kG);
  constexpr int kGM = L::kG + 4;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  int sidx, row, seq;  // state index, (batch, head) row, sequence
  // 1-D grid: the slabs of one (state, head) row get workgroup ids 8 apart, i.e. the same XCD and the same
  // dispatch wave, so the W / K / Q tiles they both load come from HBM once
  int64_t chain;
  int slab;
  if (!xcd_slot_part((int64_t)(p.geom.tab ? p.geom.nseq : p.geom.rows / p.geom.H) * p.geom.H, p.dv / BV, chain, slab)) return;
  scan_state(p.geom, (int)chain, sidx, row, seq);
  const int v0 = slab * BV;
  int c0, c1;
  seq_chunks(p.geom, seq, c0, c1);
  const SeqSpan span = seq_span(p.geom, seq, c0);

  if constexpr (L::SHARE) {
    if (wave >= 4) {
      // ---------------- movers, one tile shared by W and K ----------------
      // A fourth barrier (B2') separates the tile's two uses; whichever of W(n+1) and K(n) is not in LDS waits in
      // registers.  B1: W, U of chunk n in LDS -> loads of W, U of chunk n+1;  B2: K of chunk n -> LDS, D -> workspace;
      // B2': loads of K of chunk n+1;  B3: W, U of chunk n+1 -> LDS.
      const int mt = tid - 256;
      TileRegs<T, 64, DK> rW, rK;
      TileRegs<T, 64, BV> rU;
      float rG = 0.f;
      auto fetch_w = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        rW.load(ws_ptr<T>(p, p.off.W) + slot * 64 * DK, DK, 64, mt);
        rU.load(ws_ptr<T>(p, p.off.U) + slot * 64 * p.dv + v0, p.dv, 64, mt);
        if (GATE == LNX_GATE_SCALAR && mt < 64) rG = ws_ptr<float>(p, p.off.G)[slot * 64 + mt];
        if (GATE == LNX_GATE_VECTOR && mt < DK) rG = ws_ptr<float>(p, p.off.G)[(slot * 64 + 63) * DK + mt];
      };
      auto fetch_k = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        int tok0, len;
        chunk_span(span, n, tok0, len);
        if (GATE == LNX_GATE_VECTOR) rK.load(ws_ptr<T>(p, p.off.Kr) + slot * 64 * DK, DK, 64, mt);
        else rK.load(reinterpret_cast<const T*>(p.k) + tok_index(p.geom, row, tok0) * DK, (int64_t)p.geom.ts * DK, len, mt);
      };
      auto commit_w = [&]() {
        rW.store(sW, LDK, mt);
        rU.store(sU, LDU, mt);
        if (mt < L::kG) sG[mt] = rG;
      };
      if (c0 < c1) {
        fetch_w(c0);
        fetch_k(c0);
        commit_w();
      }
      lds_barrier();  // B1 of the first chunk
      for (int n = c0; n < c1; ++n) {
        const int64_t slot = (int64_t)row * N + n;
        if (n + 1 < c1) fetch_w(n + 1);
        lds_barrier();  // B2
        rK.store(sK, LDK, mt);
        if (p.save) unstage_tile<T, 64, BV, true>(ws_ptr<T>(p, p.off.D) + slot * 64 * p.dv + v0, p.dv, sU, LDU, 64, mt);
        lds_barrier();  // B2'
        if (n + 1 < c1) fetch_k(n + 1);
        lds_barrier();  // B3
        if (n + 1 < c1) commit_w();
        lds_barrier();  // B1 of the next chunk
      }
      return;
    }
  } else if constexpr (L::SHAREQ) {
    if (wave >= 4) {
      // ---------------- movers, one tile shared by W and Q ----------------
      // B1: W, K, U, P of chunk n in LDS -> loads of those of chunk n+1;  B2: Q of chunk n -> the W tile, D ->
      // workspace;  B2': loads of Q of chunk n+1;  B3: outputs -> global, tiles of chunk n+1 -> LDS.
      const int mt = tid - 256;
      TileRegs<T, 64, DK> rW, rK, rQ;
      TileRegs<T, 64, BV> rU;
      TileRegs<T, 64, 64> rP;
      float rG = 0.f;
      int ftok0 = 0, flen = 0;  // span of the chunk last fetched
      const int64_t tsk = (int64_t)p.geom.ts * DK;
      auto fetch_main = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        chunk_span(span, n, ftok0, flen);
        rW.load(ws_ptr<T>(p, p.off.W) + slot * 64 * DK, DK, 64, mt);
        if (GATE == LNX_GATE_VECTOR) rK.load(ws_ptr<T>(p, p.off.Kr) + slot * 64 * DK, DK, 64, mt);
        else rK.load(reinterpret_cast<const T*>(p.k) + tok_index(p.geom, row, ftok0) * DK, tsk, flen, mt);
        rU.load(ws_ptr<T>(p, p.off.U) + slot * 64 * p.dv + v0, p.dv, 64, mt);
        rP.load(ws_ptr<T>(p, p.off.P) + slot * 64 * 64, 64, 64, mt);
        if (GATE == LNX_GATE_SCALAR && mt < 64) rG = ws_ptr<float>(p, p.off.G)[slot * 64 + mt];
        if (GATE == LNX_GATE_VECTOR && mt < DK) rG = ws_ptr<float>(p, p.off.G)[(slot * 64 + 63) * DK + mt];
      };
      auto fetch_q = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        int tok0, len;
        chunk_span(span, n, tok0, len);
        if (GATE == LNX_GATE_VECTOR) rQ.load(ws_ptr<T>(p, p.off.Qg) + slot * 64 * DK, DK, 64, mt);
        else rQ.load(reinterpret_cast<const T*>(p.q) + tok_index(p.geom, row, tok0) * DK, tsk, len, mt);
      };
      auto commit_main = [&]() {
        rW.store(sW, LDK, mt);
        rK.store(sK, LDK, mt);
        rU.store(sU, LDU, mt);
        rP.store(sP, LDC, mt);
        if (mt < L::kG) sG[mt] = rG;
        if (mt == 0) {
          sMeta[0] = ftok0;
          sMeta[1] = flen;
        }
      };
      if (c0 < c1) {
        fetch_main(c0);
        fetch_q(c0);
        commit_main();
      }
      lds_barrier();  // B1 of the first chunk
      for (int n = c0; n < c1; ++n) {
        const int64_t slot = (int64_t)row * N + n;
        const int tok0 = ftok0, len = flen;
        if (n + 1 < c1) fetch_main(n + 1);
        lds_barrier();  // B2
        rQ.store(sQ, LDK, mt);
        if (p.save) unstage_tile<T, 64, BV, true>(ws_ptr<T>(p, p.off.D) + slot * 64 * p.dv + v0, p.dv, sU, LDU, 64, mt);
        lds_barrier();  // B2'
        if (n + 1 < c1) fetch_q(n + 1);
        lds_barrier();  // B3
        if (p.o_dtype == LNX_BF16 && p.o)
          unstage_tile<bf16_t, 64, BV>(reinterpret_cast<bf16_t*>(p.o) + tok_index(p.geom, row, tok0) * p.dv + v0,
                                       (int64_t)p.geom.ts * p.dv, sO, LDO, len, mt);
        if (n + 1 < c1) commit_main();
        lds_barrier();  // B1 of the next chunk
      }
      return;
    }
  } else if (wave >= 4) {
    // ---------------- movers ----------------
    const int mt = tid - 256;
    struct Tiles {
      TileRegs<T, 64, DK> W, K;
      TileRegs<T, 64, BV> U;
      TileRegs<T, 64, FUSE ? DK : 8> Q;
      TileRegs<T, 64, FUSE ? 64 : 8> P;
      float G;
      int tok0, len;
    };
    // register sets: 2-byte inputs are fetched two chunks ahead (two sets used alternately); 4-byte
    // inputs and dk = 256 one chunk ahead (a second set would not fit the register file)
    constexpr int AHEAD = (sizeof(T) == 2 && DK <= 128) ? 2 : 1;
    Tiles ta, tb;
    ta.G = tb.G = 0.f;
    ta.tok0 = ta.len = tb.tok0 = tb.len = 0;
    // part 0: W, 1: K, 2: Q, 3: the rest; < 0: everything
    auto fetch = [&](Tiles& R, int n, int part = -1) {
      const int64_t slot = (int64_t)row * N + n;
      chunk_span(span, n, R.tok0, R.len);
      const int64_t tbase = tok_index(p.geom, row, R.tok0);
      const int64_t tsk = (int64_t)p.geom.ts * DK;
      if (part < 0 || part == 0) R.W.load(ws_ptr<T>(p, p.off.W) + slot * 64 * DK, DK, 64, mt);
      if (part < 0 || part == 1) {
        if (GATE == LNX_GATE_VECTOR) R.K.load(ws_ptr<T>(p, p.off.Kr) + slot * 64 * DK, DK, 64, mt);
        else R.K.load(reinterpret_cast<const T*>(p.k) + tbase * DK, tsk, R.len, mt);
      }
      if (FUSE && (part < 0 || part == 2)) {
        if (GATE == LNX_GATE_VECTOR) R.Q.load(ws_ptr<T>(p, p.off.Qg) + slot * 64 * DK, DK, 64, mt);
        else R.Q.load(reinterpret_cast<const T*>(p.q) + tbase * DK, tsk, R.len, mt);
      }
      if (part >= 0 && part < 3) return;
      R.U.load(ws_ptr<T>(p, p.off.U) + slot * 64 * p.dv + v0, p.dv, 64, mt);
      if (FUSE) R.P.load(ws_ptr<T>(p, p.off.P) + slot * 64 * 64, 64, 64, mt);
      // every thread loads (clamped index): a load behind a branch cannot be counted
      if (GATE == LNX_GATE_SCALAR) R.G = ws_ptr<float>(p, p.off.G)[slot * 64 + (mt & 63)];
      if (GATE == LNX_GATE_VECTOR) R.G = ws_ptr<float>(p, p.off.G)[(slot * 64 + 63) * DK + min(mt, DK - 1)];  // G_last[c]
    };
    auto commit_rest = [&](const Tiles& R, int pb, int part = -1) {  // parts as in fetch (W is written by the caller)
      if (part < 0 || part == 1) R.K.store(sK + pb * L::kKT, LDK, mt);
      if (FUSE && (part < 0 || part == 2)) R.Q.store(sQ + pb * L::kQ, LDK, mt);
      if (part >= 0 && part < 3) return;
      R.U.store(sU + pb * L::kU, LDU, mt);
      if (FUSE) R.P.store(sP + pb * L::kP, LDC, mt);
      if (mt < L::kG) sG[pb * kGM + mt] = R.G;
      if (mt == 0) {
        sMeta[pb * kGM] = R.tok0;
        sMeta[pb * kGM + 1] = R.len;
      }
    };
    // cur: chunk n (in LDS already), nxt: chunk n + 1.  `steady` (a std::bool_constant) says that chunks n + 1 and
    // n + AHEAD exist, so the fetch and the commits are unconditional: behind a conditional fetch the compiler
    // cannot count how many younger loads are in flight and waits for all of them (the fetch just issued included)
    // before the first tile store.
    auto step = [&](Tiles& cur, const Tiles& nxt, int n, auto steady) {
      constexpr bool STEADY = decltype(steady)::value;
      const int64_t slot = (int64_t)row * N + n;
      const int tok0 = cur.tok0, len = cur.len;
      if constexpr (L::DB) {
        // Chunk n + 1 goes to the buffers chunk n - 1 was read from, so no tile write waits for a reader, and every
        // global store of the kernel is issued here: stores issued by the compute waves queued behind the movers'
        // loads and held the chain up.  Loads and the next chunk's tile writes in the first two phases, the chunk's
        // state and D in the second, the outputs in the third.
        const int pb = (n - c0) & 1;
        if constexpr (STEADY) {
          // chunk n's registers are free again and take chunk n + 2; the tile writes of chunk n + 1 sit between the
          // loads, a tile at a time: a wave whose load waits for a slot in the memory path issues nothing else, and
          // the writes go out while the loads before them drain.  W and K here, Q and the rest behind the stores of
          // the second phase (all in this phase: 0.322 ms at B4 H16 T8192; split: 0.310)
#pragma unroll
          for (int part = 0; part < 2; ++part) {
            fetch(cur, n + AHEAD, part);
            if (part == 0) nxt.W.store(sW + (pb ^ 1) * L::kW, LDK, mt);
            else commit_rest(nxt, pb ^ 1, part);
            __builtin_amdgcn_sched_barrier(0);
          }
        } else {
          if (n + AHEAD < c1) fetch(cur, n + AHEAD);
          if (n + 1 < c1) {
            nxt.W.store(sW + (pb ^ 1) * L::kW, LDK, mt);
            commit_rest(nxt, pb ^ 1);
          }
        }
        lds_barrier();  // B2
        if (p.save) {
          unstage_tile<T, BV, DK, true>(ws_ptr<T>(p, p.off.SnT) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sST, LDK, BV, mt);
          unstage_tile<T, 64, BV, true>(ws_ptr<T>(p, p.off.D) + slot * 64 * p.dv + v0, p.dv, sU + pb * L::kU, LDU, 64, mt);
        }
        if constexpr (STEADY) {
#pragma unroll
          for (int part = 2; part < 4; ++part) {
            fetch(cur, n + AHEAD, part);
            commit_rest(nxt, pb ^ 1, part);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        lds_barrier();  // B3
        if (p.o) {
          if (p.o_dtype == LNX_BF16)
            unstage_tile_checked<bf16_t, 64, BV>(reinterpret_cast<bf16_t*>(p.o) + tok_index(p.geom, row, tok0) * p.dv + v0,
                                                 (int64_t)p.geom.ts * p.dv, sO, LDO, len, mt);
          else
            unstage_tile_checked<float, 64, BV>(reinterpret_cast<float*>(p.o) + tok_index(p.geom, row, tok0) * p.dv + v0,
                                                (int64_t)p.geom.ts * p.dv, sOf, L::LDOF, len, mt);
        }
        lds_barrier();  // B1 of the next chunk
        return;
      }
      if (STEADY || n + AHEAD < c1) fetch(cur, n + AHEAD);  // chunk n's registers are free again
      lds_barrier();  // B2
      if (STEADY || n + 1 < c1) nxt.W.store(sW, LDK, mt);
      if (p.save) unstage_tile<T, 64, BV, true>(ws_ptr<T>(p, p.off.D) + slot * 64 * p.dv + v0, p.dv, sU, LDU, 64, mt);
      lds_barrier();  // B3
      // the output rows first, the tile commits behind them
      if (FUSE && p.o_dtype == LNX_BF16 && p.o)
        unstage_tile<bf16_t, 64, BV>(reinterpret_cast<bf16_t*>(p.o) + tok_index(p.geom, row, tok0) * p.dv + v0,
                                     (int64_t)p.geom.ts * p.dv, sO, LDO, len, mt);
      if (STEADY || n + 1 < c1) commit_rest(nxt, 0);
      lds_barrier();  // B1 of the next chunk
    };
    if (c0 < c1) {
      fetch(ta, c0);
      ta.W.store(sW, LDK, mt);
      commit_rest(ta, 0);
    }
    if (AHEAD == 2 && c0 + 1 < c1) fetch(tb, c0 + 1);
    lds_barrier();  // B1 of the first chunk
    if (AHEAD == 2) {
      // chunk c0 is in LDS, so set a is free: it takes chunk c0 + 2 in the first step
      int n = c0;
      for (; n + 3 < c1; n += 2) {  // chunks n + 2 and n + 3 exist
        step(ta, tb, n, std::true_type{});
        step(tb, ta, n + 1, std::true_type{});
      }
      for (; n < c1; n += 2) {
        step(ta, tb, n, std::false_type{});
        if (n + 1 < c1) step(tb, ta, n + 1, std::false_type{});
      }
    } else {
      for (int n = c0; n < c1; ++n) step(ta, ta, n, std::false_type{});
    }
    return;
  }

  // ---------------- compute waves ----------------
  const int srow = (DK >= 128) ? 32 * RT * wave : 32 * (wave & 1);
  const int scol = (DK >= 128) ? 0 : 32 * (wave >> 1);
  // this wave's 32x32 tile of the [64 x BV] products (a 32-column slab has two tiles: waves 0 and 1)
  const int wi = (CT == 2) ? (wave >> 1) : wave, wj = (CT == 2) ? (wave & 1) : 0;
  const bool has_tile = (CT == 2) || wave < 2;

  floatx16 S[RT][NT];
  frag_zero(S);
  if (p.s0) {
    const float* s0 = p.s0 + (int64_t)sidx * DK * p.dv + v0;
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          S[i][j][e] = s0[(int64_t)(srow + 32 * i + frag_row(e, lane)) * p.dv + scol + 32 * j + frag_col(lane)];
  }
  // entering state -> LDS, transposed [dv][dk] (B operand of W S and Q S; the movers copy it to the workspace)
  if (c0 < c1) frag_store_t<T, RT, NT>(S, sST + scol * LDK + srow, LDK, lane);
  lds_barrier();  // B1 of the first chunk
  for (int n = c0; n < c1; ++n) {
    const int pb = L::DB ? (n - c0) & 1 : 0;  // buffer of this chunk's tiles
    const T* cW = sW + pb * L::kW;
    const T* cK = sK + pb * L::kKT;
    T* cU = sU + pb * L::kU;
    const T* cQ = sQ + pb * L::kQ;
    const T* cP = sP + pb * L::kP;
    const float* cG = sG + pb * kGM;
    const int* cMeta = sMeta + pb * kGM;
    // D = U - W S  (one 32x32 tile per wave)
    const float gl = (GATE == LNX_GATE_SCALAR) ? cG[63] : 0.f;
    if (has_tile) {
      floatx16 d[1][1];
      frag_zero(d);
      mma_nt<T, 1, 1>(d, cW + 32 * wi * LDK, LDK, sST + 32 * wj * LDK, LDK, DK, lane);
      // D replaces U in place (all reads first: interleaved with the writes they would be serialised)
      float u[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) u[e] = to_f32(cU[(32 * wi + frag_row(e, lane)) * LDU + 32 * wj + frag_col(lane)]);
#pragma unroll
      for (int e = 0; e < 16; ++e) d[0][0][e] = u[e] - d[0][0][e];
#pragma unroll
      for (int e = 0; e < 16; ++e)
        cU[(32 * wi + frag_row(e, lane)) * LDU + 32 * wj + frag_col(lane)] = from_f32<T>(d[0][0][e]);
      if (GATE == LNX_GATE_SCALAR) {
#pragma unroll
        for (int e = 0; e < 16; ++e) d[0][0][e] *= __expf(fminf(gl - cG[32 * wi + frag_row(e, lane)], 0.f));
      }
      frag_store_t<T, 1, 1>(d, sDT + 32 * wj * LDC + 32 * wi, LDC, lane);
    }
    // S_n -> workspace (the movers are busy issuing loads in this phase; double-buffered form: they do it after B2)
    if (p.save && !L::DB)
      unstage_tile<T, BV, DK, true>(ws_ptr<T>(p, p.off.SnT) + ((int64_t)row * N + n) * p.dv * DK + (int64_t)v0 * DK, DK, sST, LDK, BV, tid);
    lds_barrier();  // B2

    auto outputs = [&]() {
      if (FUSE && has_tile) {
        // o = scale e^G (Q S) + P D for this slab
        floatx16 o[1][1];
        frag_zero(o);
        mma_nt<T, 1, 1>(o, cQ + 32 * wi * LDK, LDK, sST + 32 * wj * LDK, LDK, DK, lane);
        if (GATE != LNX_GATE_VECTOR) {
#pragma unroll
          for (int e = 0; e < 16; ++e)
            o[0][0][e] *= (GATE == LNX_GATE_NONE) ? p.scale : p.scale * __expf(cG[32 * wi + frag_row(e, lane)]);
        }
        mma_x<T, 1, 1, false, true>(o, cP + 32 * wi * LDC, LDC, cU + 32 * wj, LDU, 64, lane);
        if (p.o_dtype == LNX_BF16) {
          frag_store<bf16_t, 1, 1>(o, sO + 32 * wi * LDO + 32 * wj, LDO, lane);  // the movers write it out
        } else if (L::DB) {
          frag_store<float, 1, 1>(o, sOf + 32 * wi * L::LDOF + 32 * wj, L::LDOF, lane);
        } else if (p.o) {
          const int tok0 = cMeta[0], len = cMeta[1];
          frag_store<float, 1, 1>(o, reinterpret_cast<float*>(p.o) + (tok_index(p.geom, row, tok0) + (int64_t)32 * wi * p.geom.ts) * p.dv + v0 + 32 * wj,
                                  (int64_t)p.geom.ts * p.dv, lane, len - 32 * wi);
        }
      }
    };
    auto update = [&]() {
      // S <- e^{G_last} S + K^T (D e^{G_last - G})
      if (GATE == LNX_GATE_SCALAR) {
        const float dec = __expf(gl);
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) S[i][j][e] *= dec;
      }
      if (GATE == LNX_GATE_VECTOR) {  // per state row (key channel)
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) S[i][j][e] *= __expf(cG[srow + 32 * i + frag_row(e, lane)]);
      }
      mma_x<T, RT, NT, true, false>(S, cK + srow, LDK, sDT + scol * LDC, LDC, 64, lane);
    };
    if (L::SHAREQ) {
      update();
      lds_barrier();  // B2': Q has replaced W in the shared tile
      outputs();
    } else {
      outputs();
      if (L::SHARE) lds_barrier();  // B2': K has replaced W in the shared tile
      update();
    }
    lds_barrier();  // B3
    if (n + 1 < c1) frag_store_t<T, RT, NT>(S, sST + scol * LDK + srow, LDK, lane);
    lds_barrier();  // B1 of the next chunk
  }

  float* out = p.sT_out + (int64_t)sidx * DK * p.dv + v0;
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        out[(int64_t)(srow + 32 * i + frag_row(e, lane)) * p.dv + scol + 32 * j + frag_col(lane)] = S[i][j][e];
}

// ---------------------------------------------------------------------------------------
// chunk_output
// ---------------------------------------------------------------------------------------
template <typename T, int DK> struct OutSmem {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int LDK = DK + PAD;
  static constexpr int LDC = LNX_C + PAD;
  static constexpr int BV = (sizeof(T) == 4 && DK > 128) ? 32 : 64;  // 4-byte inputs with dk = 256: LDS capacity
  static constexpr size_t bytes = sizeof(T) * (64 * LDK + BV * LDK + 64 * LDC + 64 * LDC) + sizeof(float) * 64;  // Q, S^T, P, D
};

template <typename T, int DK, int GATE>
__global__ __launch_bounds__(256) void chunk_output_kernel(FwdParams p) {
  typedef OutSmem<T, DK> L;
  constexpr int LDK = L::LDK, LDC = L::LDC, BV = L::BV;
  extern __shared__ __align__(16) char smem[];
  T* sQ = reinterpret_cast<T*>(smem);
  T* sST = sQ + 64 * LDK;
  T* sP = sST + BV * LDK;
  T* sDT = sP + 64 * LDC;
  float* sG = reinterpret_cast<float*>(sDT + 64 * LDC);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  // one workgroup = one chunk and out_spw consecutive value slabs: Q and P are staged once for all of them
  const int nslab = p.dv / BV, nparts = (nslab + p.out_spw - 1) / p.out_spw;
  int64_t slot;
  int part;
  if (!xcd_slot_part((int64_t)p.geom.rows * N, nparts, slot, part)) return;
  const int row = (int)(slot / N), n = (int)(slot % N);
  const int s0 = part * p.out_spw, s1 = min(nslab, s0 + p.out_spw);
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  if (len <= 0) return;
  const int64_t tbase = tok_index(p.geom, row, tok0);
  const int64_t tsk = (int64_t)p.geom.ts * DK, tsv = (int64_t)p.geom.ts * p.dv;

  TileRegs<T, BV, DK> rS;   // S_n^T slab [v][dk]
  TileRegs<T, 64, BV> rD;   // D slab [token][v]
  auto fetch = [&](int s_) {
    const int v0 = s_ * BV;
    rS.load(ws_ptr<T>(p, p.off.SnT) + slot * p.dv * DK + (int64_t)v0 * DK, DK, BV, tid);
    rD.load(ws_ptr<T>(p, p.off.D) + slot * 64 * p.dv + v0, p.dv, 64, tid);
  };
  fetch(s0);
  if (GATE == LNX_GATE_VECTOR) {
    constexpr int VN = Vec16<T>::N;
    const T* qg = reinterpret_cast<const T*>(p.q) + tbase * DK;
    const float* Gg = ws_ptr<float>(p, p.off.G) + slot * 64 * DK;
    for (int idx = tid; idx < 64 * DK / VN; idx += 256) {
      const int r = idx / (DK / VN), c = (idx % (DK / VN)) * VN;
      typename Vec16<T>::V x = vec_zero<T>();
      if (r < len) {
        x = *reinterpret_cast<const typename Vec16<T>::V*>(qg + (int64_t)r * tsk + c);
#pragma unroll
        for (int e = 0; e < VN; ++e) x[e] = from_f32<T>(to_f32(x[e]) * p.scale * __expf(Gg[r * DK + c + e]));
      }
      *reinterpret_cast<typename Vec16<T>::V*>(sQ + r * LDK + c) = x;
    }
  } else {
    stage_tile<T, 64, DK>(sQ, LDK, reinterpret_cast<const T*>(p.q) + tbase * DK, tsk, len, tid);
  }
  stage_tile<T, 64, 64>(sP, LDC, ws_ptr<T>(p, p.off.P) + slot * 64 * 64, 64, 64, tid);
  if (tid < 64) sG[tid] = (GATE == LNX_GATE_SCALAR) ? ws_ptr<float>(p, p.off.G)[slot * 64 + tid] : 0.f;

  // one 32x32 tile of the [64 x BV] outputs per wave (a 32-column slab has two: waves 0 and 1)
  const int wi = (BV == 64) ? (wave >> 1) : wave, wj = (BV == 64) ? (wave & 1) : 0;
  const bool has_tile = BV == 64 || wave < 2;
#pragma unroll 1
  for (int s_ = s0; s_ < s1; ++s_) {
    lds_barrier();  // the previous slab's tiles have been read
    rS.store(sST, LDK, tid);
    rD.store(sDT, LDC, tid);
    lds_barrier();
    if (s_ + 1 < s1) fetch(s_ + 1);
    if (has_tile) {
      floatx16 acc[1][1];
      frag_zero(acc);
      mma_nt<T, 1, 1>(acc, sQ + 32 * wi * LDK, LDK, sST + 32 * wj * LDK, LDK, DK, lane);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float gm = (GATE == LNX_GATE_VECTOR) ? 1.f : p.scale * __expf(sG[32 * wi + frag_row(e, lane)]);
        acc[0][0][e] *= gm;
      }
      mma_x<T, 1, 1, false, true>(acc, sP + 32 * wi * LDC, LDC, sDT + 32 * wj, LDC, 64, lane);
      const int64_t obase = (tbase + (int64_t)32 * wi * p.geom.ts) * p.dv + s_ * BV + 32 * wj;
      if (p.o_dtype == LNX_BF16)
        frag_store<bf16_t, 1, 1>(acc, reinterpret_cast<bf16_t*>(p.o) + obase, tsv, lane, len - 32 * wi);
      else
        frag_store<float, 1, 1>(acc, reinterpret_cast<float*>(p.o) + obase, tsv, lane, len - 32 * wi);
    }
  }
}

// state-only path for T == 0: final = initial (or zeros)
__global__ void copy_state_kernel(const float* src, float* dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src ? src[i] : 0.f;
}

// packed batches: slot table [N][2] = (token0, len), then seq_chunk0[nseq + 1], then the sequence
// indices by decreasing length (ties by index).  One workgroup: the first chunk slot of every sequence by a serial
// prefix over the (few) sequences, then all threads fill the slots, each finding its sequence by bisection.
__global__ void build_table_kernel(const int32_t* cu, int nseq, int N, int T, int32_t* tab) {
  int32_t* chunk0 = tab + 2 * N;
  int32_t* order = chunk0 + nseq + 1;
  // a malformed table (entries outside [0, T] or decreasing) must not send any kernel outside the tensors
  auto first = [&](int s) { return seq_first(cu, s, T); };
  auto length = [&](int s) { return seq_end(cu, s, T) - seq_first(cu, s, T); };
  for (int s = threadIdx.x; s < nseq; s += blockDim.x) {
    const int ls = length(s);
    int rank = 0;
    for (int u = 0; u < nseq; ++u) {
      const int lu = length(u);
      rank += (lu > ls) || (lu == ls && u < s);
    }
    order[rank] = s;
  }
  if (threadIdx.x == 0) {
    int c = 0;
    for (int s = 0; s < nseq; ++s) {
      chunk0[s] = min(c, N);
      c += (length(s) + LNX_C - 1) / LNX_C;
    }
    chunk0[nseq] = min(c, N);
  }
  __threadfence_block();
  __syncthreads();  // chunk0 is read back from global memory by the other threads
  const int total = chunk0[nseq];
  for (int c = threadIdx.x; c < N; c += blockDim.x) {
    int t0 = 0, len = 0;
    if (c < total) {
      int lo = 0, hi = nseq - 1;  // last sequence whose first slot is <= c (empty sequences share a first slot)
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (chunk0[mid] <= c) lo = mid; else hi = mid - 1;
      }
      // skip forward over empty sequences that start at the same slot: the slot belongs to the one with tokens
      while (lo + 1 < nseq && chunk0[lo + 1] <= c) ++lo;
      t0 = first(lo) + (c - chunk0[lo]) * LNX_C;
      len = max(0, min(LNX_C, seq_end(cu, lo, T) - t0));
    }
    tab[2 * c] = t0;
    tab[2 * c + 1] = len;
  }
}

template <typename T, int DK, int GATE> struct PrepSelect {
  static constexpr size_t bytes = Prep2Cfg<T, DK>::bytes;
  static auto kernel(bool) { return chunk_prepare2_kernel<T, DK, GATE>; }
};
template <typename T, int DK> struct PrepSelect<T, DK, LNX_GATE_VECTOR> {
  static constexpr size_t bytes = KdaPrepSmem<T, DK>::bytes;
  static auto kernel(bool raw_gate) { return raw_gate ? kda_prepare_kernel<T, DK, true> : kda_prepare_kernel<T, DK, false>; }
};

template <typename T, int DK, int GATE>
int launch_fwd(const FwdParams& p, int nstate, hipStream_t st) {
  const int64_t slots = (int64_t)p.geom.rows * p.geom.N;
  auto k1 = PrepSelect<T, DK, GATE>::kernel(p.graw != nullptr);
  // 32-column slabs when 64-column ones would occupy at most half of the chip (256 CUs); always for 4-byte inputs
  // with dk = 256, whose tiles leave no room in LDS for a wider slab
  constexpr bool can_narrow = (DK >= 128 && sizeof(T) == 2) || (DK == 128 && sizeof(T) == 4);
  constexpr int WIDE = (DK > 128 && sizeof(T) == 4) ? 32 : 64, NARROW = can_narrow ? 32 : WIDE;
  const bool narrow = can_narrow && lnx_narrow_slabs((int64_t)nstate * p.geom.H * (p.dv / 64), p.slab);
  auto k2 = narrow ? chunk_scan_kernel<T, DK, GATE, NARROW> : chunk_scan_kernel<T, DK, GATE, WIDE>;
  auto k3 = chunk_output_kernel<T, DK, GATE>;
  const int bv = narrow ? NARROW : WIDE;
  const size_t b1 = PrepSelect<T, DK, GATE>::bytes, b3 = OutSmem<T, DK>::bytes;
  const size_t b2 = narrow ? ScanSmem<T, DK, NARROW>::bytes : ScanSmem<T, DK, WIDE>::bytes;
  hipError_t e;
  if ((e = hipFuncSetAttribute((const void*)k1, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b1)) != hipSuccess ||
      (e = hipFuncSetAttribute((const void*)k2, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b2)) != hipSuccess ||
      (e = hipFuncSetAttribute((const void*)k3, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b3)) != hipSuccess)
    return lnx_set_error(LNX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  lnx_profile_mark("chunk_prepare", st);
  hipLaunchKernelGGL(k1, dim3((unsigned)slots), dim3(256), b1, st, p);
  lnx_profile_mark("chunk_scan", st);
  hipLaunchKernelGGL(k2, dim3(lnx_xcd_grid((int64_t)nstate * p.geom.H, p.dv / bv)), dim3(512), b2, st, p);
  if (!ScanSmem<T, DK>::FUSE_OUT && p.o) {  // otherwise the scan has written the outputs
    lnx_profile_mark("chunk_output", st);
    // value slabs per workgroup: as many as leave about two thousand workgroups (p.out_spw > 0: the tests' override)
    const int nslab = p.dv / OutSmem<T, DK>::BV;
    FwdParams po = p;
    po.out_spw = (int)std::max<int64_t>(1, std::min<int64_t>(nslab, slots * nslab / 2048));
    if (p.out_spw > 0) po.out_spw = std::min(nslab, p.out_spw);
    hipLaunchKernelGGL(k3, dim3(lnx_xcd_grid(slots, (nslab + po.out_spw - 1) / po.out_spw)), dim3(256), b3, st, po);
  }
  lnx_profile_mark(nullptr, st);
  return LNX_OK;
}

template <typename T, int DK>
int launch_fwd_gate(int gate, const FwdParams& p, int nstate, hipStream_t st) {
  switch (gate) {
    case LNX_GATE_NONE: return launch_fwd<T, DK, LNX_GATE_NONE>(p, nstate, st);
    case LNX_GATE_SCALAR: return launch_fwd<T, DK, LNX_GATE_SCALAR>(p, nstate, st);
    case LNX_GATE_VECTOR: return launch_fwd<T, DK, LNX_GATE_VECTOR>(p, nstate, st);
    default: return lnx_set_error(LNX_ERR_SHAPE, "unknown gate kind %d", gate);
  }
}

}  // namespace

int lnx_chunk_check(const lnx_scan_args* a, bool backward) {
  if (!a) return lnx_set_error(LNX_ERR_NULL, "args is NULL");
  if (a->B < 0 || a->H <= 0 || a->T < 0) return lnx_set_error(LNX_ERR_SHAPE, "bad dimensions B=%d H=%d T=%d", a->B, a->H, a->T);
  // tensors without elements (no batch rows, or no tokens) may come with null pointers
  const bool tokens = a->B > 0 && a->T > 0;
  if (tokens && (!a->q || !a->k || !a->v || !a->beta)) return lnx_set_error(LNX_ERR_NULL, "q, k, v and beta are required");
  if (!backward && ((tokens && !a->o && !a->forward_only) || (a->B > 0 && !a->final_state)))
    return lnx_set_error(LNX_ERR_NULL, "o (unless forward_only) and final_state are required");
  if (a->value_cols != 0 && (backward || !a->forward_only || a->value_cols < 0 || a->value_cols > a->dv || a->value_cols % 64 != 0))
    return lnx_set_error(LNX_ERR_SHAPE, "value_cols = %d needs forward_only and a multiple of 64 up to dv = %d", a->value_cols, a->dv);
  if (backward && tokens && (!a->d_o || !a->d_q || !a->d_k || !a->d_v || !a->d_beta))
    return lnx_set_error(LNX_ERR_NULL, "d_o, d_q, d_k, d_v and d_beta are required");
  const bool raw_gate = a->gate_raw != nullptr;
  if (raw_gate && a->gate != LNX_GATE_VECTOR) return lnx_set_error(LNX_ERR_SHAPE, "gate_raw is the per-channel gate's raw projection: gate must be LNX_GATE_VECTOR");
  if (raw_gate && !a->gate_A_log) return lnx_set_error(LNX_ERR_NULL, "gate_raw needs gate_A_log");
  if (tokens && a->gate != LNX_GATE_NONE && !a->g && !raw_gate) return lnx_set_error(LNX_ERR_NULL, "gate kind %d needs g", a->gate);
  if (backward && tokens && a->gate != LNX_GATE_NONE && !(raw_gate ? a->d_gate_raw : (void*)a->d_g))
    return lnx_set_error(LNX_ERR_NULL, "gate kind %d needs %s", a->gate, raw_gate ? "d_gate_raw" : "d_g");
  if (a->gate < LNX_GATE_NONE || a->gate > LNX_GATE_VECTOR) return lnx_set_error(LNX_ERR_SHAPE, "unknown gate kind %d", a->gate);
  if (a->dk != 64 && a->dk != 128 && a->dk != 256)
    return lnx_set_error(LNX_ERR_SHAPE, "chunk kernels need dk in {64, 128, 256}, got %d", a->dk);
  if (a->dv <= 0 || a->dv % 64 != 0) return lnx_set_error(LNX_ERR_SHAPE, "chunk kernels need dv %% 64 == 0, got %d", a->dv);
  if (a->chunk != LNX_C) return lnx_set_error(LNX_ERR_SHAPE, "chunk length must be %d, got %d", LNX_C, a->chunk);
  if (a->dtype != LNX_F32 && a->dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "dtype %d", a->dtype);
  if (a->o_dtype != LNX_F32 && a->o_dtype != LNX_BF16) return lnx_set_error(LNX_ERR_DTYPE, "o_dtype %d", a->o_dtype);
  if (a->use_qk_l2norm && !lnx_chunk_direct(a))
    return lnx_set_error(LNX_ERR_SHAPE, "use_qk_l2norm inside the chunk kernels needs 2-byte inputs, dk <= 128 and no per-channel gate; "
                                        "normalise with lnx_l2norm_fwd first");
  if (a->token_first != 0 && a->token_first != 1) return lnx_set_error(LNX_ERR_SHAPE, "token_first must be 0 or 1");
  if ((a->test_scan_slab != 0 && a->test_scan_slab != 32 && a->test_scan_slab != 64) || a->test_out_slabs < 0)
    return lnx_set_error(LNX_ERR_SHAPE, "test_scan_slab must be 0, 32 or 64 and test_out_slabs >= 0");
  if (backward && a->forward_only) return lnx_set_error(LNX_ERR_SHAPE, "forward_only is set: the workspace holds nothing for a backward pass");
  if (a->cu_seqlens && (a->B != 1 || a->nseq <= 0))
    return lnx_set_error(LNX_ERR_SHAPE, "packed batches need B == 1 and nseq > 0 (B=%d nseq=%d)", a->B, a->nseq);
  // the kernels move rows of these tensors as 16-byte vectors (beta, the scalar gate and their gradients go by elements;
  // the workspace is checked where it is used: lnx_chunk_fwd_static ignores the field)
  const void* vec16[] = {a->q, a->k, a->v, a->o, a->initial_state, a->final_state, a->gate == LNX_GATE_VECTOR ? a->g : nullptr,
                         a->gate_raw, a->d_o, a->d_final_state, a->d_q, a->d_k, a->d_v,
                         a->gate == LNX_GATE_VECTOR ? a->d_g : nullptr, a->d_gate_raw, a->d_initial_state};
  for (const void* ptr : vec16)
    if (reinterpret_cast<uintptr_t>(ptr) & 15)
      return lnx_set_error(LNX_ERR_SHAPE, "q, k, v, o, the per-channel gate, the states, the workspace and their gradients must be 16-byte aligned (%p is not)", ptr);
  return LNX_OK;
}

namespace {

// 2-byte inputs with dk <= 128 and no per-channel gate: the prepare kernel stops at Tm, Pm and G, the scan of
// chunk_direct.hip does the rest.
template <int DK, int GATE>
void launch_prepare_lite(const FwdParams& p, hipStream_t st) {
  auto k = chunk_prepare2_kernel<bf16_t, DK, GATE, true>;
  lnx_profile_mark("chunk_prepare", st);
  const size_t b = Prep2Cfg<bf16_t, DK>::lite_bytes;
  hipLaunchKernelGGL(k, dim3((unsigned)((int64_t)p.geom.rows * p.geom.N)), dim3(256), b, st, p);
}

int launch_direct_fwd(const lnx_scan_args* a, const FwdParams& p, int nstate, hipStream_t st) {
  if (a->dk == 128) {
    if (a->gate == LNX_GATE_SCALAR) launch_prepare_lite<128, LNX_GATE_SCALAR>(p, st);
    else launch_prepare_lite<128, LNX_GATE_NONE>(p, st);
  } else {
    if (a->gate == LNX_GATE_SCALAR) launch_prepare_lite<64, LNX_GATE_SCALAR>(p, st);
    else launch_prepare_lite<64, LNX_GATE_NONE>(p, st);
  }
  DirectParams d = {};
  d.geom = p.geom;
  d.q = reinterpret_cast<const bf16_t*>(a->q); d.k = reinterpret_cast<const bf16_t*>(a->k);
  d.v = reinterpret_cast<const bf16_t*>(a->v); d.beta = a->beta; d.s0 = a->initial_state; d.sT_out = a->final_state;
  d.o = a->o; d.dv = a->dv; d.o_dtype = a->o_dtype; d.save = !a->forward_only; d.vcols = p.vcols; d.gate = a->gate;
  d.l2norm = a->use_qk_l2norm; d.slab = a->test_scan_slab;
  d.scale = a->scale; d.ws = p.ws; d.off = p.off;
  int rc = lnx_direct_scan_fwd(d, a->dk, a->gate, nstate, st);
  if (rc != LNX_OK) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "chunk forward launch: %s", hipGetErrorString(e));
  return LNX_OK;
}

// The forward pass on a caller-chosen workspace (a->workspace is not looked at).
int chunk_fwd_on(const lnx_scan_args* a, void* workspace, uint64_t workspace_bytes, hipStream_t st) {
  const bool packed = a->cu_seqlens != nullptr;
  const int nstate = packed ? a->nseq : a->B;
  if (nstate == 0) return LNX_OK;
  if (a->T == 0) {
    const int64_t n = (int64_t)nstate * a->H * a->dk * a->dv;
    hipLaunchKernelGGL(copy_state_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a->initial_state,
                       a->final_state, n);
    return LNX_OK;
  }
  const ChunkWs w = lnx_chunk_ws_layout(a);
  if (reinterpret_cast<uintptr_t>(workspace) & 15) return lnx_set_error(LNX_ERR_WORKSPACE, "the workspace must be 16-byte aligned");
  if (!workspace || workspace_bytes < w.total)
    return lnx_set_error(LNX_ERR_WORKSPACE, "workspace of %llu bytes needed, %llu given", (unsigned long long)w.total,
                         (unsigned long long)workspace_bytes);
  char* ws = reinterpret_cast<char*>(workspace);
  if (packed)
    hipLaunchKernelGGL(build_table_kernel, dim3(1), dim3(256), 0, st, a->cu_seqlens, a->nseq, lnx_chunk_slots(a), a->T,
                       reinterpret_cast<int32_t*>(ws + w.tab));
  FwdParams p;
  p.geom.H = a->H; p.geom.T = a->T; p.geom.N = lnx_chunk_slots(a); p.geom.nseq = a->nseq;
  p.geom.ts = a->token_first ? a->H : 1;
  p.geom.rows = packed ? a->H : a->B * a->H;
  p.geom.cu = a->cu_seqlens;
  p.geom.tab = packed ? reinterpret_cast<const int32_t*>(ws + w.tab) : nullptr;
  p.q = a->q; p.k = a->k; p.v = a->v; p.beta = a->beta; p.g = a->g; p.s0 = a->initial_state;
  p.sT_out = a->final_state; p.o = a->o; p.dv = a->dv; p.o_dtype = a->o_dtype; p.scale = a->scale;
  // 4-byte inputs form the outputs in a separate kernel that reads the state and D back
  p.save = !(a->forward_only && a->dtype == LNX_BF16);
  p.out_spw = a->test_out_slabs;
  p.slab = a->test_scan_slab;
  p.graw = a->gate == LNX_GATE_VECTOR ? a->gate_raw : nullptr; p.gA = a->gate_A_log; p.gbias = a->gate_bias; p.gthr = a->gate_threshold;
  p.vcols = a->value_cols ? a->value_cols : a->dv;
  p.l2norm = a->use_qk_l2norm;
  p.ws = ws; p.off = w;
  int rc;
  if (lnx_chunk_direct(a)) return launch_direct_fwd(a, p, nstate, st);
  if (a->dtype == LNX_BF16)  // dk <= 128 without a per-channel gate went to the direct-solve kernels above
    rc = (a->dk == 256)   ? launch_fwd_gate<bf16_t, 256>(a->gate, p, nstate, st)
         : (a->dk == 128) ? launch_fwd<bf16_t, 128, LNX_GATE_VECTOR>(p, nstate, st)
                          : launch_fwd<bf16_t, 64, LNX_GATE_VECTOR>(p, nstate, st);
  else
    rc = (a->dk == 256)   ? launch_fwd_gate<float, 256>(a->gate, p, nstate, st)
         : (a->dk == 128) ? launch_fwd_gate<float, 128>(a->gate, p, nstate, st)
                          : launch_fwd_gate<float, 64>(a->gate, p, nstate, st);
  if (rc != LNX_OK) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "chunk forward launch: %s", hipGetErrorString(e));
  return LNX_OK;
}

// Library-owned scratch of lnx_chunk_fwd_static: one copy per GPU, at its own address on each, alive until the
// process ends.  The name below is a host-side handle only; device code gets the address looked up per device.
static __device__ __align__(256) unsigned char scratch[LNX_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Address of `scratch` on the current device (looked up once per device, with that device current).
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return lnx_set_error(LNX_ERR_DEVICE, "hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return lnx_set_error(LNX_ERR_DEVICE, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return LNX_OK;
}

}  // namespace

extern "C" uint64_t lnx_chunk_workspace_bytes(const lnx_scan_args* a) {
  // only the geometry matters here; tensor pointers may still be unset
  if (!a || a->H <= 0 || a->T < 0 || a->B < 0 || (a->dk != 64 && a->dk != 128 && a->dk != 256) || a->dv <= 0 || a->dv % 64 != 0 ||
      (a->cu_seqlens && a->nseq <= 0))
    return 0;
  return lnx_chunk_ws_layout(a).total;
}

extern "C" int lnx_chunk_fuses_l2norm(const lnx_scan_args* a) { return a && lnx_chunk_direct(a) ? 1 : 0; }

extern "C" int lnx_chunk_fwd(const lnx_scan_args* a, void* stream) {
  int rc = lnx_chunk_check(a, false);
  if (rc != LNX_OK) return rc;
  return chunk_fwd_on(a, a->workspace, a->workspace_bytes, (hipStream_t)stream);
}

extern "C" int lnx_chunk_fwd_static_init(void) {
  void* ws = nullptr;
  return static_scratch(&ws);
}

extern "C" int lnx_chunk_fwd_static(const lnx_scan_args* a, void* stream) {
  int rc = lnx_chunk_check(a, false);
  if (rc != LNX_OK) return rc;
  if (!a->forward_only)
    return lnx_set_error(LNX_ERR_WORKSPACE, "lnx_chunk_fwd_static needs forward_only: the library's scratch does not outlive the call");
  const uint64_t need = (a->T == 0 || a->B == 0) ? 0 : lnx_chunk_ws_layout(a).total;
  if (need > (uint64_t)LNX_STATIC_SCRATCH_BYTES)
    return lnx_set_error(LNX_ERR_WORKSPACE, "lnx_chunk_fwd_static: this shape needs %llu bytes of scratch, the library holds %llu",
                         (unsigned long long)need, (unsigned long long)LNX_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if ((rc = static_scratch(&ws)) != LNX_OK) return rc;
  return chunk_fwd_on(a, ws, LNX_STATIC_SCRATCH_BYTES, (hipStream_t)stream);
}
