// Chunked delta-rule forward and backward for 2-byte inputs with dk <= 128 and no / a scalar gate, in the
// "direct solve" split: the only per-chunk tensors that cross kernels are Tm = (I + A)^-1, Pm = scale tril(E * Q K^T)
// and the cumulative gate G from the chunk-parallel prepare kernel, the states entering the chunks and D (forward scan
// -> chunk-local backward) and the state gradients leaving them and dR (reverse scan -> chunk-local backward).  W, U,
// dD, dW of the WY form are never materialised: with S the state entering a chunk,
//
//   Y = K S          R = diag(beta) (V - diag(e^G) Y)      D = Tm R                     (forward substitution applied
//   O = scale diag(e^G) (Q S) + Pm D                                                     to the chunk's right-hand
//   S' = e^{G_C} S + (diag(e^{G_C - G}) K)^T D                                           side, gated_deltanet.py:450-477)
//
// and in reverse, with dS' the gradient of the state leaving the chunk,
//
//   dD = Pm^T dO + diag(e^{G_C - G}) K dS'     dR = Tm^T dD     dY = -diag(beta e^G) dR
//   dS = e^{G_C} dS' + (scale diag(e^G) Q)^T dO + K^T dY
//
// which is the algorithm of linearnexus/modules/linear_attn/gated_deltanet.py:444-523 (delta_net.py:296-330 without
// a gate) and its hand-derived adjoint (the reference's gradients come from JAX autodiff).  Three kernels:
//
//   scan_fwd   (one workgroup per (state, slab of dv), sequential over chunks)   O, the entering states, S_T
//   scan_bwd   (same grid, reverse)                                              the leaving state gradients, dS_0
//   bwd_chunk  (one workgroup per chunk, all in parallel)                         dq, dk, dbeta, dg from q, k, v, dO, the
//              two saved states and D, dR as the scans left them (dv leaves the reverse scan)
//
// Both scans split their waves into one compute wave per 32 value columns of the slab (two for the 64-column slabs:
// matrix work on the tiles in LDS, the fp32 state in MFMA accumulators for the whole sequence) and four mover waves
// (global loads two chunks ahead into registers, the next chunk's tiles into LDS, LDS -> global copies of results as
// whole rows); all five input tiles and the per-token scalars are double-buffered in LDS, so two LDS-only barriers per
// chunk suffice.  bwd_chunk brings its slabs in with loads that go straight to LDS (mma_tiles.h).

#include <type_traits>

#include "chunk_common.h"

namespace {

using T = bf16_t;
typedef Mma<T> M;
template <typename X> __device__ __forceinline__ X* at(char* ws, uint64_t off) { return reinterpret_cast<X*>(ws + off); }

// dst[col][row0 + ...] = fragment (transposed store, four consecutive rows per 8-byte vector)
__device__ __forceinline__ void store_frag_t(const floatx16& a, T* dst, int ld, int lane) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const floatx4 x = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
    store4(dst + (lane & 31) * ld + 8 * q + 4 * (lane >> 5), x);
  }
}

// Zeroes the 224 vectors above the diagonal (row r, columns 8 c .. 8 c + 7 with 8 c > r) of `ntile` consecutive
// [64][ld] tiles of `stride` elements; 256 threads.  Group g of eight rows has 7 - g such vectors per row.
__device__ __forceinline__ void zero_upper_triangles(T* tiles, int ntile, int stride, int ld, int tid) {
  if (tid >= 512 - LNX_TRI_VECS) return;
  int g = 0;
  while (56 * (g + 1) - 4 * (g + 1) * g <= tid) ++g;  // vectors of the groups before g + 1
  const int o = tid - (56 * g - 4 * g * (g - 1)), per = 7 - g;
  const int r = 8 * g + o / per, c = g + 1 + (o - (o / per) * per);
  for (int t = 0; t < ntile; ++t) *reinterpret_cast<Vec16<T>::V*>(tiles + t * stride + r * ld + 8 * c) = vec_zero<T>();
}

// Per-token scalars of one chunk in LDS, written by the movers when they commit a chunk
struct Scal {
  enum { BETA = 0, GAM = 64, R = 128, SG = 192, DEC = 256, SIZE = 320 };  // beta, e^G, e^{G_C - G}, scale e^G, e^{G_C}
};

// ---------------------------------------------------------------------------------------
// scan_fwd.  A compute wave owns a 32-column strip of the value slab: its [dk x 32] part of the state stays in MFMA
// accumulators for the whole sequence, and the chain  S -> Y = K S -> R -> D = Tm R -> S'  never leaves the wave's
// registers -- an accumulator fragment is the B operand of the next product as it is (Mma::from_acc), only the A
// operands (K, Q, Tm, Pm rows) come from LDS.  All five input tiles are double-buffered, so the movers write chunk
// n + 1 while chunk n is being read and two barriers per chunk are enough:
//   B1    buffers of chunk n complete           compute: S^T -> LDS (saved states), Y, Q S, R, D (-> LDS, transposed), O -> LDS
//                                               movers:  loads of chunk n + 2; chunk n + 1 -> the other buffers
//   Bmid  O, S^T and D^T are in LDS             compute: state update        movers: O, S^T, D^T -> global
// ---------------------------------------------------------------------------------------
template <int DK, int BVW> struct FScanL {
  static constexpr int PAD = M::PAD, LDK = DK + PAD, LDC = LNX_C + PAD, BV = BVW, LDV = BV + PAD, NCW = BV / 32;
  static constexpr int kK = 64 * LDK, kST = BV * LDK, kV = 64 * LDV, kC = 64 * LDC;
  static constexpr int kDT = BV * LDC;
  // [2] x (K, Q, V, Tm, Pm) | O | S^T | D^T | scalars [2]
  static constexpr size_t bytes = sizeof(T) * (2 * (2 * kK + kV + 2 * kC) + kV + kST + kDT) + sizeof(float) * 2 * Scal::SIZE;
  static constexpr int threads = 64 * NCW + 256;
};

template <int DK, int GATE, int BVW, typename OT>
__global__ __launch_bounds__((FScanL<DK, BVW>::threads)) void scan_fwd_kernel(DirectParams p) {
  typedef FScanL<DK, BVW> L;
  constexpr int LDK = L::LDK, LDC = L::LDC, BV = L::BV, LDV = L::LDV, NCW = L::NCW;
  constexpr int KT = DK / 32;  // row tiles of the state strip
  static_assert(DK == 64 || DK == 128, "dk = 64 or 128");
  extern __shared__ __align__(16) char smem[];
  T* sK = reinterpret_cast<T*>(smem);  // [2][64][LDK]
  T* sQ = sK + 2 * L::kK;
  T* sV = sQ + 2 * L::kK;              // [2][64][LDV]
  T* sTm = sV + 2 * L::kV;             // [2][64][LDC]
  T* sP = sTm + 2 * L::kC;
  T* sO = sP + 2 * L::kC;              // bf16 outputs on their way out [64][LDV]
  T* sST = sO + L::kV;                 // entering state, transposed [v][dk], on its way to the workspace
  T* sDT = sST + L::kST;               // D^T [v][token] on its way to the workspace
  float* sSc = reinterpret_cast<float*>(sDT + L::kDT);  // [2][Scal::SIZE]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  int sidx, row, seq;
  int64_t chain;
  int slab;
  if (!xcd_slot_part((int64_t)(p.geom.tab ? p.geom.nseq : p.geom.rows / p.geom.H) * p.geom.H, p.dv / BV, chain, slab)) return;
  scan_state(p.geom, (int)chain, sidx, row, seq);
  const int v0 = slab * BV;
  int c0, c1;
  seq_chunks(p.geom, seq, c0, c1);
  const SeqSpan span = seq_span(p.geom, seq, c0);
  const int64_t tsk = (int64_t)p.geom.ts * DK, tsv = (int64_t)p.geom.ts * p.vcols, tso = (int64_t)p.geom.ts * p.dv;

  if (wave >= NCW) {
    // ---------------- movers ----------------
    const int mt = tid - 64 * NCW;
    typedef TileRegs<T, 64, DK> RowTile;
    typedef TileRegs<T, 64, BV> ValTile;
    struct Tiles {
      RowTile K, Q;
      ValTile V;
      TriRegs<T> Tm, P;  // lower-triangular tiles, packed in the workspace
      float g, gc, b;
      float fq[RowTile::IT], nk[RowTile::IT];  // factors of the token each of this thread's Q / K vectors belongs to
      float bv[ValTile::IT];  // beta of the token each of its V vectors belongs to
      int len;
    };
    Tiles ta, tb;
    ta.g = ta.gc = ta.b = tb.g = tb.gc = tb.b = 0.f;
    ta.Tm.init(LDC, mt), ta.P.init(LDC, mt), tb.Tm.init(LDC, mt), tb.P.init(LDC, mt);
    zero_upper_triangles(sTm, 4, L::kC, LDC, mt);  // both buffers of Tm and Pm: the packed tiles never write there
    ta.len = tb.len = 0;
#pragma unroll
    for (int it = 0; it < RowTile::IT; ++it) ta.fq[it] = tb.fq[it] = ta.nk[it] = tb.nk[it] = 0.f;
#pragma unroll
    for (int it = 0; it < ValTile::IT; ++it) ta.bv[it] = tb.bv[it] = 0.f;
    // part 0: K, 1: Q, 2: the rest; < 0: everything
    auto fetch = [&](Tiles& R, int n, int part = -1) {
      const int64_t slot = (int64_t)row * N + n;
      int tok0;
      chunk_span(span, n, tok0, R.len);
      const int64_t tbase = tok_index(p.geom, row, tok0);
      if (part < 0 || part == 0) R.K.load(p.k + tbase * DK, tsk, R.len, mt);
      if (part < 0 || part == 1) R.Q.load(p.q + tbase * DK, tsk, R.len, mt);
      if (part == 0 || part == 1) return;
      R.V.load(p.v + tbase * p.vcols + v0, tsv, (v0 < p.vcols) ? R.len : 0, mt);  // columns v does not hold read as zero
      R.Tm.load(at<const T>(p.ws, p.off.Tm) + slot * 64 * 64, mt);
      R.P.load(at<const T>(p.ws, p.off.P) + slot * 64 * 64, mt);
      // every thread loads the scalars of token mt % 64 (no load behind a branch); tokens past the end are masked below
      const int t = mt & 63;
      if (GATE == LNX_GATE_SCALAR) {
        const float* G = at<const float>(p.ws, p.off.G) + slot * 64;
        R.g = G[t];
        R.gc = G[63];
      }
#pragma unroll
      for (int it = 0; it < RowTile::IT; ++it) {
        R.fq[it] = at<const float>(p.ws, p.off.Fq)[slot * 64 + (mt + 256 * it) / RowTile::VPR];
        R.nk[it] = at<const float>(p.ws, p.off.Nk)[slot * 64 + (mt + 256 * it) / RowTile::VPR];
      }
      R.b = p.beta[tbase + (int64_t)min(t, R.len - 1) * p.geom.ts];
#pragma unroll
      for (int it = 0; it < ValTile::IT; ++it)
        R.bv[it] = p.beta[tbase + (int64_t)min(min((mt + 256 * it) / ValTile::VPR, 63), R.len - 1) * p.geom.ts];
    };
    auto commit = [&](const Tiles& R, int pb, int part = -1) {
      {  // K rows normalised; Q rows normalised and scaled by scale e^{G_i}: the outputs then need no scaling of their own
        T* dstk = sK + pb * L::kK;
        T* dst = sQ + pb * L::kK;
#pragma unroll
        for (int it = 0; it < RowTile::IT; ++it) {
          const int idx = mt + 256 * it, r = idx / RowTile::VPR, c = (idx - r * RowTile::VPR) * RowTile::N;
          if (part < 0 || part == 0) {
            typename Vec16<T>::V y = R.K.x[it];
#pragma unroll
            for (int e = 0; e < RowTile::N; ++e) y[e] = (bf16_t)((float)y[e] * R.nk[it]);
            *reinterpret_cast<typename Vec16<T>::V*>(dstk + r * LDK + c) = y;
          }
          if (part < 0 || part == 1) {
            typename Vec16<T>::V x = R.Q.x[it];
#pragma unroll
            for (int e = 0; e < RowTile::N; ++e) x[e] = (bf16_t)((float)x[e] * R.fq[it]);
            *reinterpret_cast<typename Vec16<T>::V*>(dst + r * LDK + c) = x;
          }
        }
      }
      if (part == 0 || part == 1) return;
      {  // V rows scaled by beta_i: R = beta V - (beta e^G) Y
        T* dst = sV + pb * L::kV;
#pragma unroll
        for (int it = 0; it < ValTile::IT; ++it) {
          const int idx = mt + 256 * it, r = idx / ValTile::VPR, c = (idx - r * ValTile::VPR) * ValTile::N;
          typename Vec16<T>::V x = R.V.x[it];
#pragma unroll
          for (int e = 0; e < ValTile::N; ++e) x[e] = (bf16_t)((float)x[e] * R.bv[it]);
          if (idx < ValTile::TOTAL) *reinterpret_cast<typename Vec16<T>::V*>(dst + r * LDV + c) = x;
        }
      }
      R.Tm.store(sTm + pb * L::kC);
      R.P.store(sP + pb * L::kC);
      if (mt < 64) {
        float* sc = sSc + pb * Scal::SIZE;
        const float gam = (GATE == LNX_GATE_SCALAR) ? __expf(R.g) : 1.f;
        sc[Scal::GAM + mt] = (mt < R.len) ? R.b * gam : 0.f;  // beta e^G
        sc[Scal::R + mt] = (GATE == LNX_GATE_SCALAR) ? __expf(fminf(R.gc - R.g, 0.f)) : 1.f;
        if (mt == 0) sc[Scal::DEC] = (GATE == LNX_GATE_SCALAR) ? __expf(R.gc) : 1.f;
      }
    };
    // cur: the register set that held chunk n (in LDS since the last step) and now takes chunk n + 2; nxt: chunk n + 1.
    // `steady` (a std::bool_constant): chunks n + 1 and n + 2 exist, so nothing below sits behind a branch -- behind a
    // conditional fetch the compiler cannot count the younger loads in flight and would wait for all of them.
    // The loads are admitted at the rate the memory path takes them, and a wave that has a load waiting for a slot
    // issues nothing else: so the tile writes of chunk n + 1 sit between the loads of chunk n + 2, a tile at a time, and
    // go out while the loads before them drain (issued one after the other: forward scan 237 -> 216 us).
    auto step = [&](Tiles& cur, const Tiles& nxt, int n, auto steady) {
      constexpr bool STEADY = decltype(steady)::value;
      if constexpr (STEADY) {
#pragma unroll
        for (int part = 0; part < 3; ++part) {
          fetch(cur, n + 2, part);
          commit(nxt, (n + 1 - c0) & 1, part);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        if (n + 2 < c1) fetch(cur, n + 2);
        if (n + 1 < c1) commit(nxt, (n + 1 - c0) & 1);
      }
      lds_barrier();  // Bmid
      int tok0, len;
      chunk_span(span, n, tok0, len);
      if (p.o) {
        if constexpr (std::is_same<OT, float>::value)
          unstage_tile_checked_widen<64, BV>(reinterpret_cast<float*>(p.o) + tok_index(p.geom, row, tok0) * p.dv + v0, tso, sO, LDV, len, mt);
        else
          unstage_tile_checked<bf16_t, 64, BV>(reinterpret_cast<bf16_t*>(p.o) + tok_index(p.geom, row, tok0) * p.dv + v0, tso, sO, LDV, len, mt);
      }
      if (p.save) {
        const int64_t slot = (int64_t)row * N + n;
        unstage_tile<T, BV, DK, true>(at<T>(p.ws, p.off.SnT) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sST, LDK, BV, mt);
        unstage_tile<T, BV, 64, true>(at<T>(p.ws, p.off.D) + slot * p.dv * 64 + (int64_t)v0 * 64, 64, sDT, LDC, BV, mt);
      }
      lds_barrier();  // B1 of the next chunk
    };
    // the register sets and the LDS double buffers alternate by position in the sequence (chunk c0: set a, buffer 0)
    if (c0 < c1) {
      fetch(ta, c0);
      commit(ta, 0);
    }
    if (c0 + 1 < c1) fetch(tb, c0 + 1);
    lds_barrier();  // B1 of the first chunk
    int n = c0;
    for (; n + 3 < c1; n += 2) {  // chunks n + 2 and n + 3 exist
      step(ta, tb, n, std::true_type{});
      step(tb, ta, n + 1, std::true_type{});
    }
    for (; n < c1; n += 2) {
      step(ta, tb, n, std::false_type{});
      if (n + 1 < c1) step(tb, ta, n + 1, std::false_type{});
    }
    return;
  }

  // ---------------- compute waves: wave w owns value columns [32 w, 32 w + 32) of the slab ----------------
  const int vs = 32 * wave;
  const int fr = lane & 31;
  floatx16 S[KT];
#pragma unroll
  for (int ci = 0; ci < KT; ++ci)
#pragma unroll
    for (int e = 0; e < 16; ++e) S[ci][e] = 0.f;
  if (p.s0) {
    const float* s0 = p.s0 + (int64_t)sidx * DK * p.dv + v0 + vs;
#pragma unroll
    for (int ci = 0; ci < KT; ++ci)
#pragma unroll
      for (int e = 0; e < 16; ++e) S[ci][e] = s0[(int64_t)(32 * ci + frag_row(e, lane)) * p.dv + frag_col(lane)];
    // the loads complete here: left pending into the loop, every iteration would count them down again
#pragma unroll
    for (int ci = 0; ci < KT; ++ci)
#pragma unroll
      for (int e = 0; e < 16; ++e) asm volatile("" : "+v"(S[ci][e]));
  }
  lds_barrier();  // B1 of the first chunk
  // Every LDS read is issued well ahead of the product that consumes it (A fragments two steps ahead, the next
  // phase's first fragments and scalars during the current phase's last steps): a wave alone on its SIMD has nothing
  // else to cover the LDS latency with.  The scheduling fences pin that order.
  constexpr int NK = DK / 16;  // 16-wide steps over dk
  for (int n = c0; n < c1; ++n) {
    const int pb = (n - c0) & 1;
    const T* sKc = sK + pb * L::kK;
    const T* sQc = sQ + pb * L::kK;
    const T* sVc = sV + pb * L::kV;
    const T* sTc = sTm + pb * L::kC;
    const T* sPc = sP + pb * L::kC;
    const float* sc = sSc + pb * Scal::SIZE;
    if (p.save) {
#pragma unroll
      for (int ci = 0; ci < KT; ++ci) store_frag_t(S[ci], sST + vs * LDK + 32 * ci, LDK, lane);
    }
    // ---- Y = K S (lane = value column) and (Q~ S)^T (lane = token): the state fragments are the shared operand ----
    floatx16 y[2], o[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) y[i][e] = o[i][e] = 0.f;
    M::Frag fa[3][2], fb[3][2];  // [step mod 3][row tile]
    bf16x4 vr[2][4];             // beta V at this lane's accumulator positions
    floatx4 sv[2][4];            // per-row scalars at this lane's accumulator positions: beta e^G, later e^{G_C - G}
#pragma unroll
    for (int s_ = 0; s_ < 2; ++s_)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[s_][i] = M::load_chain(sKc + (32 * i + fr) * LDK + 16 * s_, lane);
        fb[s_][i] = M::load_chain(sQc + (32 * i + fr) * LDK + 16 * s_, lane);
      }
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      if (ks + 2 < NK) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          fa[(ks + 2) % 3][i] = M::load_chain(sKc + (32 * i + fr) * LDK + 16 * (ks + 2), lane);
          fb[(ks + 2) % 3][i] = M::load_chain(sQc + (32 * i + fr) * LDK + 16 * (ks + 2), lane);
        }
      }
      if (ks == NK - 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            vr[i][q] = M::load_acc_rows_raw(sVc, LDV, 32 * i, q, vs, lane);
            sv[i][q] = load4(sc + Scal::GAM + 32 * i + 8 * q + 4 * (lane >> 5));
          }
      }
      const M::Frag b = M::from_acc(S[ks >> 1], ks & 1);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        M::mma(y[i], fa[ks % 3][i], b);
        M::mma(o[i], b, fb[ks % 3][i]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // Tm and Pm are lower-triangular: the first 32 rows of D and of the outputs take the first 32 tokens only, so the two
    // products need 6 MFMAs each, not 8, and the work on the first half (R, D, scaling, conversions, stores) runs in the
    // shadow of the second half's MFMAs.  tm[i][ks], pm[i][ks]: row tile i, 16-token step ks (i = 0: ks < 2).
    M::Frag tm0[2], tm1[4], pm0[2], pm1[4];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      tm0[ks] = M::load_chain(sTc + fr * LDC + 16 * ks, lane);
      tm1[ks] = M::load_chain(sTc + (32 + fr) * LDC + 16 * ks, lane);
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- R = beta V - (beta e^G) Y, in place of Y: tokens 0 .. 31 ----
    auto form_r = [&](int i) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int u = 0; u < 4; ++u) y[i][4 * q + u] = (float)vr[i][q][u] - sv[i][q][u] * y[i][4 * q + u];
    };
    form_r(0);
    M::Frag br[4];
    br[0] = M::from_acc(y[0], 0), br[1] = M::from_acc(y[0], 1);
    __builtin_amdgcn_sched_barrier(0);
    // ---- D = Tm R: the steps over tokens 0 .. 31, with R of tokens 32 .. 63 formed meanwhile ----
    floatx16 d[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) d[i][e] = 0.f;
#pragma unroll
    for (int ks = 2; ks < 4; ++ks) tm1[ks] = M::load_chain(sTc + (32 + fr) * LDC + 16 * ks, lane);
    M::mma(d[0], tm0[0], br[0]);
    M::mma(d[1], tm1[0], br[0]);
    M::mma(d[0], tm0[1], br[1]);
    M::mma(d[1], tm1[1], br[1]);
    form_r(1);
    br[2] = M::from_acc(y[1], 0), br[3] = M::from_acc(y[1], 1);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      pm0[ks] = M::load_chain(sPc + fr * LDC + 16 * ks, lane);
      pm1[ks] = M::load_chain(sPc + (32 + fr) * LDC + 16 * ks, lane);
    }
    if (GATE == LNX_GATE_SCALAR) {  // e^{G_C - G} for the state update
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) sv[i][q] = load4(sc + Scal::R + 32 * i + 8 * q + 4 * (lane >> 5));
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- the last two steps of D's second half; the first half goes on to the outputs ----
    M::Frag fu[2][KT];  // K^T fragments of the state update, [step parity][row tile of the state]
    M::Frag bd[4];      // D as the outputs' operand; br becomes the state update's operand (rows scaled by e^{G_C - G})
    M::mma(d[1], tm1[2], br[2]);
    M::mma(d[1], tm1[3], br[3]);
    store_frag_t(d[0], sDT + vs * LDC, LDC, lane);  // also when nothing is saved: a branch here would split the schedule
    bd[0] = M::from_acc(d[0], 0), bd[1] = M::from_acc(d[0], 1);
    __builtin_amdgcn_sched_barrier(0);
    // ---- O^T = (Q~ S)^T + D^T Pm^T ----
#pragma unroll
    for (int ks = 2; ks < 4; ++ks) pm1[ks] = M::load_chain(sPc + (32 + fr) * LDC + 16 * ks, lane);
    M::mma(o[0], bd[0], pm0[0]);
    M::mma(o[1], bd[0], pm1[0]);
    M::mma(o[0], bd[1], pm0[1]);
    M::mma(o[1], bd[1], pm1[1]);
    store_frag_t(d[1], sDT + vs * LDC + 32, LDC, lane);
    bd[2] = M::from_acc(d[1], 0), bd[3] = M::from_acc(d[1], 1);
#pragma unroll
    for (int ci = 0; ci < KT; ++ci) fu[0][ci] = M::load_t_chain(sKc, LDK, 0, 32 * ci, lane);
    __builtin_amdgcn_sched_barrier(0);
    M::mma(o[1], bd[2], pm1[2]);
    M::mma(o[1], bd[3], pm1[3]);
    store_frag_t(o[0], sO + vs, LDV, lane);  // [token][value column]
    // the state update's operand while the last products finish: D rows scaled by e^{G_C - G}
    if (GATE == LNX_GATE_SCALAR) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int u = 0; u < 4; ++u) d[i][4 * q + u] *= sv[i][q][u];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) br[ks] = M::from_acc(d[ks >> 1], ks & 1);
    } else {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) br[ks] = bd[ks];
    }
    const float dec = (GATE == LNX_GATE_SCALAR) ? sc[Scal::DEC] : 1.f;
    __builtin_amdgcn_sched_barrier(0);
    store_frag_t(o[1], sO + 32 * LDV + vs, LDV, lane);
    lds_barrier();  // Bmid
    // ---- S <- e^{G_C} S + K^T (e^{G_C - G} D) ----
    if (GATE == LNX_GATE_SCALAR) {
#pragma unroll
      for (int ci = 0; ci < KT; ++ci)
#pragma unroll
        for (int e = 0; e < 16; ++e) S[ci][e] *= dec;
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) {
#pragma unroll
        for (int ci = 0; ci < KT; ++ci) fu[(ks + 1) & 1][ci] = M::load_t_chain(sKc, LDK, 16 * (ks + 1), 32 * ci, lane);
      }
#pragma unroll
      for (int ci = 0; ci < KT; ++ci) M::mma(S[ci], fu[ks & 1][ci], br[ks]);
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();  // B1 of the next chunk
  }
  float* out = p.sT_out + (int64_t)sidx * DK * p.dv + v0 + vs + frag_col(lane);
#pragma unroll
  for (int ci = 0; ci < KT; ++ci)
#pragma unroll
    for (int e = 0; e < 16; ++e) out[(int64_t)(32 * ci + frag_row(e, lane)) * p.dv] = S[ci][e];
}

template <int DK, int GATE, typename OT>
int launch_scan_fwd(const DirectParams& p, int nstate, hipStream_t st) {
  // 32-column slabs (one compute wave) when 64-column ones would occupy at most half of the chip
  const bool narrow = lnx_narrow_slabs((int64_t)nstate * p.geom.H * (p.dv / 64), p.slab);
  auto k = narrow ? scan_fwd_kernel<DK, GATE, 32, OT> : scan_fwd_kernel<DK, GATE, 64, OT>;
  const size_t b = narrow ? FScanL<DK, 32>::bytes : FScanL<DK, 64>::bytes;
  const int bv = narrow ? 32 : 64, threads = narrow ? FScanL<DK, 32>::threads : FScanL<DK, 64>::threads;
  hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b);
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  lnx_profile_mark("chunk_scan", st);
  hipLaunchKernelGGL(k, dim3(lnx_xcd_grid((int64_t)nstate * p.geom.H, p.dv / bv)), dim3(threads), b, st, p);
  lnx_profile_mark(nullptr, st);
  return LNX_OK;
}

// ---------------------------------------------------------------------------------------
// scan_bwd: the reverse pass, same organisation as scan_fwd.  A compute wave owns a 32-column strip of dS (the
// gradient of the state leaving the chunk); the chain  dS' -> Z = K dS' -> dD -> dR = Tm^T dD -> dY -> dS  stays in
// its registers.  Needs no forward state: only K, Q, dO, Tm, Pm and the per-token scalars.
//   B1    buffers of chunk n complete           compute: dS'^T -> LDS (saved), Z, Pm^T dO, dD, dR (-> LDS, transposed),
//                                                        dv = beta dR -> LDS, dY
//                                               movers:  loads of chunk n - 2; chunk n - 1 -> the other buffers
//   Bmid  dS'^T, dR^T and dv are in LDS         compute: dS update          movers: dS'^T, dR^T -> workspace, dv out
// ---------------------------------------------------------------------------------------
template <int DK, int BVW> struct BScanL {
  static constexpr int PAD = M::PAD, LDK = DK + PAD, LDC = LNX_C + PAD, BV = BVW, LDV = BV + PAD, NCW = BV / 32;
  static constexpr int kK = 64 * LDK, kST = BV * LDK, kV = 64 * LDV, kC = 64 * LDC;
  static constexpr int kDT = BV * LDC;
  // [2] x (K, scaled Q, dO, Tm, Pm) | dS'^T | dR^T | dv | scalars [2]
  static constexpr size_t bytes = sizeof(T) * (2 * (2 * kK + kV + 2 * kC) + kST + kDT + kV) + sizeof(float) * 2 * Scal::SIZE;
  static constexpr int threads = 64 * NCW + 256;
};

template <int DK, int GATE, int BVW>
__global__ __launch_bounds__((BScanL<DK, BVW>::threads)) void scan_bwd_kernel(DirectParams p) {
  typedef BScanL<DK, BVW> L;
  constexpr int LDK = L::LDK, LDC = L::LDC, BV = L::BV, LDV = L::LDV, NCW = L::NCW;
  constexpr int KT = DK / 32;
  extern __shared__ __align__(16) char smem[];
  T* sK = reinterpret_cast<T*>(smem);  // [2][64][LDK]
  T* sQ = sK + 2 * L::kK;              // rows scaled by scale e^G
  T* sdO = sQ + 2 * L::kK;             // [2][64][LDV]
  T* sTm = sdO + 2 * L::kV;
  T* sP = sTm + 2 * L::kC;
  T* sdST = sP + 2 * L::kC;            // dS'^T [v][dk] on its way to the workspace
  T* sdRT = sdST + L::kST;             // dR^T [v][token] on its way to the workspace
  T* sdV = sdRT + L::kDT;              // dv = beta dR [token][v] on its way out
  float* sSc = reinterpret_cast<float*>(sdV + L::kV);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  int sidx, row, seq;
  int64_t chain;
  int slab;
  if (!xcd_slot_part((int64_t)(p.geom.tab ? p.geom.nseq : p.geom.rows / p.geom.H) * p.geom.H, p.dv / BV, chain, slab)) return;
  scan_state(p.geom, (int)chain, sidx, row, seq);
  const int v0 = slab * BV;
  int c0, c1;
  seq_chunks(p.geom, seq, c0, c1);
  const SeqSpan span = seq_span(p.geom, seq, c0);
  const int64_t tsk = (int64_t)p.geom.ts * DK, tsv = (int64_t)p.geom.ts * p.dv;

  if (wave >= NCW) {
    // ---------------- movers ----------------
    const int mt = tid - 64 * NCW;
    typedef TileRegs<T, 64, DK> RowTile;
    struct Tiles {
      RowTile K, Q;
      TileRegs<T, 64, BV> dO;
      TriRegs<T> Tm, P;  // lower-triangular tiles, packed in the workspace
      float g, gc, b;
      float fq[RowTile::IT], nk[RowTile::IT];  // factors of the token each of this thread's Q / K vectors belongs to
      int len;
    };
    Tiles ta, tb;
    ta.g = ta.gc = ta.b = tb.g = tb.gc = tb.b = 0.f;
    ta.Tm.init(LDC, mt), ta.P.init(LDC, mt), tb.Tm.init(LDC, mt), tb.P.init(LDC, mt);
    zero_upper_triangles(sTm, 4, L::kC, LDC, mt);  // both buffers of Tm and Pm: the packed tiles never write there
    ta.len = tb.len = 0;
#pragma unroll
    for (int it = 0; it < RowTile::IT; ++it) ta.fq[it] = tb.fq[it] = ta.nk[it] = tb.nk[it] = 0.f;
    auto fetch = [&](Tiles& R, int n, int part = -1) {  // part 0: K, 1: Q, 2: the rest; < 0: everything
      const int64_t slot = (int64_t)row * N + n;
      int tok0;
      chunk_span(span, n, tok0, R.len);
      const int64_t tbase = tok_index(p.geom, row, tok0);
      if (part < 0 || part == 0) R.K.load(p.k + tbase * DK, tsk, R.len, mt);
      if (part < 0 || part == 1) R.Q.load(p.q + tbase * DK, tsk, R.len, mt);
      if (part == 0 || part == 1) return;
      R.dO.load(p.d_o + tbase * p.dv + v0, tsv, R.len, mt);
      R.Tm.load(at<const T>(p.ws, p.off.Tm) + slot * 64 * 64, mt);
      R.P.load(at<const T>(p.ws, p.off.P) + slot * 64 * 64, mt);
      const int t = mt & 63;
      if (GATE == LNX_GATE_SCALAR) {
        const float* G = at<const float>(p.ws, p.off.G) + slot * 64;
        R.g = G[t];
        R.gc = G[63];
      }
#pragma unroll
      for (int it = 0; it < RowTile::IT; ++it) {
        R.fq[it] = at<const float>(p.ws, p.off.Fq)[slot * 64 + (mt + 256 * it) / RowTile::VPR];
        R.nk[it] = at<const float>(p.ws, p.off.Nk)[slot * 64 + (mt + 256 * it) / RowTile::VPR];
      }
      R.b = p.beta[tbase + (int64_t)min(t, R.len - 1) * p.geom.ts];
    };
    auto commit = [&](const Tiles& R, int pb, int part = -1) {
      {  // K rows normalised; Q rows normalised and scaled by scale e^{G_i}: (scale diag(e^G) Q)^T dO needs no scaled copy of dO
        T* dstk = sK + pb * L::kK;
        T* dst = sQ + pb * L::kK;
#pragma unroll
        for (int it = 0; it < RowTile::IT; ++it) {
          const int idx = mt + 256 * it, r = idx / RowTile::VPR, c = (idx - r * RowTile::VPR) * RowTile::N;
          if (part < 0 || part == 0) {
            typename Vec16<T>::V y = R.K.x[it];
#pragma unroll
            for (int e = 0; e < RowTile::N; ++e) y[e] = (bf16_t)((float)y[e] * R.nk[it]);
            *reinterpret_cast<typename Vec16<T>::V*>(dstk + r * LDK + c) = y;
          }
          if (part < 0 || part == 1) {
            typename Vec16<T>::V x = R.Q.x[it];
#pragma unroll
            for (int e = 0; e < RowTile::N; ++e) x[e] = (bf16_t)((float)x[e] * R.fq[it]);
            *reinterpret_cast<typename Vec16<T>::V*>(dst + r * LDK + c) = x;
          }
        }
      }
      if (part == 0 || part == 1) return;
      R.dO.store(sdO + pb * L::kV, LDV, mt);
      R.Tm.store(sTm + pb * L::kC);
      R.P.store(sP + pb * L::kC);
      if (mt < 64) {
        float* sc = sSc + pb * Scal::SIZE;
        const float gam = (GATE == LNX_GATE_SCALAR) ? __expf(R.g) : 1.f;
        const float bt = (mt < R.len) ? R.b : 0.f;
        sc[Scal::BETA + mt] = bt;
        sc[Scal::GAM + mt] = bt * gam;  // beta e^G: dY = -(beta e^G) dR
        sc[Scal::R + mt] = (GATE == LNX_GATE_SCALAR) ? __expf(fminf(R.gc - R.g, 0.f)) : 1.f;
        if (mt == 0) sc[Scal::DEC] = (GATE == LNX_GATE_SCALAR) ? __expf(R.gc) : 1.f;
      }
    };
    // cur: the register set that held chunk n and now takes chunk n - 2; nxt: chunk n - 1 (see scan_fwd)
    auto step = [&](Tiles& cur, const Tiles& nxt, int n, auto steady) {
      constexpr bool STEADY = decltype(steady)::value;
      const int pbn = (c1 - n) & 1;  // position of chunk n - 1 from the end: c1 - 1 - (n - 1)
      if constexpr (STEADY) {  // tile writes between the loads, a tile at a time (see scan_fwd)
#pragma unroll
        for (int part = 0; part < 3; ++part) {
          fetch(cur, n - 2, part);
          commit(nxt, pbn, part);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        if (n - 2 >= c0) fetch(cur, n - 2);
        if (n - 1 >= c0) commit(nxt, pbn);
      }
      lds_barrier();  // Bmid
      const int64_t slot = (int64_t)row * N + n;
      unstage_tile<T, BV, DK, true>(at<T>(p.ws, p.off.dSn) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sdST, LDK, BV, mt);
      unstage_tile<T, BV, 64, true>(at<T>(p.ws, p.off.dD) + slot * p.dv * 64 + (int64_t)v0 * 64, 64, sdRT, LDC, BV, mt);
      int tok0, len;
      chunk_span(span, n, tok0, len);
      unstage_tile_checked<T, 64, BV>(p.dv_out + tok_index(p.geom, row, tok0) * p.dv + v0, tsv, sdV, LDV, len, mt);
      lds_barrier();  // B1 of the next chunk
    };
    if (c0 < c1) {
      fetch(ta, c1 - 1);
      commit(ta, 0);
    }
    if (c1 - 2 >= c0) fetch(tb, c1 - 2);
    lds_barrier();  // B1 of the first chunk
    int n = c1 - 1;
    for (; n - 3 >= c0; n -= 2) {  // chunks n - 2 and n - 3 exist
      step(ta, tb, n, std::true_type{});
      step(tb, ta, n - 1, std::true_type{});
    }
    for (; n >= c0; n -= 2) {
      step(ta, tb, n, std::false_type{});
      if (n - 1 >= c0) step(tb, ta, n - 1, std::false_type{});
    }
    return;
  }

  // ---------------- compute waves ----------------
  const int vs = 32 * wave;
  const int fr = lane & 31;
  floatx16 dS[KT];
#pragma unroll
  for (int ci = 0; ci < KT; ++ci)
#pragma unroll
    for (int e = 0; e < 16; ++e) dS[ci][e] = 0.f;
  if (p.d_sT) {
    const float* src = p.d_sT + (int64_t)sidx * DK * p.dv + v0 + vs;
#pragma unroll
    for (int ci = 0; ci < KT; ++ci)
#pragma unroll
      for (int e = 0; e < 16; ++e) dS[ci][e] = src[(int64_t)(32 * ci + frag_row(e, lane)) * p.dv + frag_col(lane)];
  }
  lds_barrier();  // B1 of the first chunk
  // LDS reads are issued ahead of the products that consume them, as in scan_fwd.  The products that do not depend on
  // the incoming dS' (Pm^T dO, Q~^T dO) fill the gaps of the chain  dS' -> Z -> dD -> dR -> dY -> dS.
  constexpr int NK = DK / 16;
  for (int n = c1 - 1; n >= c0; --n) {
    const int pb = (c1 - 1 - n) & 1;
    const T* sKc = sK + pb * L::kK;
    const T* sQc = sQ + pb * L::kK;
    const T* sOc = sdO + pb * L::kV;
    const T* sTc = sTm + pb * L::kC;
    const T* sPc = sP + pb * L::kC;
    const float* sc = sSc + pb * Scal::SIZE;
    M::Frag fa[3][2], fp[2][2], fo[2];
    floatx4 sv[2][4];  // per-row scalars at this lane's accumulator positions: e^{G_C - G}, later beta e^G
#pragma unroll
    for (int s_ = 0; s_ < 2; ++s_)
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[s_][i] = M::load_chain(sKc + (32 * i + fr) * LDK + 16 * s_, lane);
    fp[0][0] = M::load_t(sPc, LDC, 0, 0, lane);  // Pm^T and Tm^T are upper-triangular: row tile 1 takes steps 2, 3 only
    fo[0] = M::load_t(sOc, LDV, 0, vs, lane);
    // the state gradient as the B operand of Z = K dS'; its accumulators are then free to take the next dS
    M::Frag bs[NK];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) bs[ks] = M::from_acc(dS[ks >> 1], ks & 1);
#pragma unroll
    for (int ci = 0; ci < KT; ++ci) store_frag_t(dS[ci], sdST + vs * LDK + 32 * ci, LDK, lane);
    const float dec = (GATE == LNX_GATE_SCALAR) ? sc[Scal::DEC] : 1.f;
    __builtin_amdgcn_sched_barrier(0);
    // ---- Z = K dS' and the chunk-local part Pm^T dO ----
    floatx16 z[2], dd[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) z[i][e] = dd[i][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      if (ks + 2 < NK) {
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[(ks + 2) % 3][i] = M::load_chain(sKc + (32 * i + fr) * LDK + 16 * (ks + 2), lane);
      }
      if (ks + 1 < 4) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          if (i == 0 || ks + 1 >= 2) fp[(ks + 1) & 1][i] = M::load_t(sPc, LDC, 16 * (ks + 1), 32 * i, lane);
        fo[(ks + 1) & 1] = M::load_t(sOc, LDV, 16 * (ks + 1), vs, lane);
      }
      if (ks == NK - 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) sv[i][q] = load4(sc + Scal::R + 32 * i + 8 * q + 4 * (lane >> 5));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) M::mma(z[i], fa[ks % 3][i], bs[ks]);
      if (ks < 4) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          if (i == 0 || ks >= 2) M::mma(dd[i], fp[ks & 1][i], fo[ks & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // first fragments of Tm^T, and of the (scale e^G Q)^T dO product that fills the wait for Z
    M::Frag fq[2][KT];
#pragma unroll
    for (int s_ = 0; s_ < 2; ++s_) fa[s_][0] = M::load_t_chain(sTc, LDC, 16 * s_, 0, lane);
#pragma unroll
    for (int ci = 0; ci < KT; ++ci) fq[0][ci] = M::load_t(sQc, LDK, 0, 32 * ci, lane);
    fo[0] = M::load_t(sOc, LDV, 0, vs, lane);
    if (GATE == LNX_GATE_SCALAR) {
#pragma unroll
      for (int ci = 0; ci < KT; ++ci)
#pragma unroll
        for (int e = 0; e < 16; ++e) dS[ci][e] *= dec;
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- dS <- e^{G_C} dS' + (scale e^G Q)^T dO ----
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) {
#pragma unroll
        for (int ci = 0; ci < KT; ++ci) fq[(ks + 1) & 1][ci] = M::load_t(sQc, LDK, 16 * (ks + 1), 32 * ci, lane);
        fo[(ks + 1) & 1] = M::load_t(sOc, LDV, 16 * (ks + 1), vs, lane);
      }
#pragma unroll
      for (int ci = 0; ci < KT; ++ci) M::mma(dS[ci], fq[ks & 1][ci], fo[ks & 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- dD = Pm^T dO + e^{G_C - G} Z ----
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int u = 0; u < 4; ++u) dd[i][4 * q + u] += sv[i][q][u] * z[i][4 * q + u];
    M::Frag bd[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bd[ks] = M::from_acc(dd[ks >> 1], ks & 1);
    __builtin_amdgcn_sched_barrier(0);
    // ---- dR = Tm^T dD (lane = value column, in z) and once more with the operands exchanged (lane = token, in dd), which
    //      is the orientation dv = beta dR leaves in ----
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) z[i][e] = dd[i][e] = 0.f;
    M::Frag fu[2][KT];  // K^T fragments of the dS update
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 2 < 4) {
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[(ks + 2) % 3][i] = M::load_t_chain(sTc, LDC, 16 * (ks + 2), 32 * i, lane);
      } else if (ks == 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) sv[i][q] = load4(sc + Scal::GAM + 32 * i + 8 * q + 4 * (lane >> 5));
      } else {
#pragma unroll
        for (int ci = 0; ci < KT; ++ci) fu[0][ci] = M::load_t_chain(sKc, LDK, 0, 32 * ci, lane);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (i == 0 || ks >= 2) M::mma(z[i], fa[ks % 3][i], bd[ks]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (i == 0 || ks >= 2) M::mma(dd[i], bd[ks], fa[ks % 3][i]);
      __builtin_amdgcn_sched_barrier(0);
    }
    const float bl0 = sc[Scal::BETA + fr], bl1 = sc[Scal::BETA + 32 + fr];
#pragma unroll
    for (int i = 0; i < 2; ++i) store_frag_t(z[i], sdRT + vs * LDC + 32 * i, LDC, lane);
    // dY = -beta e^G dR
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int u = 0; u < 4; ++u) z[i][4 * q + u] *= -sv[i][q][u];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bd[ks] = M::from_acc(z[ks >> 1], ks & 1);
    __builtin_amdgcn_sched_barrier(0);
    // dv = beta dR: fragment dd[i] holds tokens 32 i .. (one per lane) x the strip's value columns
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dd[0][e] *= bl0;
      dd[1][e] *= bl1;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) store_frag_t(dd[i], sdV + 32 * i * LDV + vs, LDV, lane);
    lds_barrier();  // Bmid
    // ---- dS += K^T dY ----
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) {
#pragma unroll
        for (int ci = 0; ci < KT; ++ci) fu[(ks + 1) & 1][ci] = M::load_t_chain(sKc, LDK, 16 * (ks + 1), 32 * ci, lane);
      }
#pragma unroll
      for (int ci = 0; ci < KT; ++ci) M::mma(dS[ci], fu[ks & 1][ci], bd[ks]);
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();  // B1 of the next chunk
  }
  if (p.ds0) {
    float* out = p.ds0 + (int64_t)sidx * DK * p.dv + v0 + vs + frag_col(lane);
#pragma unroll
    for (int ci = 0; ci < KT; ++ci)
#pragma unroll
      for (int e = 0; e < 16; ++e) out[(int64_t)(32 * ci + frag_row(e, lane)) * p.dv] = dS[ci][e];
  }
}

template <int DK, int GATE>
int launch_scan_bwd(const DirectParams& p, int nstate, hipStream_t st) {
  const bool narrow = lnx_narrow_slabs((int64_t)nstate * p.geom.H * (p.dv / 64), p.slab);
  auto k = narrow ? scan_bwd_kernel<DK, GATE, 32> : scan_bwd_kernel<DK, GATE, 64>;
  const size_t b = narrow ? BScanL<DK, 32>::bytes : BScanL<DK, 64>::bytes;
  const int bv = narrow ? 32 : 64, threads = narrow ? BScanL<DK, 32>::threads : BScanL<DK, 64>::threads;
  hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b);
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  lnx_profile_mark("bwd_scan", st);
  hipLaunchKernelGGL(k, dim3(lnx_xcd_grid((int64_t)nstate * p.geom.H, p.dv / bv)), dim3(threads), b, st, p);
  return LNX_OK;
}

// ---------------------------------------------------------------------------------------
// bwd_chunk: the chunk-local gradients, one workgroup per chunk, all chunks in parallel.  Reads q, k, v, dO of the
// chunk, the states S (entering) and dS' (leaving) and D, dR from the two scans; writes dq, dk, dbeta, dg (dv left
// the reverse scan).  A loop over 32-column slabs of the value dimension accumulates every product that contracts
// over value columns; the slabs arrive in two LDS buffers through loads that bypass the registers, two slabs ahead:
//   dQa = dO S^T     dK1 = dR S^T     dK2 = D dS'^T     dPm = dO D^T     dAm = dR D^T     <dR_t, v_t>     <dS', S>
// then an epilogue over the chunk's tokens:
//   dPe = scale tril(E * dPm)          dXa = -tril(E * dAm, -1)          dXe = diag(beta) dXa
//   dq  = scale e^G dQa + dPe K
//   row = dXa K - e^G dK1              m_t = <k_t, row_t>                 dbeta = <dR, v> + m
//   dk  = beta row + e^{G_C - G} dK2 + dPe^T Q + dXe^T K
//   dG  = <q, dq> - <k, dk> + 2 beta m;   dG_C += sum_t e^{G_C - G_t} <k_t, dK2_t> + e^{G_C} <dS', S>;   dg = reverse cumsum(dG)
// Wave (wi, wj) owns the token-row tile wi and the key-column tiles NKT wj .. of the [64 x dk] accumulators and the
// (wi, wj) tile of the [64 x 64] ones.  The epilogue's tiles that are only read through transposing LDS loads get a row
// stride of 64 bytes mod 256, which spreads the four rows that half a wave reads over all banks.
// Measured per workgroup at B8 H16 T4096 d128 (wall clock of wave 0, 2 workgroups per CU): 4.3 us until the first slab
// is there, 6.2 us for the loop, 2.1 us staging K, Q and the four small tiles, 1.8 us for the epilogue's products and
// 3.4 us until dq, dk have left -- memory latency at every step; the kernel moves 4.9 TB/s.
// ---------------------------------------------------------------------------------------
template <int DK> struct BChunkL {
  static constexpr int SV = 32;
  typedef SwzTile<64, SV> TokT;            // dO, V slabs [64][SV], read by rows
  typedef SwzTile<SV, 64, false> TrT;      // D^T, dR^T slabs [SV][64], transposing reads only
  typedef SwzTile<SV, DK, false> StT;      // S^T, dS'^T slabs [SV][DK], transposing reads only
  static constexpr int LDKT = DK + 32;     // the epilogue's K, Q tiles [64][DK], transposing reads
  static constexpr int LDC = 64 + 8;       // dPe, dPe^T, dXa, dXe^T [64][64], read by rows
  static constexpr int LDK = DK + 8;       // staging tile for dq, dk [64][DK]
  static constexpr int kC = 64 * LDC, kRow = 64 * LDKT;
  // one slab of the loop: dO | V | D^T | dR^T | S^T | dS'^T, unpadded; two of them, filled by LDS-direct loads in turn
  static constexpr int oV = TokT::BYTES, oDT = 2 * TokT::BYTES, odRT = oDT + TrT::BYTES, oSn = odRT + TrT::BYTES, odSn = oSn + StT::BYTES;
  static constexpr int slab_bytes = odSn + StT::BYTES;
  static constexpr size_t loop_bytes = 2 * slab_bytes;
  static constexpr size_t epi_bytes = sizeof(T) * (2 * kRow + 4 * kC);
  static_assert(64 * LDK <= 2 * kC, "the staging tile overlays dPe and dPe^T");
  static constexpr int nfloat = 64 * 8;
  static constexpr size_t bytes = sizeof(float) * nfloat + (epi_bytes > loop_bytes ? epi_bytes : loop_bytes);
  static_assert(bytes <= 80 * 1024, "two workgroups per CU");
};

template <int DK, int GATE>
__global__ __launch_bounds__(256, 2) void bwd_chunk_kernel(DirectParams p) {
  typedef BChunkL<DK> L;
  constexpr int SV = L::SV, LDKT = L::LDKT, LDC = L::LDC, LDK = L::LDK;
  typedef typename L::TokT TokT;
  typedef typename L::TrT TrT;
  typedef typename L::StT StT;
  constexpr int NKT = DK / 64;  // key-column tiles per wave
  extern __shared__ __align__(16) char smem[];
  float* sG = reinterpret_cast<float*>(smem);
  float* sBeta = sG + 64;
  float* sRdv = sBeta + 64;   // <dR_t, v_t>
  float* sM = sRdv + 64;      // m_t
  float* sdG = sM + 64;
  float* sMisc = sdG + 64;    // [4 + wave] = the wave's share of sum_t r_t <k_t, dK2_t>, [8 + wave] = of <dS', S>
  float* sNq = sMisc + 64;    // normalisation factors of the q and k rows (1 when the inputs come normalised)
  float* sNk = sNq + 64;
  T* tiles = reinterpret_cast<T*>(smem + sizeof(float) * L::nfloat);
  char* sSlab = reinterpret_cast<char*>(tiles);  // [2][slab_bytes]
  // epilogue
  T* sPe = tiles;             // [i][j]
  T* sPeT = sPe + L::kC;      // [j][i]
  T* sXa = sPeT + L::kC;      // [i][j]
  T* sXeT = sXa + L::kC;      // [j][i]
  T* sK = sXeT + L::kC;       // [token][dk]
  T* sQ = sK + L::kRow;
  T* sSt = tiles;             // staging for dq (over dPe, dPe^T) and dk (over dXa, dXe^T), once the four small tiles are dead
  T* sSt2 = sXa;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  const int64_t slot = blockIdx.x;
  const int row = (int)(slot / N), n = (int)(slot % N);
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  if (len <= 0) return;
  const int64_t tbase = tok_index(p.geom, row, tok0);
  const int64_t ts = p.geom.ts, tsk = ts * DK, tsv = ts * p.dv;
  const int wi = wave >> 1, wj = wave & 1;
  const int fr = lane & 31, kg8 = 8 * (lane >> 5);

  TileRegs<T, 64, DK> rK, rQ;  // the epilogue's tiles, requested during the last slab
  floatx16 aP[1][1], aA[1][1], aQ[1][NKT], aK1[1][NKT], aK2[1][NKT];
  frag_zero(aP);
  frag_zero(aA);
  frag_zero(aQ);
  frag_zero(aK1);
  frag_zero(aK2);
  float ss = 0.f, rdv = 0.f;
  if (tid < 64) {
    sG[tid] = (GATE == LNX_GATE_SCALAR) ? at<const float>(p.ws, p.off.G)[slot * 64 + tid] : 0.f;
    sBeta[tid] = (tid < len) ? p.beta[tbase + tid * ts] : 0.f;
    sM[tid] = 0.f;
    sMisc[tid] = 0.f;
    sNq[tid] = at<const float>(p.ws, p.off.Nq)[slot * 64 + tid];
    sNk[tid] = at<const float>(p.ws, p.off.Nk)[slot * 64 + tid];
  }
  // ---- the slab loads: 32 one-KB instructions per slab, eight per wave, straight into LDS buffer `b` ----
  // Token rows past the chunk's end fetch the chunk's last row instead of zeros: whatever they hold only reaches rows of
  // dq, dk, dbeta, dg that are not stored (q, k and beta of those rows are zero).
  const unsigned slab0 = lds_byte_addr(sSlab);
  const T* gSn = at<const T>(p.ws, p.off.SnT) + slot * p.dv * DK;
  const T* gdSn = at<const T>(p.ws, p.off.dSn) + slot * p.dv * DK;
  const T* gDT = at<const T>(p.ws, p.off.D) + slot * p.dv * 64;
  const T* gdRT = at<const T>(p.ws, p.off.dD) + slot * p.dv * 64;
  const T* gdO = p.d_o + tbase * p.dv;
  const T* gV = p.v + tbase * p.dv;
  auto issue = [&](int v0, int b) {
    const unsigned dst = slab0 + b * L::slab_bytes;
    int r, c;
    // wave w: instructions w, w + 4, ... of each tile
#pragma unroll
    for (int j = wave; j < StT::NINSTR; j += 4) {
      StT::src(j, lane, r, c);
      dma16(gSn + (int64_t)(v0 + r) * DK + c, dst + L::oSn + 1024 * j);
      dma16(gdSn + (int64_t)(v0 + r) * DK + c, dst + L::odSn + 1024 * j);
    }
#pragma unroll
    for (int j = wave; j < TokT::NINSTR; j += 4) {
      TokT::src(j, lane, r, c);
      r = min(r, len - 1);
      dma16(gdO + (int64_t)r * tsv + v0 + c, dst + 1024 * j);
      dma16(gV + (int64_t)r * tsv + v0 + c, dst + L::oV + 1024 * j);
    }
#pragma unroll
    for (int j = wave; j < TrT::NINSTR; j += 4) {
      TrT::src(j, lane, r, c);
      dma16(gDT + (int64_t)(v0 + r) * 64 + c, dst + L::oDT + 1024 * j);
      dma16(gdRT + (int64_t)(v0 + r) * 64 + c, dst + L::odRT + 1024 * j);
    }
  };
  constexpr int PER_WAVE = (2 * StT::NINSTR + 2 * TokT::NINSTR + 2 * TrT::NINSTR) / 4;  // loads per wave and slab
  static_assert(StT::NINSTR % 4 == 0 && TokT::NINSTR % 4 == 0 && TrT::NINSTR % 4 == 0, "the same count for every wave");
  __builtin_amdgcn_s_waitcnt(0);  // the small loads above are behind us: from here on this wave's vmcnt counts slab loads only
  issue(0, 0);
  if (SV < p.dv) issue(SV, 1);
  int b = 0;
#pragma unroll 1
  for (int v0 = 0; v0 < p.dv; v0 += SV, b ^= 1) {
    // this slab has landed: all but the next slab's loads of this wave, then every wave's
    if (v0 + SV < p.dv) dma_wait<PER_WAVE>();
    else dma_wait<0>();
    lds_barrier();
    const T* sdO = reinterpret_cast<const T*>(sSlab + b * L::slab_bytes);
    const T* sV = reinterpret_cast<const T*>(sSlab + b * L::slab_bytes + L::oV);
    const T* sDT = reinterpret_cast<const T*>(sSlab + b * L::slab_bytes + L::oDT);
    const T* sdRT = reinterpret_cast<const T*>(sSlab + b * L::slab_bytes + L::odRT);
    const T* sSn = reinterpret_cast<const T*>(sSlab + b * L::slab_bytes + L::oSn);
    const T* sdSn = reinterpret_cast<const T*>(sSlab + b * L::slab_bytes + L::odSn);
    static_assert(SV == 32, "two 16-wide steps per slab");
    if (v0 + SV >= p.dv) {  // last slab: the epilogue's K and Q tiles (a slab earlier gains nothing)
      rK.load(p.k + tbase * DK, tsk, len, tid);
      rQ.load(p.q + tbase * DK, tsk, len, tid);
    }
#pragma unroll
    for (int k0 = 0; k0 < SV; k0 += 16) {
      const M::Frag fdO = TokT::load(sdO, 32 * wi + fr, k0 + kg8);
      const M::Frag fdR = TrT::load_t(sdRT, k0, 32 * wi, lane);
      const M::Frag fDi = TrT::load_t(sDT, k0, 32 * wi, lane);
      const M::Frag fDj = TrT::load_t(sDT, k0, 32 * wj, lane);
      M::mma(aP[0][0], fdO, fDj);
      M::mma(aA[0][0], fdR, fDj);
#pragma unroll
      for (int c = 0; c < NKT; ++c) {
        const M::Frag fS = StT::load_t(sSn, k0, 32 * (NKT * wj + c), lane);
        const M::Frag fdS = StT::load_t(sdSn, k0, 32 * (NKT * wj + c), lane);
        M::mma(aQ[0][c], fdO, fS);
        M::mma(aK1[0][c], fdR, fS);
        M::mma(aK2[0][c], fDi, fdS);
      }
    }
    {  // <dR_t, v_t> over this slab: thread = (token tid / 4, eight value columns)
      const int t = tid >> 2, c0 = 8 * (tid & 3);
      const M::Frag vv = TokT::load(sV, t, c0);
#pragma unroll
      for (int e = 0; e < 8; ++e) rdv += (float)vv[e] * (float)sdRT[TrT::at(c0 + e, t)];
    }
    if (GATE == LNX_GATE_SCALAR) {  // <dS', S> over this slab: the two tiles share one layout, so granule by granule
#pragma unroll
      for (int u = 0; u < StT::BYTES / 16 / 256; ++u) {
        const M::Frag a = *reinterpret_cast<const M::Frag*>(sSn + 8 * (tid + 256 * u));
        const M::Frag b2 = *reinterpret_cast<const M::Frag*>(sdSn + 8 * (tid + 256 * u));
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += (float)a[e] * (float)b2[e];
      }
    }
    if (v0 + 2 * SV < p.dv) {  // this buffer takes the slab after the next, once every wave has read it
      lds_barrier();
      issue(v0 + 2 * SV, b);
    }
  }
  rdv += __shfl_xor(rdv, 1, LNX_WAVE);
  rdv += __shfl_xor(rdv, 2, LNX_WAVE);
  if ((tid & 3) == 0) sRdv[tid >> 2] = rdv;
  if (GATE == LNX_GATE_SCALAR) {
    ss = wave_sum(ss);
    if (lane == 0) sMisc[8 + wave] = ss;  // one slot per wave, added in a fixed order below
  }
  lds_barrier();  // slab tiles are dead from here on

  // ---- epilogue ----
  {  // K and Q rows, normalised
    typedef TileRegs<T, 64, DK> RowTile;
#pragma unroll
    for (int it = 0; it < RowTile::IT; ++it) {
      const int idx = tid + 256 * it, r = idx / RowTile::VPR, c = (idx - r * RowTile::VPR) * RowTile::N;
      const float fk = sNk[r], fq = sNq[r];
      typename Vec16<T>::V x = rK.x[it], y = rQ.x[it];
#pragma unroll
      for (int e = 0; e < RowTile::N; ++e) x[e] = (bf16_t)((float)x[e] * fk), y[e] = (bf16_t)((float)y[e] * fq);
      *reinterpret_cast<typename Vec16<T>::V*>(sK + r * LDKT + c) = x;
      *reinterpret_cast<typename Vec16<T>::V*>(sQ + r * LDKT + c) = y;
    }
  }
  // The cumulative gate and beta of this lane's sixteen accumulator rows (four runs of four), as vectors and once: read one
  // by one between the tile stores below, each read would wait out its own round trip to LDS (the stores might alias it).
  floatx4 gi[4], bi[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int i0 = 32 * wi + 8 * q + 4 * (lane >> 5);
    gi[q] = load4(sG + i0);
    bi[q] = load4(sBeta + i0);
  }
  const float gC = sG[63];
  {
    floatx16 pe[1][1];
    const int j = 32 * wj + frag_col(lane);
    const float gj = sG[j];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = 32 * wi + frag_row(e, lane);
      const float dec = (GATE == LNX_GATE_NONE) ? 1.f : __expf(fminf(gi[e >> 2][e & 3] - gj, 0.f));
      pe[0][0][e] = (i >= j) ? p.scale * dec * aP[0][0][e] : 0.f;
      aA[0][0][e] = (i > j) ? -dec * aA[0][0][e] : 0.f;  // dXa
    }
    frag_store<T, 1, 1>(pe, sPe + 32 * wi * LDC + 32 * wj, LDC, lane);
    frag_store_t<T, 1, 1>(pe, sPeT + 32 * wj * LDC + 32 * wi, LDC, lane);
    frag_store<T, 1, 1>(aA, sXa + 32 * wi * LDC + 32 * wj, LDC, lane);
#pragma unroll
    for (int e = 0; e < 16; ++e) aA[0][0][e] *= bi[e >> 2][e & 3];  // dXe
    frag_store_t<T, 1, 1>(aA, sXeT + 32 * wj * LDC + 32 * wi, LDC, lane);
  }
  lds_barrier();
  // dq = scale e^G dQa + dPe K;   row = dXa K - e^G dK1 (in aK1)
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const float gm = (GATE == LNX_GATE_NONE) ? 1.f : __expf(gi[e >> 2][e & 3]);
#pragma unroll
    for (int c = 0; c < NKT; ++c) {
      aQ[0][c][e] *= p.scale * gm;
      aK1[0][c][e] *= -gm;
    }
  }
#pragma unroll
  for (int k0 = 0; k0 < 64; k0 += 16) {
    const M::Frag fPe = M::load(sPe + (32 * wi + fr) * LDC + k0 + kg8);
    const M::Frag fXa = M::load(sXa + (32 * wi + fr) * LDC + k0 + kg8);
#pragma unroll
    for (int c = 0; c < NKT; ++c) {
      const M::Frag fK = M::load_t(sK, LDKT, k0, 32 * (NKT * wj + c), lane);
      M::mma(aQ[0][c], fPe, fK);
      M::mma(aK1[0][c], fXa, fK);
    }
  }
  // m_t = <k_t, row_t>;  chunk-end gate term sum_t r_t <k_t, dK2_t>;  dk <- beta row + r dK2 (in aK2)
  {
    float mv[16], tot = 0.f;
    floatx4 kq[NKT][4];  // K at this lane's accumulator positions, one transposing read per run of four rows
#pragma unroll
    for (int c = 0; c < NKT; ++c)
#pragma unroll
      for (int q = 0; q < 4; ++q) kq[c][q] = M::load_acc_rows(sK, LDKT, 32 * wi, q, 32 * (NKT * wj + c), lane);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float rr = (GATE == LNX_GATE_NONE) ? 1.f : __expf(fminf(gC - gi[e >> 2][e & 3], 0.f));
      const float bt = bi[e >> 2][e & 3];
      mv[e] = 0.f;
#pragma unroll
      for (int c = 0; c < NKT; ++c) {
        const float kk = kq[c][e >> 2][e & 3];
        mv[e] += kk * aK1[0][c][e];
        aK2[0][c][e] *= rr;
        tot += kk * aK2[0][c][e];
        aK2[0][c][e] += bt * aK1[0][c][e];
      }
    }
    rows_reduce_add<1>(mv, 32 * wi, lane, sM);  // two waves (wj = 0, 1) add to a zeroed entry: order-independent
    if (GATE == LNX_GATE_SCALAR) {
      tot = wave_sum(tot);
      if (lane == 0) sMisc[4 + wave] = tot;
    }
  }
  // dk += dPe^T Q + dXe^T K
#pragma unroll
  for (int k0 = 0; k0 < 64; k0 += 16) {
    const M::Frag fPt = M::load(sPeT + (32 * wi + fr) * LDC + k0 + kg8);
    const M::Frag fXt = M::load(sXeT + (32 * wi + fr) * LDC + k0 + kg8);
#pragma unroll
    for (int c = 0; c < NKT; ++c) {
      M::mma(aK2[0][c], fPt, M::load_t(sQ, LDKT, k0, 32 * (NKT * wj + c), lane));
      M::mma(aK2[0][c], fXt, M::load_t(sK, LDKT, k0, 32 * (NKT * wj + c), lane));
    }
  }
  lds_barrier();  // the four small tiles are dead; sM and sMisc are complete
  // dq and dk through their staging tiles.  Thread = (token tid / 4, the 8-column groups tid % 4, tid % 4 + 4, ...): the
  // row dots <q_t, dq_t> and <k_t, dk_t> give the gate gradient and carry the gradients through the normalisation,
  //   d/dx of x / (|x| + eps) applied to dy:  dy / (|x| + eps) - y <y, dy> / |x|.
  const int tr = tid >> 2, tq = 8 * (tid & 3);
  float dgp = 0.f;
  auto emit = [&](const T* sSt, const T* sIn, float fac, T* out, float sign) {
    float dot = 0.f;
#pragma unroll
    for (int u = 0; u < DK; u += 32) {
      const M::Frag a = M::load(sSt + tr * LDK + tq + u), b = M::load(sIn + tr * LDKT + tq + u);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += (float)a[e] * (float)b[e];
    }
    dot = quad_sum(dot);
    dgp += sign * dot;
    const float nrm = 1.f / fac - LNX_L2_EPS;
    const float cf = (p.l2norm && nrm > 0.f) ? dot / nrm : 0.f;
    if (tr < len) {
#pragma unroll
      for (int u = 0; u < DK; u += 32) {
        M::Frag a = M::load(sSt + tr * LDK + tq + u);
        const M::Frag b = M::load(sIn + tr * LDKT + tq + u);
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = (bf16_t)(fac * (float)a[e] - cf * (float)b[e]);
        *reinterpret_cast<M::Frag*>(out + tbase * DK + (int64_t)tr * tsk + tq + u) = a;
      }
    }
  };
  frag_store<T, 1, NKT>(aQ, sSt + 32 * wi * LDK + 32 * NKT * wj, LDK, lane);
  frag_store<T, 1, NKT>(aK2, sSt2 + 32 * wi * LDK + 32 * NKT * wj, LDK, lane);
  lds_barrier();
  emit(sSt, sQ, sNq[tr], p.dq, 1.f);
  emit(sSt2, sK, sNk[tr], p.dk, -1.f);
  if (GATE == LNX_GATE_SCALAR) {
    if ((tid & 3) == 0) {
      float d = dgp + 2.f * sBeta[tr] * sM[tr];
      if (tr == 63) d += ((sMisc[4] + sMisc[5]) + (sMisc[6] + sMisc[7])) + __expf(gC) * ((sMisc[8] + sMisc[9]) + (sMisc[10] + sMisc[11]));
      sdG[tr] = d;
    }
    lds_barrier();
  }
  if (wave == 0) {
    const int t = lane;
    if (t < len) p.dbeta[tbase + t * ts] = sRdv[t] + sM[t];
    if (GATE == LNX_GATE_SCALAR) {  // dg = reverse cumulative sum of dG over the chunk
      float d = sdG[t];
#pragma unroll
      for (int s_ = 1; s_ < 64; s_ <<= 1) {
        const float y = __shfl_down(d, s_, LNX_WAVE);
        if (t + s_ < 64) d += y;
      }
      if (t < len) p.dg[tbase + t * ts] = d;
    }
  }
}

template <int DK, int GATE>
int launch_bwd_chunk(const DirectParams& p, hipStream_t st) {
  auto k = bwd_chunk_kernel<DK, GATE>;
  const size_t b = BChunkL<DK>::bytes;
  hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b);
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  lnx_profile_mark("bwd_chunk", st);
  hipLaunchKernelGGL(k, dim3((unsigned)((int64_t)p.geom.rows * p.geom.N)), dim3(256), b, st, p);
  lnx_profile_mark(nullptr, st);
  return LNX_OK;
}

template <int DK, int GATE>
int launch_bwd(const DirectParams& p, int nstate, hipStream_t st) {
  int rc = launch_scan_bwd<DK, GATE>(p, nstate, st);
  if (rc != LNX_OK) return rc;
  return launch_bwd_chunk<DK, GATE>(p, st);
}

}  // namespace

namespace {
template <typename OT>
int scan_fwd_by_shape(const DirectParams& p, int dk, int gate, int nstate, hipStream_t st) {
  if (dk == 128)
    return gate == LNX_GATE_SCALAR ? launch_scan_fwd<128, LNX_GATE_SCALAR, OT>(p, nstate, st) : launch_scan_fwd<128, LNX_GATE_NONE, OT>(p, nstate, st);
  return gate == LNX_GATE_SCALAR ? launch_scan_fwd<64, LNX_GATE_SCALAR, OT>(p, nstate, st) : launch_scan_fwd<64, LNX_GATE_NONE, OT>(p, nstate, st);
}
}  // namespace

int lnx_direct_scan_fwd(const DirectParams& p, int dk, int gate, int nstate, hipStream_t st) {
  return p.o_dtype == LNX_F32 ? scan_fwd_by_shape<float>(p, dk, gate, nstate, st) : scan_fwd_by_shape<bf16_t>(p, dk, gate, nstate, st);
}

int lnx_direct_bwd(const DirectParams& p, int dk, int gate, int nstate, hipStream_t st) {
  if (dk == 128)
    return gate == LNX_GATE_SCALAR ? launch_bwd<128, LNX_GATE_SCALAR>(p, nstate, st) : launch_bwd<128, LNX_GATE_NONE>(p, nstate, st);
  return gate == LNX_GATE_SCALAR ? launch_bwd<64, LNX_GATE_SCALAR>(p, nstate, st) : launch_bwd<64, LNX_GATE_NONE>(p, nstate, st);
}
