// Chunked delta-rule backward on gfx950 MFMA.  Gradients of <o, dO> + <S_T, dS_T> with respect
// to q, k, v, beta, g and S_0, from the tensors lnx_chunk_fwd left in the workspace.  The
// reference has no backward code (its gradients come from JAX autodiff of the recurrent scan,
// linearnexus/train/sft.py:126-127); this is the hand-derived adjoint of the chunk algorithm of
// gated_deltanet.py:444-523.  Four kernels:
//
//   bwd_local  (chunk x dv-slab parallel)   dD_loc = P^T dO
//   bwd_scan   (sequential, reverse)        dD = dD_loc + (K r) dS;  dS <- e^{G_last} dS + (Q~ e^G)^T dO - W^T dD
//   bwd_dqk    (chunk parallel)             dP, dq, the P/K^r parts of dk, dW = -dD S^T, gate terms
//   bwd_wy     (chunk parallel)             through W = Tm B_w, U = Tm B_u and Tm = (I + A)^-1:
//                                           dv, dbeta, the remaining parts of dk, dg (reverse cumsum)
// with r_j = exp(G_last - G_j), G the cumulative log-decay inside the chunk.

#include "chunk_common.h"
#include "reduce_rows.h"

namespace {

struct BwdParams {
  ChunkGeom geom;
  const void* q;
  const void* k;
  const void* v;
  const float* beta;
  const void* d_o;
  const float* d_sT;
  void* dq;
  void* dk;
  void* dv_out;
  float* dbeta;
  float* dg;
  float* ds0;
  int dv, gate;
  int slab;  // lnx_scan_args.test_scan_slab
  // per-channel gate activated inside the op (lnx_scan_args.gate_raw): bwd_wy2 carries dg through the activation
  const void* graw;
  const float* gA;
  const float* gbias;
  float gthr;
  bool gband;  // softplus(threshold) != threshold in fp32: the activation's two branches overlap in the gate's values
  void* dgraw;
  float* gpart;       // [2][prows + LNX_SUM_SLICES][H * dk]: per-chunk partial sums of d_bias and of dg * g
  int64_t gprows;     // partial rows: chunk slots per head
  float scale;
  char* ws;
  ChunkWs off;
};

template <typename T> __device__ __forceinline__ T* wsp(const BwdParams& p, uint64_t off) {
  return reinterpret_cast<T*>(p.ws + off);
}

// ---------------------------------------------------------------------------------------
// bwd_local: dD_loc[j][v] = sum_i P[i][j] dO[i][v]; dO^T slab to the workspace
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_local_kernel(BwdParams p) {
  constexpr int LDC = LNX_C + Mma<T>::PAD;
  __shared__ __align__(16) T sP[64 * LDC];    // P  [i][j]
  __shared__ __align__(16) T sdO[64 * LDC];   // dO [i][v]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  int64_t slot;
  int part;
  if (!xcd_slot_part((int64_t)p.geom.rows * N, p.dv / 64, slot, part)) return;
  const int row = (int)(slot / N), n = (int)(slot % N);
  const int v0 = part * 64;
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  if (len <= 0) return;
  const int64_t tbase = tok_index(p.geom, row, tok0);
  TileRegs<T, 64, 64> rP, rdO;
  rP.load(wsp<T>(p, p.off.P) + slot * 64 * 64, 64, 64, tid);
  rdO.load(reinterpret_cast<const T*>(p.d_o) + tbase * p.dv + v0, (int64_t)p.geom.ts * p.dv, len, tid);
  rP.store(sP, LDC, tid);
  rdO.store(sdO, LDC, tid);
  lds_barrier();
  const int wi = wave >> 1, wj = wave & 1;
  floatx16 acc[1][1];
  frag_zero(acc);
  // dD_loc[j][v] = sum_i P[i][j] dO[i][v]: both operands contract along the rows of their tiles
  mma_x<T, 1, 1, true, true>(acc, sP + 32 * wi, LDC, sdO + 32 * wj, LDC, 64, lane);
  frag_store<T, 1, 1>(acc, wsp<T>(p, p.off.dD) + slot * 64 * p.dv + (int64_t)(32 * wi) * p.dv + v0 + 32 * wj, p.dv, lane);
}

// ---------------------------------------------------------------------------------------
// bwd_scan: the reverse sequential pass over the chunks of one (state, slab of dv).  Per chunk:
//   dD = dD_loc + r_j (K dS)_j   (the complete gradient of D, back to the workspace),
//   dS <- e^{G_last} dS + (scale Q e^G)^T dO - W^T dD,
// with dS the gradient of the state leaving the chunk (stored transposed for bwd_dqk).
// Same organisation as the forward scan: waves 0-3 compute on the tiles in LDS, waves 4-7 move
// data (global loads two chunks ahead, tile writes as soon as a tile's reader is done, LDS ->
// global copies of dS and dD), three barriers per chunk:
//   B1  tiles of chunk n and dS^T are in LDS      compute: dD          movers: loads of chunk n-2, dS -> workspace
//   B2  dD is in LDS (plain and negated-transposed)  compute: dS update   movers: K of chunk n-1 -> LDS, dD -> workspace
//   B3  all reads of chunk n's tiles are done     compute: dS^T -> LDS  movers: remaining tiles of chunk n-1 -> LDS
// ---------------------------------------------------------------------------------------
// BVW = columns of dv per workgroup: 64 by default; 32 for dk = 128 with 4-byte inputs (LDS capacity) and,
// on request, for dk = 128 with 2-byte inputs when 64-column slabs would leave most CUs idle.
template <typename T, int DK, int BVW = 64> struct BScanCfg {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int BV = (DK > 128 && sizeof(T) == 4) ? 32 : BVW;
  static constexpr int LDK = DK + PAD, LDU = BV + PAD;
  static constexpr int LDC = LNX_C + PAD;
  static constexpr int kRow = 64 * LDK, kSlab = 64 * LDU, kdST = BV * LDK, kdDT = BV * LDC;
  // 2-byte inputs: the chunk-local part dD_loc = P^T dO is formed here as well (P and the unscaled dO
  // tile fit LDS), so bwd_local does not run
  static constexpr bool FUSE_LOCAL = sizeof(T) == 2;
  static constexpr int kP = FUSE_LOCAL ? 64 * LDC : 0, kRaw = FUSE_LOCAL ? kSlab : 0;
  static constexpr int kG = DK > 128 ? DK : 128;  // gate values: 64 tokens (scalar gate) or dk channels (vector gate)
  // 4-byte inputs with dk = 256: K (read for dD), Q and W (read for the dS update) of a chunk take turns in one tile
  static constexpr bool SHARE = sizeof(T) == 4 && DK > 128;
  // 64-column slabs of 2-byte inputs with dk = 256 and of 4-byte inputs with dk = 128: K (read for dD) and Q (read
  // for the dS update) share a tile
  static constexpr bool SHAREK = BV == 64 && ((sizeof(T) == 2 && DK > 128) || (sizeof(T) == 4 && DK == 128));
  static constexpr int nRow = SHARE ? 1 : SHAREK ? 2 : 3;
  // 32-column slabs of 2-byte inputs with dk = 128: every input tile twice, so that the movers write chunk n - 1
  // while chunk n is being read
  static constexpr bool DB = sizeof(T) == 2 && DK == 128 && BV == 32;
  static constexpr int NB = DB ? 2 : 1;
  // K, Q, W rows [token][dk];  dO, dD slabs [token][BV];  -dD^T [BV][token];  dS^T [BV][dk];  P;  unscaled dO
  static constexpr size_t bytes = sizeof(T) * (NB * (nRow * kRow + kSlab + kP + kRaw) + kSlab + kdDT + kdST) + sizeof(float) * NB * kG;
};

template <typename T, int DK, int GATE, int BVW = 64>
__global__ __launch_bounds__(512) void bwd_scan_kernel(BwdParams p) {
  typedef BScanCfg<T, DK, BVW> L;
  constexpr int LDK = L::LDK, LDU = L::LDU, LDC = L::LDC, BV = L::BV;
  constexpr bool FUSE = L::FUSE_LOCAL;
  constexpr int CT = BV / 32;                      // column tiles of the slab
  constexpr int RT = (DK >= 128) ? DK / 128 : 1;   // state tiles per wave: RT row tiles (from RT * wave, or wave & 1
  constexpr int NT = (DK >= 128) ? CT : 1;         //   for dk = 64) x NT column tiles
  static_assert(DK >= 128 || BV == 64, "dk = 64 needs a 64-column slab");
  extern __shared__ __align__(16) char smem[];
  constexpr int NB = L::NB;  // buffers per input tile (the second of a pair follows the first)
  T* sK = reinterpret_cast<T*>(smem);
  T* sQ = (L::SHARE || L::SHAREK) ? sK : sK + NB * L::kRow;
  T* sW = L::SHARE ? sK : sQ + NB * L::kRow;
  T* sdO = sK + NB * L::nRow * L::kRow;
  T* sdDl = sdO + NB * L::kSlab;
  T* sdDT = sdDl + L::kSlab;
  T* sdST = sdDT + L::kdDT;
  T* sP = sdST + L::kdST;   // fused local part only: P [i][j] and the unscaled dO slab
  T* sdOr = sP + NB * L::kP;
  float* sG = reinterpret_cast<float*>(sdOr + NB * L::kRaw);

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
      // ---------------- movers, one tile shared by K, Q and W ----------------
      // Three more barriers separate the tile's uses; the tiles not in LDS wait in registers.
      //   B1   K of chunk n in LDS            -> loads of Q, W of chunk n; dS -> workspace
      //   B2   dD done, K dead                -> Q -> LDS, dD -> workspace
      //   B2a  Q in LDS (compute: Q^T dO)     -> loads of K and the slabs of chunk n-1
      //   B2b  Q dead                         -> W -> LDS
      //   B2c  W in LDS (compute: W^T dD)
      //   B3   W dead                         -> K and the slabs of chunk n-1 -> LDS
      const int mt = tid - 256;
      typedef TileRegs<T, 64, BV> Slab;
      TileRegs<T, 64, DK> rX, rY;  // X: K, then Q; Y: W
      Slab rdO, rdD;
      float os[Slab::IT], rG = 0.f;
      const int64_t tsk = (int64_t)p.geom.ts * DK;
      auto tok_base = [&](int n, int& len) {
        int tok0;
        chunk_span(span, n, tok0, len);
        return tok_index(p.geom, row, tok0);
      };
      auto fetch_k = [&](int n) {  // K and the slabs of chunk n
        const int64_t slot = (int64_t)row * N + n;
        int len;
        const int64_t tbase = tok_base(n, len);
        if (GATE == LNX_GATE_VECTOR) rX.load(wsp<T>(p, p.off.Kr) + slot * 64 * DK, DK, 64, mt);
        else rX.load(reinterpret_cast<const T*>(p.k) + tbase * DK, tsk, len, mt);
        rdO.load(reinterpret_cast<const T*>(p.d_o) + tbase * p.dv + v0, (int64_t)p.geom.ts * p.dv, len, mt);
        rdD.load(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, 64, mt);
        if (GATE == LNX_GATE_SCALAR && mt < 64) rG = wsp<float>(p, p.off.G)[slot * 64 + mt];
        if (GATE == LNX_GATE_VECTOR && mt < DK) rG = wsp<float>(p, p.off.G)[(slot * 64 + 63) * DK + mt];
#pragma unroll
        for (int it = 0; it < Slab::IT; ++it) {
          const int r = min((mt + 256 * it) / Slab::VPR, 63);
          os[it] = (GATE == LNX_GATE_SCALAR) ? wsp<float>(p, p.off.G)[slot * 64 + r] : 0.f;
        }
      };
      auto fetch_qw = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        int len;
        const int64_t tbase = tok_base(n, len);
        if (GATE == LNX_GATE_VECTOR) rX.load(wsp<T>(p, p.off.Qg) + slot * 64 * DK, DK, 64, mt);
        else rX.load(reinterpret_cast<const T*>(p.q) + tbase * DK, tsk, len, mt);
        rY.load(wsp<T>(p, p.off.W) + slot * 64 * DK, DK, 64, mt);
      };
      auto commit_k = [&]() {
        rX.store(sK, LDK, mt);
        rdD.store(sdDl, LDU, mt);
#pragma unroll
        for (int it = 0; it < Slab::IT; ++it) {
          const int idx = mt + 256 * it, r = idx / Slab::VPR, c = (idx - r * Slab::VPR) * Slab::N;
          typename Vec16<T>::V o = rdO.get(it, mt);
          if (GATE != LNX_GATE_VECTOR) {  // dO rows scaled by scale e^{G_i}
            const float f = (GATE == LNX_GATE_NONE) ? p.scale : p.scale * __expf(os[it]);
#pragma unroll
            for (int e = 0; e < Slab::N; ++e) o[e] = from_f32<T>(to_f32(o[e]) * f);
          }
          if (idx < Slab::TOTAL) *reinterpret_cast<typename Vec16<T>::V*>(sdO + r * LDU + c) = o;
        }
        if (mt < L::kG) sG[mt] = rG;
      };
      if (c0 < c1) {
        fetch_k(c1 - 1);
        commit_k();
      }
      lds_barrier();  // B1 of the first chunk
      for (int n = c1 - 1; n >= c0; --n) {
        const int64_t slot = (int64_t)row * N + n;
        fetch_qw(n);
        unstage_tile<T, BV, DK, true>(wsp<T>(p, p.off.dSn) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sdST, LDK, BV, mt);
        lds_barrier();  // B2
        rX.store(sQ, LDK, mt);
        unstage_tile<T, 64, BV, true>(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, sdDl, LDU, 64, mt);
        lds_barrier();  // B2a
        if (n - 1 >= c0) fetch_k(n - 1);
        lds_barrier();  // B2b
        rY.store(sW, LDK, mt);
        lds_barrier();  // B2c
        lds_barrier();  // B3
        if (n - 1 >= c0) commit_k();
        lds_barrier();  // B1 of the next chunk
      }
      return;
    }
  } else if constexpr (L::SHAREK) {
    if (wave >= 4) {
      // ---------------- movers, one tile shared by K and Q ----------------
      // B1: K, W, P, dO of chunk n in LDS -> loads of those of chunk n-1, dS -> workspace;  B2: Q of chunk n -> the K
      // tile, dD -> workspace;  B2': loads of Q of chunk n-1;  B3: tiles of chunk n-1 -> LDS.
      const int mt = tid - 256;
      typedef TileRegs<T, 64, BV> Slab;
      TileRegs<T, 64, DK> rK, rQ, rW;
      Slab rdO, rdD;                      // dD: the chunk-local part from bwd_local (not fused only)
      TileRegs<T, 64, FUSE ? 64 : 8> rP;  // fused only
      float os[Slab::IT], rG = 0.f;
      const int64_t tsk = (int64_t)p.geom.ts * DK;
      auto fetch_main = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        int tok0, len;
        chunk_span(span, n, tok0, len);
        const int64_t tbase = tok_index(p.geom, row, tok0);
        if (GATE == LNX_GATE_VECTOR) rK.load(wsp<T>(p, p.off.Kr) + slot * 64 * DK, DK, 64, mt);
        else rK.load(reinterpret_cast<const T*>(p.k) + tbase * DK, tsk, len, mt);
        rW.load(wsp<T>(p, p.off.W) + slot * 64 * DK, DK, 64, mt);
        rdO.load(reinterpret_cast<const T*>(p.d_o) + tbase * p.dv + v0, (int64_t)p.geom.ts * p.dv, len, mt);
        if (FUSE) rP.load(wsp<T>(p, p.off.P) + slot * 64 * 64, 64, 64, mt);
        else rdD.load(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, 64, mt);
        if (GATE == LNX_GATE_SCALAR && mt < 64) rG = wsp<float>(p, p.off.G)[slot * 64 + mt];
        if (GATE == LNX_GATE_VECTOR && mt < DK) rG = wsp<float>(p, p.off.G)[(slot * 64 + 63) * DK + mt];
#pragma unroll
        for (int it = 0; it < Slab::IT; ++it) {
          const int r = min((mt + 256 * it) / Slab::VPR, 63);
          os[it] = (GATE == LNX_GATE_SCALAR) ? wsp<float>(p, p.off.G)[slot * 64 + r] : 0.f;
        }
      };
      auto fetch_q = [&](int n) {
        const int64_t slot = (int64_t)row * N + n;
        int tok0, len;
        chunk_span(span, n, tok0, len);
        if (GATE == LNX_GATE_VECTOR) rQ.load(wsp<T>(p, p.off.Qg) + slot * 64 * DK, DK, 64, mt);
        else rQ.load(reinterpret_cast<const T*>(p.q) + tok_index(p.geom, row, tok0) * DK, tsk, len, mt);
      };
      auto commit_main = [&]() {
        rK.store(sK, LDK, mt);
        rW.store(sW, LDK, mt);
        if (FUSE) {
          rP.store(sP, LDC, mt);
          rdO.store(sdOr, LDU, mt);
        } else {
          rdD.store(sdDl, LDU, mt);
        }
#pragma unroll
        for (int it = 0; it < Slab::IT; ++it) {
          const int idx = mt + 256 * it, r = idx / Slab::VPR, c = (idx - r * Slab::VPR) * Slab::N;
          typename Vec16<T>::V o = rdO.get(it, mt);
          if (GATE != LNX_GATE_VECTOR) {  // dO rows scaled by scale e^{G_i}
            const float f = (GATE == LNX_GATE_NONE) ? p.scale : p.scale * __expf(os[it]);
#pragma unroll
            for (int e = 0; e < Slab::N; ++e) o[e] = from_f32<T>(to_f32(o[e]) * f);
          }
          if (idx < Slab::TOTAL) *reinterpret_cast<typename Vec16<T>::V*>(sdO + r * LDU + c) = o;
        }
        if (mt < L::kG) sG[mt] = rG;
      };
      if (c0 < c1) {
        fetch_main(c1 - 1);
        fetch_q(c1 - 1);
        commit_main();
      }
      lds_barrier();  // B1 of the first chunk
      for (int n = c1 - 1; n >= c0; --n) {
        const int64_t slot = (int64_t)row * N + n;
        if (n - 1 >= c0) fetch_main(n - 1);
        unstage_tile<T, BV, DK, true>(wsp<T>(p, p.off.dSn) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sdST, LDK, BV, mt);
        lds_barrier();  // B2
        rQ.store(sQ, LDK, mt);
        unstage_tile<T, 64, BV, true>(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, sdDl, LDU, 64, mt);
        lds_barrier();  // B2'
        if (n - 1 >= c0) fetch_q(n - 1);
        lds_barrier();  // B3
        if (n - 1 >= c0) commit_main();
        lds_barrier();  // B1 of the next chunk
      }
      return;
    }
  } else if (wave >= 4) {
    // ---------------- movers ----------------
    const int mt = tid - 256;
    typedef TileRegs<T, 64, BV> Slab;
    struct Tiles {
      TileRegs<T, 64, DK> K, Q, W;
      Slab dO, dD;                       // dD: the chunk-local part from bwd_local (not fused only)
      TileRegs<T, 64, FUSE ? 64 : 8> P;  // fused only
      float os[Slab::IT];  // G_i of the dO row each vector belongs to (scalar gate)
      float G;
    };
    constexpr int AHEAD = (sizeof(T) == 2 && DK <= 128) ? 2 : 1;  // chunks fetched ahead (register sets in use)
    Tiles ta, tb;
    ta.G = tb.G = 0.f;
    // Loads of chunk n into a register set, in three parts (part < 0: all at once).  A CU accepts vector memory
    // instructions at a limited rate, so the parts are issued in different phases of a chunk instead of holding up
    // the first one.  Nothing is computed from loaded values here: that would wait for every load issued before.
    auto fetch = [&](Tiles& R, int n, int part) {
      const int64_t slot = (int64_t)row * N + n;
      int tok0, len;
      chunk_span(span, n, tok0, len);
      const int64_t tbase = tok_index(p.geom, row, tok0);
      const int64_t tsk = (int64_t)p.geom.ts * DK;
      // vector gate: K e^{G_last - G} and scale Q e^G were stored by the forward pass (all 64 rows defined)
      if (part < 0 || part == 0) {
        if (GATE == LNX_GATE_VECTOR) R.K.load(wsp<T>(p, p.off.Kr) + slot * 64 * DK, DK, 64, mt);
        else R.K.load(reinterpret_cast<const T*>(p.k) + tbase * DK, tsk, len, mt);
      }
      if (part < 0 || part == 1) {
        R.dO.load(reinterpret_cast<const T*>(p.d_o) + tbase * p.dv + v0, (int64_t)p.geom.ts * p.dv, len, mt);
        if (FUSE) R.P.load(wsp<T>(p, p.off.P) + slot * 64 * 64, 64, 64, mt);
        else R.dD.load(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, 64, mt);
        // every thread loads (clamped index): a load behind a branch cannot be counted
        if (GATE == LNX_GATE_SCALAR) R.G = wsp<float>(p, p.off.G)[slot * 64 + (mt & 63)];
        if (GATE == LNX_GATE_VECTOR) R.G = wsp<float>(p, p.off.G)[(slot * 64 + 63) * DK + min(mt, DK - 1)];
      }
      if (part < 0 || part == 2) {
        if (GATE == LNX_GATE_VECTOR) R.Q.load(wsp<T>(p, p.off.Qg) + slot * 64 * DK, DK, 64, mt);
        else R.Q.load(reinterpret_cast<const T*>(p.q) + tbase * DK, tsk, len, mt);
        R.W.load(wsp<T>(p, p.off.W) + slot * 64 * DK, DK, 64, mt);
#pragma unroll
        for (int it = 0; it < Slab::IT; ++it) {
          const int r = min((mt + 256 * it) / Slab::VPR, 63);
          R.os[it] = (GATE == LNX_GATE_SCALAR) ? wsp<float>(p, p.off.G)[slot * 64 + r] : 0.f;
        }
      }
    };
    auto commit_rest = [&](const Tiles& R, int pb, int part = -1) {  // parts as in fetch (K is written by the caller)
      if (part < 0 || part == 2) {
        R.Q.store(sQ + pb * L::kRow, LDK, mt);
        R.W.store(sW + pb * L::kRow, LDK, mt);
      }
      if (part == 0 || part == 2) return;
      if (FUSE) {
        R.P.store(sP + pb * L::kP, LDC, mt);
        R.dO.store(sdOr + pb * L::kRaw, LDU, mt);
      } else {
        R.dD.store(sdDl, LDU, mt);
      }
#pragma unroll
      for (int it = 0; it < Slab::IT; ++it) {
        const int idx = mt + 256 * it, r = idx / Slab::VPR, c = (idx - r * Slab::VPR) * Slab::N;
        typename Vec16<T>::V o = R.dO.get(it, mt);
        if (GATE != LNX_GATE_VECTOR) {  // dO rows scaled by scale e^{G_i}: (scale Q e^G)^T dO = Q^T (that)
          const float os = (GATE == LNX_GATE_NONE) ? p.scale : p.scale * __expf(R.os[it]);
#pragma unroll
          for (int e = 0; e < Slab::N; ++e) o[e] = from_f32<T>(to_f32(o[e]) * os);
        }
        if (idx < Slab::TOTAL) *reinterpret_cast<typename Vec16<T>::V*>(sdO + pb * L::kSlab + r * LDU + c) = o;
      }
      if (mt < L::kG) sG[pb * L::kG + mt] = R.G;
    };
    // Double-buffered form.  Chunk n - 1 goes to the buffers chunk n + 1 was read from, so no tile write waits for a
    // reader: loads of chunk n - 2 and the tile writes in the first two phases, dS', dD -> workspace in the second.
    // `steady` (a std::bool_constant): chunks n - 1 and n - 2 exist, so nothing sits behind a branch and the compiler
    // can count the loads in flight.
    auto step_db = [&](Tiles& cur, const Tiles& nxt, int n, auto steady) {
      constexpr bool STEADY = decltype(steady)::value;
      const int64_t slot = (int64_t)row * N + n;
      const int pb = (c1 - 1 - n) & 1;
      if constexpr (STEADY) {
        // chunk n's registers are free again and take chunk n - 2; the tile writes of chunk n - 1 sit between the loads,
        // a part at a time: a wave whose load waits for a slot in the memory path issues nothing else, and the writes
        // go out while the loads before them drain.  Q and W follow the stores of the second phase.
#pragma unroll
        for (int part = 0; part < 2; ++part) {
          fetch(cur, n - 2, part);
          if (part == 0) nxt.K.store(sK + (pb ^ 1) * L::kRow, LDK, mt);
          else commit_rest(nxt, pb ^ 1, part);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        if (n - 2 >= c0) fetch(cur, n - 2, -1);
        if (n - 1 >= c0) {
          nxt.K.store(sK + (pb ^ 1) * L::kRow, LDK, mt);
          commit_rest(nxt, pb ^ 1);
        }
      }
      lds_barrier();  // B2
      unstage_tile<T, BV, DK, true>(wsp<T>(p, p.off.dSn) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sdST, LDK, BV, mt);
      unstage_tile<T, 64, BV, true>(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, sdDl, LDU, 64, mt);
      if constexpr (STEADY) {
        fetch(cur, n - 2, 2);
        commit_rest(nxt, pb ^ 1, 2);
      }
      lds_barrier();  // B3
      lds_barrier();  // B1 of the next chunk
    };
    auto step = [&](Tiles& cur, const Tiles& nxt, int n) {  // cur: chunk n (in LDS already), nxt: chunk n - 1
      const int64_t slot = (int64_t)row * N + n;
      const bool more = n - AHEAD >= c0;  // chunk n's registers are free again: they take chunk n - AHEAD
      if (more) fetch(cur, n - AHEAD, AHEAD == 2 ? 0 : -1);
      unstage_tile<T, BV, DK, true>(wsp<T>(p, p.off.dSn) + slot * p.dv * DK + (int64_t)v0 * DK, DK, sdST, LDK, BV, mt);
      lds_barrier();  // B2
      if (n - 1 >= c0) nxt.K.store(sK, LDK, mt);
      if (more && AHEAD == 2) fetch(cur, n - AHEAD, 1);  // before the stores below: see the forward scan
      unstage_tile<T, 64, BV, true>(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, sdDl, LDU, 64, mt);
      lds_barrier();  // B3
      if (more && AHEAD == 2) fetch(cur, n - AHEAD, 2);
      if (n - 1 >= c0) commit_rest(nxt, 0);
      lds_barrier();  // B1 of the next chunk
    };
    if (c0 < c1) {
      fetch(ta, c1 - 1, -1);
      ta.K.store(sK, LDK, mt);
      commit_rest(ta, 0);
    }
    if (AHEAD == 2 && c1 - 2 >= c0) fetch(tb, c1 - 2, -1);
    lds_barrier();  // B1 of the first chunk
    if constexpr (L::DB) {
      int n = c1 - 1;
      for (; n - 3 >= c0; n -= 2) {  // chunks n - 2 and n - 3 exist
        step_db(ta, tb, n, std::true_type{});
        step_db(tb, ta, n - 1, std::true_type{});
      }
      for (; n >= c0; n -= 2) {
        step_db(ta, tb, n, std::false_type{});
        if (n - 1 >= c0) step_db(tb, ta, n - 1, std::false_type{});
      }
    } else if (AHEAD == 2) {
      for (int n = c1 - 1; n >= c0; n -= 2) {
        step(ta, tb, n);
        if (n - 1 >= c0) step(tb, ta, n - 1);
      }
    } else {
      for (int n = c1 - 1; n >= c0; --n) step(ta, ta, n);
    }
    return;
  }

  // ---------------- compute waves ----------------
  const int srow = (DK >= 128) ? 32 * RT * wave : 32 * (wave & 1);
  const int scol = (DK >= 128) ? 0 : 32 * (wave >> 1);
  // tile of the [64 x BV] token-by-value products owned by this wave (none for CT == 1, wave >= 2)
  const int wi = (CT == 2) ? (wave >> 1) : wave, wj = (CT == 2) ? (wave & 1) : 0;
  const bool has_tile = (CT == 2) || wave < 2;

  floatx16 dS[RT][NT];
  frag_zero(dS);
  if (p.d_sT) {
    const float* src = p.d_sT + (int64_t)sidx * DK * p.dv + v0;
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          dS[i][j][e] = src[(int64_t)(srow + 32 * i + frag_row(e, lane)) * p.dv + scol + 32 * j + frag_col(lane)];
  }
  // dS (gradient of the state leaving the chunk) -> LDS, transposed [dv][dk]; the movers copy it to the workspace
  if (c0 < c1) frag_store_t<T, RT, NT>(dS, sdST + scol * LDK + srow, LDK, lane);
  lds_barrier();  // B1 of the first chunk
  for (int n = c1 - 1; n >= c0; --n) {
    const int pb = L::DB ? (c1 - 1 - n) & 1 : 0;  // buffer of this chunk's tiles
    const T* cK = sK + pb * L::kRow;
    const T* cQ = sQ + pb * L::kRow;
    const T* cW = sW + pb * L::kRow;
    const T* cdO = sdO + pb * L::kSlab;
    const T* cP = sP + pb * L::kP;
    const T* cdOr = sdOr + pb * L::kRaw;
    const float* cG = sG + pb * L::kG;
    const float gl = (GATE == LNX_GATE_SCALAR) ? cG[63] : 0.f;
    // dD = dD_loc + r_j (K dS)_j
    if (has_tile) {
      floatx16 d[1][1];
      frag_zero(d);
      mma_nt<T, 1, 1>(d, cK + 32 * wi * LDK, LDK, sdST + 32 * wj * LDK, LDK, DK, lane);
      // the complete dD replaces the local part in place (all reads first: interleaved with the
      // writes they would be serialised); the movers write it out
      float dl[16];
      if (FUSE) {  // dD_loc[j][v] = sum_i P[i][j] dO[i][v]: both operands contract along the rows of their tiles
        floatx16 l[1][1];
        frag_zero(l);
        mma_x<T, 1, 1, true, true>(l, cP + 32 * wi, LDC, cdOr + 32 * wj, LDU, 64, lane);
#pragma unroll
        for (int e = 0; e < 16; ++e) dl[e] = l[0][0][e];
      } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) dl[e] = to_f32(sdDl[(32 * wi + frag_row(e, lane)) * LDU + 32 * wj + frag_col(lane)]);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float rj = (GATE == LNX_GATE_SCALAR) ? __expf(fminf(gl - cG[32 * wi + frag_row(e, lane)], 0.f)) : 1.f;
        d[0][0][e] = dl[e] + rj * d[0][0][e];
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        sdDl[(32 * wi + frag_row(e, lane)) * LDU + 32 * wj + frag_col(lane)] = from_f32<T>(d[0][0][e]);
        d[0][0][e] = -d[0][0][e];
      }
      frag_store_t<T, 1, 1>(d, sdDT + 32 * wj * LDC + 32 * wi, LDC, lane);
    }
    lds_barrier();  // B2

    // dS <- e^{G_last} dS + (scale Q e^G)^T dO - W^T dD   (token-contracted: rows of the tiles)
    if (GATE == LNX_GATE_SCALAR) {
      const float dec = __expf(gl);
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) dS[i][j][e] *= dec;
    }
    if (GATE == LNX_GATE_VECTOR) {
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) dS[i][j][e] *= __expf(cG[srow + 32 * i + frag_row(e, lane)]);
    }
    if (L::SHAREK) {  // W first: Q is still on its way into the tile it shares with K
      mma_x<T, RT, NT, true, false>(dS, cW + srow, LDK, sdDT + scol * LDC, LDC, 64, lane);
      lds_barrier();  // B2'
      mma_x<T, RT, NT, true, true>(dS, cQ + srow, LDK, cdO + scol, LDU, 64, lane);
    } else {
      if (L::SHARE) lds_barrier();  // B2a: Q has replaced K in the shared tile
      mma_x<T, RT, NT, true, true>(dS, cQ + srow, LDK, cdO + scol, LDU, 64, lane);
      if (L::SHARE) {
        lds_barrier();  // B2b
        lds_barrier();  // B2c: W has replaced Q
      }
      mma_x<T, RT, NT, true, false>(dS, cW + srow, LDK, sdDT + scol * LDC, LDC, 64, lane);
    }
    lds_barrier();  // B3
    if (n > c0) frag_store_t<T, RT, NT>(dS, sdST + scol * LDK + srow, LDK, lane);
    lds_barrier();  // B1 of the next chunk
  }
  if (p.ds0) {
    float* out = p.ds0 + (int64_t)sidx * DK * p.dv + v0;
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          out[(int64_t)(srow + 32 * i + frag_row(e, lane)) * p.dv + scol + 32 * j + frag_col(lane)] = dS[i][j][e];
  }
}

// ---------------------------------------------------------------------------------------
// bwd_dqk: one workgroup per (chunk, 64-channel part of dk).  Loop over 32-column slabs of dv, every product one 32x32
// tile per wave.  A slab's compute time is a fraction of a memory round trip, so with 2-byte inputs the slabs arrive
// through loads that bypass the registers (mma_tiles.h) into NBUF unpadded LDS buffers, NBUF - 1 slabs ahead of the
// one being multiplied; 4-byte inputs prefetch the next slab into registers.
// ---------------------------------------------------------------------------------------
template <typename T, int DK, int GATE> struct DqkCfg {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int LDC = LNX_C + PAD, LDF = 64 + 4;
  static constexpr int kTile = 64 * LDC;
  // loop phase: dO, D, dD slabs [64][SV] and S_n, dS_n slabs [SV][64], five tiles of kLoop elements
  static constexpr int SV = 32, LDSV = SV + PAD;
  static constexpr int kLoop = (64 * LDSV > SV * LDC) ? 64 * LDSV : SV * LDC;
  // 2-byte inputs: NBUF buffers of dO | D | dD ([64][SV], read by rows) | S_n | dS_n ([SV][64], transposing reads)
  static constexpr bool DMA = sizeof(T) == 2;
  static constexpr int NBUF = GATE == LNX_GATE_VECTOR ? 3 : 2;  // what two / three workgroups per CU leave room for
  static constexpr int slab_bytes = 5 * 64 * SV * 2;
  static constexpr size_t loop_bytes = DMA ? (size_t)NBUF * slab_bytes : sizeof(T) * 5 * kLoop;
  // scalar epilogue: dPe, K rows, Q rows and one staging tile (dW, then dk), four [64][64] tiles
  static constexpr size_t scalar_bytes = sizeof(T) * 4 * kTile;
  // vector epilogue: alpha, out (fp32 [64][LDF]) and K, Q rows, plus dP in fp32
  static constexpr size_t vec_bytes = sizeof(float) * 2 * 64 * LDF + sizeof(T) * 2 * kTile;
  static constexpr size_t epi_bytes = (GATE == LNX_GATE_VECTOR) ? vec_bytes : scalar_bytes;
  static constexpr size_t big = epi_bytes > loop_bytes ? epi_bytes : loop_bytes;
  static constexpr int kSmall = 64 * 4 + (GATE == LNX_GATE_VECTOR ? 64 * LNX_LDA : 0);  // floats
  static constexpr size_t bytes = sizeof(float) * kSmall + big;
  static_assert(!DMA || bytes * (GATE == LNX_GATE_VECTOR ? 2 : 3) <= 160 * 1024, "workgroups per CU");
};

template <typename T, int DK, int GATE>
__global__ __launch_bounds__(256, (GATE == LNX_GATE_VECTOR ? (sizeof(T) == 2 ? 2 : 1) : sizeof(T) == 2 ? 3 : 2)) void bwd_dqk_kernel(BwdParams p) {
  typedef DqkCfg<T, DK, GATE> L;
  constexpr int LDC = L::LDC, LDF = L::LDF;
  extern __shared__ __align__(16) char smem[];
  float* sG = reinterpret_cast<float*>(smem);
  float* sSS = sG + 64;     // vector gate: per key channel sum_v dS_n[c][v] S_n[c][v]
  float* sMisc = sSS + 64;  // scalar gate: [4 + wave] = the wave's share of sum_j r_j <dKr_j, k_j>, [8 + wave] = of <dS_n, S_n>
  float* sR = sMisc + 64;   // vector gate only: dP [64][LNX_LDA]
  T* sdO = reinterpret_cast<T*>(sMisc + 64 + (GATE == LNX_GATE_VECTOR ? 64 * LNX_LDA : 0));
  T* sD = sdO + L::kLoop;
  T* sdD = sD + L::kLoop;
  T* sSn = sdD + L::kLoop;
  T* sdSn = sSn + L::kLoop;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  int64_t slot;
  int part;
  if (!xcd_slot_part((int64_t)p.geom.rows * N, DK / 64, slot, part)) return;
  const int ch0 = part * 64;  // first key channel of this half
  const int row = (int)(slot / N), n = (int)(slot % N);
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  if (len <= 0) return;
  const int64_t tbase = tok_index(p.geom, row, tok0);
  const int64_t tsk = (int64_t)p.geom.ts * DK, tsv = (int64_t)p.geom.ts * p.dv;  // row strides of the token tiles
  const T* qg = reinterpret_cast<const T*>(p.q) + tbase * DK + ch0;
  const T* kg = reinterpret_cast<const T*>(p.k) + tbase * DK + ch0;
  const int wi = wave >> 1, wj = wave & 1;

  // dv is consumed in slabs of SV columns
  constexpr int SV = L::SV, LDS_ = L::LDSV;
  // per-channel gate: K, Q rows and the cumulative gate of this half for the epilogue, fetched during the last slab
  TileRegs<T, 64, (GATE == LNX_GATE_VECTOR ? 64 : 8)> rk, rq;
  TileRegs<float, 64, (GATE == LNX_GATE_VECTOR ? 64 : 4)> rGe;
  auto fetch_epilogue = [&]() {
    rk.load(kg, tsk, len, tid);
    rq.load(qg, tsk, len, tid);
    rGe.load(wsp<float>(p, p.off.G) + slot * 64 * DK + ch0, DK, 64, tid);
  };
  floatx16 aP[1][1], aQ[1][1], aW[1][1], aK[1][1];
  frag_zero(aP);
  frag_zero(aQ);
  frag_zero(aW);
  frag_zero(aK);
  float ss = 0.f;
  if constexpr (L::DMA) {
    typedef Mma<bf16_t> M;
    typedef SwzTile<64, SV> TokT;  // dO, D, dD slabs
    typedef SwzTile<SV, 64> TrT;   // S_n, dS_n slabs of this part's channels
    static_assert(TokT::NINSTR == 4 && TrT::NINSTR == 4, "one 1 KB load per wave and tile");
    constexpr int PER_WAVE = 5, NBUF = L::NBUF;
    char* sSlab = reinterpret_cast<char*>(sdO);
    const unsigned slab0 = lds_byte_addr(sSlab);
    const bf16_t* gdO = reinterpret_cast<const bf16_t*>(p.d_o) + tbase * p.dv;
    const bf16_t* gD = wsp<bf16_t>(p, p.off.D) + slot * 64 * p.dv;
    const bf16_t* gdD = wsp<bf16_t>(p, p.off.dD) + slot * 64 * p.dv;
    const bf16_t* gSn = wsp<bf16_t>(p, p.off.SnT) + slot * p.dv * DK + ch0;
    const bf16_t* gdSn = wsp<bf16_t>(p, p.off.dSn) + slot * p.dv * DK + ch0;
    // Token rows of dO past the chunk's end fetch the chunk's last row instead of zeros: they only reach rows of dq and
    // products with rows of q that are zero.
    auto issue = [&](int v0, int b) {
      const unsigned dst = slab0 + b * L::slab_bytes + 1024 * wave;
      int r, c;
      TokT::src(wave, lane, r, c);
      dma16(gdO + (int64_t)min(r, len - 1) * tsv + v0 + c, dst);
      dma16(gD + (int64_t)r * p.dv + v0 + c, dst + 4096);
      dma16(gdD + (int64_t)r * p.dv + v0 + c, dst + 2 * 4096);
      TrT::src(wave, lane, r, c);
      dma16(gSn + (int64_t)(v0 + r) * DK + c, dst + 3 * 4096);
      dma16(gdSn + (int64_t)(v0 + r) * DK + c, dst + 4 * 4096);
    };
    const int nslab = p.dv / SV;
#pragma unroll
    for (int b = 0; b < NBUF; ++b)
      if (b < nslab) issue(b * SV, b);  // first, so that the small load below does not hold them up
    if (tid < 64) {
      sG[tid] = (GATE == LNX_GATE_SCALAR) ? wsp<float>(p, p.off.G)[slot * 64 + tid] : 0.f;
      sSS[tid] = 0.f;
      sMisc[tid] = 0.f;
    }
    const int fr = lane & 31, kg8 = 8 * (lane >> 5);
    int b = 0;
#pragma unroll 1
    for (int s_ = 0; s_ < nslab; ++s_, b = (b + 1 == NBUF) ? 0 : b + 1) {
      // this slab has landed: all but the loads of the slabs behind it that have been requested
      const int behind = min(NBUF - 1, nslab - 1 - s_);
      if (behind >= 2) dma_wait<2 * PER_WAVE>();
      else if (behind == 1) dma_wait<PER_WAVE>();
      else dma_wait<0>();
      lds_barrier();
      if (GATE == LNX_GATE_VECTOR && s_ + 1 == nslab) fetch_epilogue();
      const bf16_t* tdO = reinterpret_cast<const bf16_t*>(sSlab + b * L::slab_bytes);
      const bf16_t* tD = tdO + 2048;
      const bf16_t* tdD = tD + 2048;
      const bf16_t* tSn = tdD + 2048;
      const bf16_t* tdSn = tSn + 2048;
#pragma unroll
      for (int k0 = 0; k0 < SV; k0 += 16) {
        const M::Frag fdO = TokT::load(tdO, 32 * wi + fr, k0 + kg8);
        const M::Frag fDi = TokT::load(tD, 32 * wi + fr, k0 + kg8);
        const M::Frag fDj = TokT::load(tD, 32 * wj + fr, k0 + kg8);
        const M::Frag fdD = TokT::load(tdD, 32 * wi + fr, k0 + kg8);
        const M::Frag fS = TrT::load_t(tSn, k0, 32 * wj, lane);
        const M::Frag fdS = TrT::load_t(tdSn, k0, 32 * wj, lane);
        M::mma(aP[0][0], fdO, fDj);
        M::mma(aQ[0][0], fdO, fS);
        M::mma(aW[0][0], fdD, fS);
        M::mma(aK[0][0], fDi, fdS);
      }
      if (GATE != LNX_GATE_NONE) {  // <dS_n, S_n> per channel: thread = (channel tid / 4, quarter of the slab's rows)
        constexpr int QV = SV / 4;
        const int r = tid >> 2, q4 = (tid & 3) * QV;
        float t = 0.f;
#pragma unroll
        for (int e = 0; e < QV; ++e) t += to_f32(tSn[TrT::at(q4 + e, r)]) * to_f32(tdSn[TrT::at(q4 + e, r)]);
        ss += t;
      }
      if (s_ + NBUF < nslab) {  // this buffer takes the slab NBUF ahead, once every wave has read it
        lds_barrier();
        issue((s_ + NBUF) * SV, b);
      }
    }
  } else {
  TileRegs<T, 64, SV> rdO, rD, rdD;
  TileRegs<T, SV, 64> rSn, rdSn;  // S_n and dS_n slabs stay [v][c]: contracted along their rows
  auto fetch = [&](int v0) {
    rdO.load(reinterpret_cast<const T*>(p.d_o) + tbase * p.dv + v0, tsv, len, tid);
    rD.load(wsp<T>(p, p.off.D) + slot * 64 * p.dv + v0, p.dv, 64, tid);
    rdD.load(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, 64, tid);
    rSn.load(wsp<T>(p, p.off.SnT) + slot * p.dv * DK + (int64_t)v0 * DK + ch0, DK, SV, tid);
    rdSn.load(wsp<T>(p, p.off.dSn) + slot * p.dv * DK + (int64_t)v0 * DK + ch0, DK, SV, tid);
  };
  fetch(0);  // first, so that the small load below does not hold it up
  if (tid < 64) {
    sG[tid] = (GATE == LNX_GATE_SCALAR) ? wsp<float>(p, p.off.G)[slot * 64 + tid] : 0.f;
    sSS[tid] = 0.f;
    sMisc[tid] = 0.f;
  }
  for (int v0 = 0; v0 < p.dv; v0 += SV) {
    lds_barrier();
    rdO.store(sdO, LDS_, tid);
    rD.store(sD, LDS_, tid);
    rdD.store(sdD, LDS_, tid);
    rSn.store(sSn, LDC, tid);
    rdSn.store(sdSn, LDC, tid);
    lds_barrier();
    if (v0 + SV < p.dv) fetch(v0 + SV);
    else if (GATE == LNX_GATE_VECTOR) fetch_epilogue();  // last slab: the epilogue's K, Q and gate tiles instead
    mma_nt<T, 1, 1>(aP, sdO + 32 * wi * LDS_, LDS_, sD + 32 * wj * LDS_, LDS_, SV, lane);
    mma_x<T, 1, 1, false, true>(aQ, sdO + 32 * wi * LDS_, LDS_, sSn + 32 * wj, LDC, SV, lane);
    mma_x<T, 1, 1, false, true>(aW, sdD + 32 * wi * LDS_, LDS_, sSn + 32 * wj, LDC, SV, lane);
    mma_x<T, 1, 1, false, true>(aK, sD + 32 * wi * LDS_, LDS_, sdSn + 32 * wj, LDC, SV, lane);
    if (GATE != LNX_GATE_NONE) {  // thread = (channel row tid / 4, quarter of the slab)
      constexpr int QV = SV / 4;
      const int r = tid >> 2, q4 = (tid & 3) * QV;
      float t = 0.f;
#pragma unroll
      for (int e = 0; e < QV; ++e) t += to_f32(sSn[(q4 + e) * LDC + r]) * to_f32(sdSn[(q4 + e) * LDC + r]);
      ss += t;
    }
  }
  }
  if (GATE == LNX_GATE_VECTOR) {
    ss += __shfl_xor(ss, 1, LNX_WAVE);
    ss += __shfl_xor(ss, 2, LNX_WAVE);
    if ((tid & 3) == 0) sSS[tid >> 2] = ss;
  } else if (GATE == LNX_GATE_SCALAR) {
    ss = wave_sum(ss);
    if (lane == 0) sMisc[8 + wave] = ss;  // one slot per wave, added in a fixed order where the sum is used
  }
  lds_barrier();  // slab tiles are dead from here on

  if constexpr (GATE == LNX_GATE_VECTOR) {
    // ---- per-channel gate: element-wise decays, pair terms on the VALU (64 channels) ----
    float* sAl = reinterpret_cast<float*>(sdO);      // [64][LDF] cumulative gate G_j[c] of this half's channels
    float* sOut = sAl + 64 * LDF;                    // [64][LDF]
    T* sKr = reinterpret_cast<T*>(sOut + 64 * LDF);  // K rows [64][LDC] (this half's channels)
    T* sQr = sKr + L::kTile;
    float* dGg = wsp<float>(p, p.off.dG) + slot * 64 * DK + ch0;
    // dW half through sOut (fp32) -> global
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = 32 * wi + frag_row(e, lane), j = 32 * wj + frag_col(lane);
      sR[i * LNX_LDA + j] = (i >= j) ? aP[0][0][e] : 0.f;
      sOut[i * LDF + j] = -aW[0][0][e];
    }
    rk.store(sKr, LDC, tid);
    rq.store(sQr, LDC, tid);
    rGe.store(sAl, LDF, tid);
    lds_barrier();
    {
      T* dWg = wsp<T>(p, p.off.dW) + slot * 64 * DK + ch0;
      for (int idx = tid; idx < 64 * 16; idx += 256) {
        const int r = idx >> 4, c = (idx & 15) * 4;
        store4(dWg + (int64_t)r * DK + c, load4(sOut + r * LDF + c));
      }
    }
    lds_barrier();
    // dq = scale e^G dQg + intra-chunk part
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int r = 32 * wi + frag_row(e, lane), c = 32 * wj + frag_col(lane);
      sOut[r * LDF + c] = aQ[0][0][e] * p.scale * __expf(sAl[r * LDF + c]);
    }
    lds_barrier();
    // both pair sums of dP: 2-byte inputs take them together on the bf16 MFMA and keep them in registers until used
    float pr[16], pc[16];
    const int pch = 16 * wave + (lane & 15), ptok = 4 * (lane >> 4);  // this lane's channel; its tokens are 16 t + ptok + e
    if constexpr (sizeof(T) == 2) {
      pair_levels<false>(pr, pc, sR, sAl, LDF, sKr, LDC, sQr, LDC, tid);
#pragma unroll
      for (int x = 0; x < 16; ++x) sOut[(16 * (x >> 2) + ptok + (x & 3)) * LDF + pch] += p.scale * pr[x];
    } else {
      pair_row<T, 64, false>(sOut, sR, sAl, LDF, sKr, LDC, p.scale, tid);
    }
    lds_barrier();
    T* dqg = reinterpret_cast<T*>(p.dq) + tbase * DK + ch0;
    floatx4 qdq[4];  // q dq, kept until k dk is known: the gate gradient leaves once
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
      const floatx4 v = load4(sOut + r * LDF + c), qq = load4(sQr + r * LDC + c);
      if (r < len) store4(dqg + (int64_t)r * tsk + c, v);
      qdq[it] = qq * v;
    }
    lds_barrier();
    // dk (column-type parts): e^{G_last - G} dKr + P part; chunk-end gate term from the Kr part
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int r = 32 * wi + frag_row(e, lane), c = 32 * wj + frag_col(lane);
      sOut[r * LDF + c] = aK[0][0][e] * __expf(fminf(sAl[63 * LDF + c] - sAl[r * LDF + c], 0.f));
    }
    lds_barrier();
    {  // chunk-end gate term per channel: sum_r out[r][c] k[r][c].  A wave owns sixteen channels, lane group lane / 16
       // the rows congruent to it mod 4, and the four groups meet through two shuffles: no atomics, one order of addition
      const int c = 16 * wave + (lane & 15), rq = lane >> 4;
      float part = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) part += sOut[(4 * j + rq) * LDF + c] * to_f32(sKr[(4 * j + rq) * LDC + c]);
      part += __shfl_xor(part, 16, LNX_WAVE);
      part += __shfl_xor(part, 32, LNX_WAVE);
      if (lane < 16) sMisc[c] = part;
    }
    lds_barrier();
    if (tid < 64) sSS[tid] = sMisc[tid] + __expf(sAl[63 * LDF + tid]) * sSS[tid];  // added to row 63 below
    lds_barrier();
    if constexpr (sizeof(T) == 2) {
#pragma unroll
      for (int x = 0; x < 16; ++x) sOut[(16 * (x >> 2) + ptok + (x & 3)) * LDF + pch] += p.scale * pc[x];
    } else {
      pair_col<T, 64, false>(sOut, sR, sAl, LDF, sQr, LDC, p.scale, tid);
    }
    lds_barrier();
    T* dkg = reinterpret_cast<T*>(p.dk) + tbase * DK + ch0;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
      const floatx4 v = load4(sOut + r * LDF + c), kk = load4(sKr + r * LDC + c);
      if (r < len) store4(dkg + (int64_t)r * tsk + c, v);
      floatx4 dgv = qdq[it] - kk * v;
      if (r == 63) dgv += load4(sSS + c);
      store4(dGg + r * DK + c, dgv);
    }
  } else {
    // ---- scalar / no gate ----
    T* sPe = sdO;                 // scale E dP   [i][j]
    T* sKr = sPe + L::kTile;      // K rows of this half [token][c]
    T* sQr = sKr + L::kTile;      // Q rows
    T* sOut = sQr + L::kTile;     // staging for dW ...
    T* sOut2 = sOut;              // ... and, once dW has left, for dk
    TileRegs<T, 64, 64> rKT, rQT;
    rKT.load(kg, tsk, len, tid);
    rQT.load(qg, tsk, len, tid);
    {
      floatx16 pe[1][1], nw[1][1];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int i = 32 * wi + frag_row(e, lane), j = 32 * wj + frag_col(lane);
        const float dec = (GATE == LNX_GATE_NONE) ? 1.f : __expf(fminf(sG[i] - sG[j], 0.f));
        pe[0][0][e] = (i >= j) ? p.scale * dec * aP[0][0][e] : 0.f;
        nw[0][0][e] = -aW[0][0][e];
      }
      frag_store<T, 1, 1>(pe, sPe + 32 * wi * LDC + 32 * wj, LDC, lane);
      frag_store<T, 1, 1>(nw, sOut + 32 * wi * LDC + 32 * wj, LDC, lane);
    }
    rKT.store(sKr, LDC, tid);
    rQT.store(sQr, LDC, tid);
    lds_barrier();
    unstage_tile<T, 64, 64>(wsp<T>(p, p.off.dW) + slot * 64 * DK + ch0, DK, sOut, LDC, 64, tid);
    // inter-chunk parts scaled, then the intra-chunk products on top
    const float gl = sG[63];
    float tot = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int r = 32 * wi + frag_row(e, lane), c = 32 * wj + frag_col(lane);
      const float gq = (GATE == LNX_GATE_NONE) ? p.scale : p.scale * __expf(sG[r]);
      const float gk = (GATE == LNX_GATE_NONE) ? 1.f : __expf(fminf(gl - sG[r], 0.f));
      aQ[0][0][e] *= gq;
      aK[0][0][e] *= gk;
      tot += aK[0][0][e] * to_f32(sKr[r * LDC + c]);
    }
    // dq += dPe K,  dk += dPe^T Q: K, Q (and dPe for the second product) contracted along tile rows
    mma_x<T, 1, 1, false, true>(aQ, sPe + 32 * wi * LDC, LDC, sKr + 32 * wj, LDC, 64, lane);
    mma_x<T, 1, 1, true, true>(aK, sPe + 32 * wi, LDC, sQr + 32 * wj, LDC, 64, lane);
    if (GATE != LNX_GATE_NONE) {
      tot = wave_sum(tot);
      if (lane == 0) sMisc[4 + wave] = tot;
    }
    lds_barrier();  // all reads of sPe / sOut done
    frag_store<T, 1, 1>(aQ, sPe + 32 * wi * LDC + 32 * wj, LDC, lane);
    frag_store<T, 1, 1>(aK, sOut2 + 32 * wi * LDC + 32 * wj, LDC, lane);
    lds_barrier();
    unstage_tile<T, 64, 64>(reinterpret_cast<T*>(p.dq) + tbase * DK + ch0, tsk, sPe, LDC, len, tid);
    unstage_tile<T, 64, 64>(reinterpret_cast<T*>(p.dk) + tbase * DK + ch0, tsk, sOut2, LDC, len, tid);
    if (GATE != LNX_GATE_NONE) {
      // d/dG_i = <q_i, dq_i> - <k_i, dk_i> over this half's channels (dk = its column-type parts), from the
      // staged tiles; thread = (row, quarter of the channels)
      const int r = tid >> 2, q0 = (tid & 3) * 16;
      float d = 0.f;
#pragma unroll
      for (int u = 0; u < 16; u += 4) {
        const floatx4 dq4 = load4(sPe + r * LDC + q0 + u), q4 = load4(sQr + r * LDC + q0 + u);
        const floatx4 dk4 = load4(sOut2 + r * LDC + q0 + u), k4 = load4(sKr + r * LDC + q0 + u);
#pragma unroll
        for (int e = 0; e < 4; ++e) d += dq4[e] * q4[e] - dk4[e] * k4[e];
      }
      d += __shfl_xor(d, 1, LNX_WAVE);
      d += __shfl_xor(d, 2, LNX_WAVE);
      if ((tid & 3) == 0) {
        if (r == 63) d += ((sMisc[4] + sMisc[5]) + (sMisc[6] + sMisc[7])) + __expf(gl) * ((sMisc[8] + sMisc[9]) + (sMisc[10] + sMisc[11]));
        // one slot per 64-channel part; bwd_wy2 adds the parts in order (no atomics: the same bits from run to run)
        wsp<float>(p, p.off.dG)[((int64_t)part * p.geom.rows * N + slot) * 64 + r] = d;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// bwd_wy2: gradients through the WY transform (dBw = Tm^T dW, dBu = Tm^T dD, dv, dbeta,
// dA = -tril(dBw W^T + dBu U^T, -1) and its contributions to dk and dg) as one loop over 64-column
// slabs of [dk | dv] with the next slab's tiles prefetched into registers, every product one
// 32x32 tile per wave, row and column sums taken from the fragments, results stored through LDS
// with 16-byte vectors.  The per-channel (vector) gate replaces the dense dA products of the
// epilogue by the pair-term helpers, one 64-channel half at a time.
// ---------------------------------------------------------------------------------------
template <typename T, int DK, int GATE> struct Wy2Cfg {
  static constexpr int PAD = Mma<T>::PAD;
  static constexpr int LDC = LNX_C + PAD, LDF = 64 + 4;
  static constexpr int kTile = 64 * LDC;
  static constexpr size_t nfloat = 64 * 6 + (GATE == LNX_GATE_VECTOR ? 64 * LNX_LDA : 0);  // + dA (vector gate)
  // vector-gate epilogue inside the tile region: G and out [64][LDF] fp32, K rows [64][LDC]
  static constexpr size_t vec_bytes = sizeof(float) * 2 * 64 * LDF + sizeof(T) * kTile;
  static_assert(GATE != LNX_GATE_VECTOR || vec_bytes <= sizeof(T) * 5 * kTile, "epilogue tiles overlay the loop tiles");
  // tiles: Tm^T, dW/dD slab, dB slab, K/V slab, and the W/U slab (vector gate) or all K slabs but the last kept
  // for the epilogue (other gates; 4-byte inputs with dk <= 128 read K again instead, so that two workgroups fit a CU)
  static constexpr bool KEEP_K = GATE != LNX_GATE_VECTOR && (sizeof(T) == 2 || DK > 128);
  static constexpr int ntile = (GATE == LNX_GATE_VECTOR) ? 5 : KEEP_K ? 4 + (DK / 64 - 1) : 4;
  // vector gate, 2-byte inputs, dk = 128: the second half's dBw fragments wait in LDS while the first half's pair sums
  // run (one value per thread and fragment element; in registers they went to scratch memory)
  static constexpr bool STASH = GATE == LNX_GATE_VECTOR && sizeof(T) == 2 && DK == 128;
  static constexpr size_t stash_off = sizeof(T) * ntile * kTile + sizeof(float) * nfloat;
  static constexpr size_t bytes = stash_off + (STASH ? sizeof(float) * 16 * 256 : 0);
};

// GRAW (per-channel gate only): the gate was activated inside the op from the raw projection; dg goes on through the
// activation to d_gate_raw and to the per-chunk partial sums of the parameter gradients.
template <typename T, int DK, int GATE, bool GRAW = false>
__global__ __launch_bounds__(256, (sizeof(T) == 2 ? (GATE == LNX_GATE_VECTOR || DK > 128 ? 2 : 3) : (GATE == LNX_GATE_VECTOR || DK > 128 ? 1 : 2))) void bwd_wy2_kernel(BwdParams p) {
  typedef Wy2Cfg<T, DK, GATE> L;
  constexpr int LDC = L::LDC, LDF = L::LDF, NKS = DK / 64;
  extern __shared__ __align__(16) char smem[];
  float* sG = reinterpret_cast<float*>(smem);
  float* sBeta = sG + 64;
  float* sdB = sBeta + 64;   // dbeta: <dBu, v>
  float* sdGk = sdB + 64;    // e^{G} <dBw, k>
  float* sRow = sdGk + 64;   // sum_j dA_ij E_ij X_ij
  float* sCol = sRow + 64;   // sum_i beta_i dA_ij E_ij X_ij
  float* sR = sCol + 64;     // vector gate only: dA, then beta dA  [64][LNX_LDA]
  T* sTmT = reinterpret_cast<T*>(smem + sizeof(float) * L::nfloat);
  T* sIn = sTmT + L::kTile;   // dW / dD slab      [token][col]
  T* sdBt = sIn + L::kTile;   // dB slab           [token][col]
  T* sKs = sdBt + L::kTile;   // K / V slab        [token][col]
  T* sWU = sKs + L::kTile;    // W / U slab        [token][col]; vector gate only
  T* sK0 = sWU;               // other gates: the K slabs before the last stay here until the epilogue

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int N = p.geom.N;
  const int64_t slot = blockIdx.x;
  const int row = (int)(slot / N), n = (int)(slot % N);
  int tok0, len;
  chunk_span(p.geom, n, tok0, len);
  // fused gate activation: this chunk's row of the parameter-gradient partial sums, columns of this head
  auto gate_part = [&](int which) {
    const int64_t gD = (int64_t)p.geom.H * DK;
    return p.gpart + (which * (p.gprows + LNX_SUM_SLICES) + (int64_t)(row / p.geom.H) * N + n) * gD + (row % p.geom.H) * DK;
  };
  if (len <= 0) {  // an unused slot of a packed batch: its partial sums are zero
    if constexpr (GRAW)
      for (int c = tid; c < DK; c += 256) gate_part(0)[c] = gate_part(1)[c] = 0.f;
    return;
  }
  const int64_t tbase = tok_index(p.geom, row, tok0);
  const int64_t ts = p.geom.ts, tsk = ts * DK, tsv = ts * p.dv;  // token stride, row strides of the token tiles
  const T* kg = reinterpret_cast<const T*>(p.k) + tbase * DK;
  const T* vg = reinterpret_cast<const T*>(p.v) + tbase * p.dv;
  const int wi = wave >> 1, wj = wave & 1;
  // The head's gate scale -e^{A_log}, fetched here: a load issued behind the epilogue's stores would have to wait for
  // every one of them to be acknowledged (the memory counter retires in order).
  float gna = 0.f;
  if constexpr (GRAW) gna = -__expf(p.gA[row % p.geom.H]);
  // V slabs first, K slabs last: without a per-channel gate the K slabs then stay in LDS for the epilogue
  const int nvs = p.dv / 64, nslab = NKS + nvs;
  constexpr bool KEEP_K = L::KEEP_K;
  constexpr bool RESTAGE = GATE != LNX_GATE_VECTOR && !KEEP_K;  // K slabs staged again in the epilogue

  // dA needs M = dBw W^T + dBu U^T.  With a per-channel gate W and U are read back from the workspace.  Otherwise
  // W = Tm diag(beta e^G) K and U = Tm diag(beta) V give M = (Zw diag(beta e^G) + Zu diag(beta)) Tm^T with
  // Zw = dBw K^T and Zu = dBu V^T summed over the slabs already in LDS: W and U are never loaded.
  constexpr bool LOAD_WU = GATE == LNX_GATE_VECTOR;
  TileRegs<T, 64, 64> rIn, rWU, rKs;  // dW / dD slab [token][col], W / U slab, K / V slab
  auto fetch = [&](int s_) {
    if (s_ >= nvs) {
      const int c0 = 64 * (s_ - nvs);
      rIn.load(wsp<T>(p, p.off.dW) + slot * 64 * DK + c0, DK, 64, tid);
      if (LOAD_WU) rWU.load(wsp<T>(p, p.off.W) + slot * 64 * DK + c0, DK, 64, tid);
      rKs.load(kg + c0, tsk, len, tid);
    } else {
      const int v0 = 64 * s_;
      rIn.load(wsp<T>(p, p.off.dD) + slot * 64 * p.dv + v0, p.dv, 64, tid);
      if (LOAD_WU) rWU.load(wsp<T>(p, p.off.U) + slot * 64 * p.dv + v0, p.dv, 64, tid);
      rKs.load(vg + v0, tsv, len, tid);
    }
  };
  floatx16 aBw[NKS][1][1], aM[1][1], aZu[1][1];  // aM doubles as Zw inside the loop
  floatx16 aX[1][1];                             // X = K K^T: summed in the loop when the K slabs are not kept
  frag_zero(aX);
#pragma unroll
  for (int s_ = 0; s_ < NKS; ++s_) frag_zero(aBw[s_]);
  frag_zero(aM);
  frag_zero(aZu);

  fetch(0);  // first, so that the small loads below do not hold it up
  if (tid < 64) {
    sG[tid] = (GATE == LNX_GATE_SCALAR) ? wsp<float>(p, p.off.G)[slot * 64 + tid] : 0.f;
    sBeta[tid] = (tid < len) ? p.beta[tbase + tid * ts] : 0.f;
    sdB[tid] = 0.f;
    sdGk[tid] = 0.f;
    sRow[tid] = 0.f;
    sCol[tid] = 0.f;
  }
  stage_tile<T, 64, 64>(sTmT, LDC, wsp<T>(p, p.off.TmT) + slot * 64 * 64, 64, 64, tid);

#pragma unroll 1
  for (int s_ = 0; s_ < nslab; ++s_) {
    const bool is_k = s_ >= nvs;
    // the K/V slab tile of this iteration: the K slabs before the last go to tiles of their own when they are kept
    T* sKc = (KEEP_K && s_ >= nvs && s_ + 1 < nslab) ? sK0 + (s_ - nvs) * L::kTile : sKs;
    lds_barrier();
    rIn.store(sIn, LDC, tid);
    if (LOAD_WU) rWU.store(sWU, LDC, tid);
    rKs.store(sKc, LDC, tid);
    lds_barrier();
    if (s_ + 1 < nslab) fetch(s_ + 1);
    floatx16 b[1][1];
    frag_zero(b);
    mma_x<T, 1, 1, false, true>(b, sTmT + 32 * wi * LDC, LDC, sIn + 32 * wj, LDC, 64, lane);
    frag_store<T, 1, 1>(b, sdBt + 32 * wi * LDC + 32 * wj, LDC, lane);
    if (is_k) {
#pragma unroll
      for (int u = 0; u < NKS; ++u)
        if (u == s_ - nvs) {
#pragma unroll
          for (int e = 0; e < 16; ++e) aBw[u][0][0][e] = b[0][0][e];
        }
    }
    lds_barrier();
    if (LOAD_WU) mma_nt<T, 1, 1>(aM, sdBt + 32 * wi * LDC, LDC, sWU + 32 * wj * LDC, LDC, 64, lane);
    else if (is_k) mma_nt<T, 1, 1>(aM, sdBt + 32 * wi * LDC, LDC, sKc + 32 * wj * LDC, LDC, 64, lane);
    else mma_nt<T, 1, 1>(aZu, sdBt + 32 * wi * LDC, LDC, sKc + 32 * wj * LDC, LDC, 64, lane);
    if (RESTAGE && is_k && !(wi == 0 && wj == 1))
      mma_nt<T, 1, 1>(aX, sKc + 32 * wi * LDC, LDC, sKc + 32 * wj * LDC, LDC, 64, lane);
    if (GATE != LNX_GATE_VECTOR || !is_k) {  // <dB row, k row> / <dB row, v row>; thread = (row, quarter of the slab)
      const int r = tid >> 2, q0 = (tid & 3) * 16;
      float t = 0.f;
#pragma unroll
      for (int u = 0; u < 16; u += 4) {
        const floatx4 b4 = load4(sdBt + r * LDC + q0 + u), k4 = load4(sKc + r * LDC + q0 + u);
#pragma unroll
        for (int e = 0; e < 4; ++e) t += b4[e] * k4[e];
      }
      t += __shfl_xor(t, 1, LNX_WAVE);
      t += __shfl_xor(t, 2, LNX_WAVE);
      if ((tid & 3) == 0) (is_k ? sdGk : sdB)[r] += t;  // row r has this one writer in every phase
    }
    if (!is_k) {  // dv = beta dBu, 16-byte stores
      constexpr int VN = Vec16<T>::N;
      T* dvg = reinterpret_cast<T*>(p.dv_out) + tbase * p.dv + 64 * s_;
      for (int idx = tid; idx < 64 * 64 / VN; idx += 256) {
        const int r = idx / (64 / VN), c = (idx % (64 / VN)) * VN;
        if (r < len) {
          typename Vec16<T>::V x = *reinterpret_cast<const typename Vec16<T>::V*>(sdBt + r * LDC + c);
#pragma unroll
          for (int e = 0; e < VN; ++e) x[e] = from_f32<T>(to_f32(x[e]) * sBeta[r]);
          *reinterpret_cast<typename Vec16<T>::V*>(dvg + (int64_t)r * tsv + c) = x;
        }
      }
    }
  }
  if constexpr (GATE == LNX_GATE_VECTOR) {
    lds_barrier();  // loop tiles dead
    // ---- per-channel gate: the pair terms of dk and dG, one 64-channel half at a time ----
    float* sGc = reinterpret_cast<float*>(sTmT);     // [64][LDF] cumulative gate of the half
    float* sOut = sGc + 64 * LDF;                    // [64][LDF] row-type part of dk, then the column-type part
    T* sKr = reinterpret_cast<T*>(sOut + 64 * LDF);  // K rows [64][LDC]
    T* sXp = reinterpret_cast<T*>(sOut);             // X = <k_i, k_j>_E from the forward pass, until out is needed
    const float* Gg = wsp<float>(p, p.off.G) + slot * 64 * DK;
    float* dGg = wsp<float>(p, p.off.dG) + slot * 64 * DK;
    T* dkg = reinterpret_cast<T*>(p.dk) + tbase * DK;
    stage_tile<T, 64, 64>(sXp, LDC, wsp<T>(p, p.off.X) + slot * 64 * 64, 64, 64, tid);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = 32 * wi + frag_row(e, lane), j = 32 * wj + frag_col(lane);
      sR[i * LNX_LDA + j] = (i > j) ? -aM[0][0][e] : 0.f;  // dA
    }
    float* sStash = reinterpret_cast<float*>(smem + L::stash_off);
    if constexpr (L::STASH) {
#pragma unroll
      for (int e = 0; e < 16; ++e) sStash[e * 256 + tid] = aBw[NKS - 1][0][0][e];
    }
    lds_barrier();
    {  // dbeta += sum_j dA_ij X_ij, then dX = beta_i dA_ij in place; thread = (row, quarter of the columns)
      const int r = tid >> 2, j0 = (tid & 3) * 16;
      float rs = 0.f;
#pragma unroll
      for (int u = 0; u < 16; u += 4) {
        const floatx4 a4 = load4(sR + r * LNX_LDA + j0 + u), x4 = load4(sXp + r * LDC + j0 + u);
#pragma unroll
        for (int e = 0; e < 4; ++e) rs += a4[e] * x4[e];
        store4(sR + r * LNX_LDA + j0 + u, a4 * sBeta[r]);
      }
      rs += __shfl_xor(rs, 1, LNX_WAVE);
      rs += __shfl_xor(rs, 2, LNX_WAVE);
      if ((tid & 3) == 0) sdB[r] += rs;
    }
#pragma unroll 1
    for (int h = 0; h < DK / 64; ++h) {
      const int ch0 = 64 * h;
      floatx4 dk0[4], dg0[4], up[4];
      lds_barrier();  // X tile / the previous half's tiles are dead
      auto fetch_partial = [&]() {  // what bwd_dqk left of dk and dG for this half
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
          dk0[it] = (r < len) ? load4(dkg + (int64_t)r * tsk + ch0 + c) : floatx4{0.f, 0.f, 0.f, 0.f};
          dg0[it] = load4(dGg + r * DK + ch0 + c);
        }
      };
#pragma unroll
      for (int it = 0; it < 4; ++it) {  // all global reads of the half first
        const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
        up[it] = load4(Gg + r * DK + ch0 + c);
      }
      fetch_partial();
      stage_tile<T, 64, 64>(sKr, LDC, kg + ch0, tsk, len, tid);
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
        store4(sGc + r * LDF + c, up[it]);
      }
      lds_barrier();
      if (L::STASH && h == NKS - 1) {  // out = e^G dBw
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int r = 32 * wi + frag_row(e, lane), c = 32 * wj + frag_col(lane);
          sOut[r * LDF + c] = sStash[e * 256 + tid] * __expf(sGc[r * LDF + c]);
        }
      } else {
#pragma unroll
        for (int u = 0; u < NKS; ++u)
          if (u == h) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int r = 32 * wi + frag_row(e, lane), c = 32 * wj + frag_col(lane);
              sOut[r * LDF + c] = aBw[u][0][0][e] * __expf(sGc[r * LDF + c]);
            }
          }
      }
      lds_barrier();
      {  // dbeta += <e^G dBw, k>;  out = beta e^G dBw; thread = (row, quarter of the channels)
        const int r = tid >> 2, q0 = (tid & 3) * 16;
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < 16; u += 4) {
          const floatx4 o4 = load4(sOut + r * LDF + q0 + u), k4 = load4(sKr + r * LDC + q0 + u);
#pragma unroll
          for (int e = 0; e < 4; ++e) t += o4[e] * k4[e];
          store4(sOut + r * LDF + q0 + u, o4 * sBeta[r]);
        }
        t += __shfl_xor(t, 1, LNX_WAVE);
        t += __shfl_xor(t, 2, LNX_WAVE);
        if ((tid & 3) == 0) sdB[r] += t;
      }
      lds_barrier();
      float pr[16], pc[16];
      const int pch = 16 * wave + (lane & 15), ptok = 4 * (lane >> 4);  // this lane's channel; its tokens are 16 t + ptok + e
      constexpr bool LEVELS = DK <= 128;  // beyond that the live accumulators leave too few registers for it
      if constexpr (sizeof(T) == 2 && LEVELS) {  // both pair sums of dA together on the bf16 MFMA
        pair_levels<true>(pr, pc, sR, sGc, LDF, sKr, LDC, sKr, LDC, tid);
#pragma unroll
        for (int x = 0; x < 16; ++x) sOut[(16 * (x >> 2) + ptok + (x & 3)) * LDF + pch] += pr[x];
      } else {
        pair_row<T, 64, true>(sOut, sR, sGc, LDF, sKr, LDC, 1.f, tid);
      }
      lds_barrier();
#pragma unroll
      for (int it = 0; it < 4; ++it) {  // row-type part to registers, out restarts from zero
        const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
        up[it] = load4(sOut + r * LDF + c);
        if (!(sizeof(T) == 2 && LEVELS)) store4(sOut + r * LDF + c, floatx4{0.f, 0.f, 0.f, 0.f});
      }
      lds_barrier();
      if constexpr (sizeof(T) == 2 && LEVELS) {
#pragma unroll
        for (int x = 0; x < 16; ++x) sOut[(16 * (x >> 2) + ptok + (x & 3)) * LDF + pch] = pc[x];
      } else {
        pair_col<T, 64, true>(sOut, sR, sGc, LDF, sKr, LDC, 1.f, tid);
      }
      lds_barrier();
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int idx = tid + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
        const floatx4 um = load4(sOut + r * LDF + c), kk = load4(sKr + r * LDC + c);
        if (r < len) store4(dkg + (int64_t)r * tsk + ch0 + c, dk0[it] + up[it] + um);
        store4(sOut + r * LDF + c, dg0[it] + kk * (up[it] - um));  // dG of this half, in place of the column-type part
      }
      lds_barrier();
      // From here to the end of the half every index is derived from a thread id that has passed through an empty asm:
      // addresses formed outside the loop over the halves are spilled across its first part, and a reload behind the
      // stores of dk waits until every one of them has been acknowledged (the memory counter retires in order).
      int tl = tid;
      asm volatile("" : "+v"(tl));
      {  // dg = reverse cumulative sum of dG over the chunk, per channel: 16-token segments in parallel, then their offsets
        const int c = tl & 63, seg = tl >> 6;
        float acc = 0.f;  // running sums written back in place: no array of sixteen values held across the barrier
#pragma unroll 4
        for (int i = 15; i >= 0; --i) {
          acc += sOut[(16 * seg + i) * LDF + c];
          sOut[(16 * seg + i) * LDF + c] = acc;
        }
        float* sSeg = reinterpret_cast<float*>(sKr);  // segment totals [4][64]: the K tile is dead
        sSeg[seg * 64 + c] = acc;
        lds_barrier();
        float off = 0.f;
        for (int s_ = seg + 1; s_ < 4; ++s_) off += sSeg[s_ * 64 + c];
#pragma unroll 4
        for (int i = 0; i < 16; ++i) sOut[(16 * seg + i) * LDF + c] += off;
      }
      // dg leaves by rows: thread = (row tid / 16 + 16 it, four channels), 16-byte accesses (one channel per lane and
      // token, as in the pass above, makes four times as many memory instructions).  With the gate activated inside
      // the op, g = -e^{A_log} softplus(x), x = raw + bias (kda.py:153-165), the gradient goes on to the raw projection,
      // d_raw = dg (-e^{A_log}) softplus'(x), and the rows add to the channel's sums of d_raw (-> d_bias) and of dg g
      // (-> d_A_log).  Neither x nor a logarithm is needed for that: the activated gate is the difference of two rows of
      // the cumulative gate in LDS, g_t = G_t - G_{t-1}, and with s = softplus(x) = g / -e^{A_log} the derivative is
      // sigmoid(x) = 1 - e^{-s}; beyond the threshold s = x and the derivative is 1.  That needs s to tell the branch:
      // true when softplus(threshold) rounds to the threshold (from about 15 on; the reference's default is 20).  A lower
      // threshold leaves a band of s that both branches reach; then (gband) x is read again and decides.
      lds_barrier();
      if constexpr (!GRAW) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int idx = tl + 256 * it, r = idx >> 4, c = (idx & 15) * 4;
          if (r < len) store4(p.dg + (tbase + (int64_t)r * ts) * DK + ch0 + c, load4(sOut + r * LDF + c));
        }
      } else {
        const int c = (tl & 15) * 4;
        const float na = gna, inv_na = 1.f / na;
        floatx4 sb = {0.f, 0.f, 0.f, 0.f}, sa = sb;
        typedef typename Mma<T>::Quad Quad;  // four elements of T
        const int r0 = tl >> 4;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int r = r0 + 16 * it;
          const floatx4 dgv = load4(sOut + r * LDF + c);
          floatx4 gv = load4(sGc + r * LDF + c);
          if (r > 0) gv = gv - load4(sGc + (r - 1) * LDF + c);
          floatx4 xv = {0.f, 0.f, 0.f, 0.f};  // x = raw + bias, fetched where it is used: the unusual case may wait
          if (p.gband) {
            if (p.gbias) xv = load4(p.gbias + (row % p.geom.H) * DK + ch0 + c);
            const Quad rq = *reinterpret_cast<const Quad*>(reinterpret_cast<const T*>(p.graw) + (tbase + (int64_t)min(r, len - 1) * ts) * DK + ch0 + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) xv[e] += to_f32(rq[e]);
          }
          floatx4 dr;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float sp = gv[e] * inv_na;
            const bool lin = p.gband ? xv[e] > p.gthr : sp > p.gthr;
            const float ds = lin ? 1.f : 1.f - __expf(-sp);
            dr[e] = r < len ? dgv[e] * na * ds : 0.f;
            sb[e] += dr[e];
            sa[e] += r < len ? dgv[e] * gv[e] : 0.f;
          }
          if (r < len) store4(reinterpret_cast<T*>(p.dgraw) + (tbase + (int64_t)r * ts) * DK + ch0 + c, dr);
        }
        float* sPart = reinterpret_cast<float*>(sKr);  // [2][16 row groups][64]: the K tile is dead, the segment totals read
        store4(sPart + r0 * 64 + c, sb);
        store4(sPart + 1024 + r0 * 64 + c, sa);
        lds_barrier();
        if (tl < 128) {  // the sixteen row groups in a fixed order
          const float* src = sPart + (tl >> 6) * 1024 + (tl & 63);
          float t = 0.f;
#pragma unroll
          for (int q = 0; q < 16; ++q) t += src[64 * q];
          gate_part(tl >> 6)[ch0 + (tl & 63)] = t;
        }
      }
    }
    if (tid < 64 && tid < len) p.dbeta[tbase + tid * ts] = sdB[tid];
    return;
  }
  // The K slabs are still in LDS (the last one in the slab tile, the others in tiles of their own); the partial dk of
  // bwd_dqk is fetched one slab at a time.
  TileRegs<T, 64, 64> rdk;
  auto k_tile = [&](int u) -> const T* { return (KEEP_K && u + 1 < NKS) ? sK0 + u * L::kTile : sKs; };
  lds_barrier();  // loop tiles dead
  {  // M = (Zw diag(beta e^G) + Zu diag(beta)) Tm^T
    floatx16 z[1][1];
    const int j = 32 * wj + frag_col(lane);
    const float cu = sBeta[j], cw = (GATE == LNX_GATE_NONE) ? cu : cu * __expf(sG[j]);
#pragma unroll
    for (int e = 0; e < 16; ++e) z[0][0][e] = aM[0][0][e] * cw + aZu[0][0][e] * cu;
    frag_store<T, 1, 1>(z, sIn + 32 * wi * LDC + 32 * wj, LDC, lane);
    frag_zero(aM);
    lds_barrier();
    mma_x<T, 1, 1, false, true>(aM, sIn + 32 * wi * LDC, LDC, sTmT + 32 * wj, LDC, 64, lane);
    lds_barrier();  // Z is overwritten below
  }
  T* sYa = sIn;   // beta dA E (strictly lower); its transpose is read through the same tile
  {
    floatx16 y[1][1];
    if (!RESTAGE && !(wi == 0 && wj == 1)) {
#pragma unroll
      for (int u = 0; u < NKS; ++u) {
        const T* sKT = k_tile(u);
        mma_nt<T, 1, 1>(aX, sKT + 32 * wi * LDC, LDC, sKT + 32 * wj * LDC, LDC, 64, lane);
      }
    }
    float v[16], cs = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int i = 32 * wi + frag_row(e, lane), j = 32 * wj + frag_col(lane);
      const float dec = (GATE == LNX_GATE_NONE) ? 1.f : __expf(fminf(sG[i] - sG[j], 0.f));
      const float da = (i > j) ? -aM[0][0][e] * dec : 0.f;
      v[e] = da * aX[0][0][e];
      cs += sBeta[i] * v[e];
      y[0][0][e] = sBeta[i] * da;
    }
    frag_store<T, 1, 1>(y, sYa + 32 * wi * LDC + 32 * wj, LDC, lane);
    // two waves add to each entry of sRow (wj = 0, 1) and of sCol (wi = 0, 1), both zeroed above: 0 + a + b is the same
    // number in either order, so these sums do not depend on which wave arrives first
    rows_reduce_add<1>(v, 32 * wi, lane, sRow);
    cs += __shfl_xor(cs, 32, LNX_WAVE);
    if (lane < 32) atomicAdd(&sCol[32 * wj + lane], cs);
  }
  lds_barrier();
#pragma unroll
  for (int u = 0; u < NKS; ++u) {
    const T* sKT = k_tile(u);
    rdk.load(reinterpret_cast<const T*>(p.dk) + tbase * DK + 64 * u, tsk, len, tid);  // partial dk of bwd_dqk
    if (RESTAGE) {
      if (u > 0) lds_barrier();  // the previous slab's K tile has been read
      stage_tile<T, 64, 64>(sKs, LDC, kg + 64 * u, tsk, len, tid);
      lds_barrier();
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int r = 32 * wi + frag_row(e, lane);
      const float gm = (GATE == LNX_GATE_NONE) ? 1.f : __expf(sG[r]);
      aBw[u][0][0][e] *= sBeta[r] * gm;
    }
    mma_x<T, 1, 1, false, true>(aBw[u], sYa + 32 * wi * LDC, LDC, sKT + 32 * wj, LDC, 64, lane);
    mma_x<T, 1, 1, true, true>(aBw[u], sYa + 32 * wi, LDC, sKT + 32 * wj, LDC, 64, lane);
    if (u > 0) lds_barrier();
    frag_store<T, 1, 1>(aBw[u], sdBt + 32 * wi * LDC + 32 * wj, LDC, lane);
    lds_barrier();
    {
      constexpr int VN = Vec16<T>::N, VPR = 64 / VN;
      T* dkg = reinterpret_cast<T*>(p.dk) + tbase * DK + 64 * u;
#pragma unroll
      for (int it = 0; it < TileRegs<T, 64, 64>::IT; ++it) {
        const int idx = tid + 256 * it, r = idx / VPR, c = (idx % VPR) * VN;
        if (r < len) {
          typename Vec16<T>::V x = *reinterpret_cast<const typename Vec16<T>::V*>(sdBt + r * LDC + c);
#pragma unroll
          for (int e = 0; e < VN; ++e) x[e] = from_f32<T>(to_f32(x[e]) + to_f32(rdk.x[it][e]));
          *reinterpret_cast<typename Vec16<T>::V*>(dkg + (int64_t)r * tsk + c) = x;
        }
      }
    }
  }
  // dbeta and dg
  if (wave == 0) {
    const int t = lane;
    const float gm = (GATE == LNX_GATE_NONE) ? 1.f : __expf(sG[t]);
    const float w = gm * sdGk[t], rs = sRow[t];
    if (t < len) p.dbeta[tbase + t * ts] = sdB[t] + w + rs;
    if (GATE != LNX_GATE_NONE) {
      float d = 0.f;  // bwd_dqk's share, one slot per 64-channel part
#pragma unroll
      for (int part = 0; part < DK / 64; ++part) d += wsp<float>(p, p.off.dG)[((int64_t)part * p.geom.rows * p.geom.N + slot) * 64 + t];
      d += sBeta[t] * (w + rs) - sCol[t];
#pragma unroll
      for (int s_ = 1; s_ < 64; s_ <<= 1) {
        const float y = __shfl_down(d, s_, LNX_WAVE);
        if (t + s_ < 64) d += y;
      }
      if (t < len) p.dg[tbase + t * ts] = d;
    }
  }
}


template <typename T, int DK, int GATE>
int launch_bwd(const BwdParams& p, int nstate, hipStream_t st) {
  const int64_t slots = (int64_t)p.geom.rows * p.geom.N;
  // 32-column slabs when 64-column ones would leave more than half of the CUs without a workgroup (2-byte inputs with
  // dk >= 128, 4-byte inputs with dk = 128; 4-byte inputs with dk = 256 always get 32 columns from BScanCfg)
  constexpr bool can_narrow = (DK >= 128 && sizeof(T) == 2) || (DK == 128 && sizeof(T) == 4);
  constexpr int WIDE = 64, NARROW = can_narrow ? 32 : WIDE;
  const bool narrow = can_narrow && lnx_narrow_slabs((int64_t)nstate * p.geom.H * (p.dv / 64), p.slab);
  auto k1 = narrow ? bwd_scan_kernel<T, DK, GATE, NARROW> : bwd_scan_kernel<T, DK, GATE, WIDE>;
  const int bv = narrow ? BScanCfg<T, DK, NARROW>::BV : BScanCfg<T, DK, WIDE>::BV;
  auto k2 = bwd_dqk_kernel<T, DK, GATE>;
  auto k3 = (GATE == LNX_GATE_VECTOR && p.graw) ? bwd_wy2_kernel<T, DK, GATE, GATE == LNX_GATE_VECTOR> : bwd_wy2_kernel<T, DK, GATE>;
  const size_t b1 = narrow ? BScanCfg<T, DK, NARROW>::bytes : BScanCfg<T, DK, WIDE>::bytes;
  const size_t b2 = DqkCfg<T, DK, GATE>::bytes, b3 = Wy2Cfg<T, DK, GATE>::bytes;
  hipError_t e;
  if ((e = hipFuncSetAttribute((const void*)k1, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b1)) != hipSuccess ||
      (e = hipFuncSetAttribute((const void*)k2, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b2)) != hipSuccess ||
      (e = hipFuncSetAttribute((const void*)k3, hipFuncAttributeMaxDynamicSharedMemorySize, (int)b3)) != hipSuccess)
    return lnx_set_error(LNX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  if (!BScanCfg<T, DK>::FUSE_LOCAL) {  // otherwise bwd_scan forms the chunk-local part itself
    lnx_profile_mark("bwd_local", st);
    hipLaunchKernelGGL(bwd_local_kernel<T>, dim3(lnx_xcd_grid(slots, p.dv / 64)), dim3(256), 0, st, p);
  }
  lnx_profile_mark("bwd_scan", st);
  hipLaunchKernelGGL(k1, dim3(lnx_xcd_grid((int64_t)nstate * p.geom.H, p.dv / bv)), dim3(512), b1, st, p);
  lnx_profile_mark("bwd_dqk", st);
  hipLaunchKernelGGL(k2, dim3(lnx_xcd_grid(slots, DK / 64)), dim3(256), b2, st, p);
  lnx_profile_mark("bwd_wy", st);
  hipLaunchKernelGGL(k3, dim3((unsigned)slots), dim3(256), b3, st, p);
  lnx_profile_mark(nullptr, st);
  return LNX_OK;
}

template <typename T, int DK>
int launch_bwd_gate(int gate, const BwdParams& p, int nstate, hipStream_t st) {
  switch (gate) {
    case LNX_GATE_NONE: return launch_bwd<T, DK, LNX_GATE_NONE>(p, nstate, st);
    case LNX_GATE_SCALAR: return launch_bwd<T, DK, LNX_GATE_SCALAR>(p, nstate, st);
    case LNX_GATE_VECTOR: return launch_bwd<T, DK, LNX_GATE_VECTOR>(p, nstate, st);
    default: return lnx_set_error(LNX_ERR_SHAPE, "unknown gate kind %d", gate);
  }
}

__global__ void copy_dstate_kernel(const float* src, float* dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src ? src[i] : 0.f;
}

}  // namespace

extern "C" int lnx_chunk_bwd(const lnx_scan_args* a, void* stream) {
  int rc = lnx_chunk_check(a, true);
  if (rc != LNX_OK) return rc;
  hipStream_t st = (hipStream_t)stream;
  const bool packed = a->cu_seqlens != nullptr;
  const int nstate = packed ? a->nseq : a->B;
  if (nstate == 0) return LNX_OK;
  if (a->T == 0) {
    if (a->d_initial_state) {
      const int64_t n = (int64_t)nstate * a->H * a->dk * a->dv;
      hipLaunchKernelGGL(copy_dstate_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a->d_final_state,
                         a->d_initial_state, n);
    }
    return LNX_OK;
  }
  const ChunkWs w = lnx_chunk_ws_layout(a);
  if (reinterpret_cast<uintptr_t>(a->workspace) & 15) return lnx_set_error(LNX_ERR_WORKSPACE, "the workspace must be 16-byte aligned");
  if (!a->workspace || a->workspace_bytes < w.total)
    return lnx_set_error(LNX_ERR_WORKSPACE, "workspace of %llu bytes needed, %llu given", (unsigned long long)w.total,
                         (unsigned long long)a->workspace_bytes);
  BwdParams p;
  p.geom.H = a->H; p.geom.T = a->T; p.geom.N = lnx_chunk_slots(a); p.geom.nseq = a->nseq;
  p.geom.ts = a->token_first ? a->H : 1;
  p.geom.rows = packed ? a->H : a->B * a->H;
  p.geom.cu = a->cu_seqlens;
  p.geom.tab = packed ? reinterpret_cast<const int32_t*>(reinterpret_cast<char*>(a->workspace) + w.tab) : nullptr;
  p.q = a->q; p.k = a->k; p.v = a->v; p.beta = a->beta; p.d_o = a->d_o; p.d_sT = a->d_final_state;
  p.dq = a->d_q; p.dk = a->d_k; p.dv_out = a->d_v; p.dbeta = a->d_beta; p.dg = a->d_g; p.ds0 = a->d_initial_state;
  p.dv = a->dv; p.gate = a->gate; p.scale = a->scale; p.slab = a->test_scan_slab;
  const bool raw_gate = a->gate == LNX_GATE_VECTOR && a->gate_raw != nullptr;
  p.graw = raw_gate ? a->gate_raw : nullptr; p.gA = a->gate_A_log; p.gbias = a->gate_bias; p.gthr = a->gate_threshold;
  p.gband = a->gate_threshold + log1pf(expf(-a->gate_threshold)) != a->gate_threshold;
  p.dgraw = a->d_gate_raw;
  p.gprows = (int64_t)(packed ? 1 : a->B) * lnx_chunk_slots(a);
  p.gpart = raw_gate ? reinterpret_cast<float*>(reinterpret_cast<char*>(a->workspace) + w.gpart) : nullptr;
  p.ws = reinterpret_cast<char*>(a->workspace); p.off = w;
  if (lnx_chunk_direct(a)) {
    DirectParams d = {};
    d.geom = p.geom;
    d.q = reinterpret_cast<const bf16_t*>(a->q); d.k = reinterpret_cast<const bf16_t*>(a->k);
    d.v = reinterpret_cast<const bf16_t*>(a->v); d.beta = a->beta; d.dv = a->dv; d.vcols = a->dv; d.gate = a->gate;
    d.l2norm = a->use_qk_l2norm; d.slab = a->test_scan_slab;
    d.scale = a->scale; d.ws = p.ws; d.off = w;
    d.d_o = reinterpret_cast<const bf16_t*>(a->d_o); d.d_sT = a->d_final_state;
    d.dq = reinterpret_cast<bf16_t*>(a->d_q); d.dk = reinterpret_cast<bf16_t*>(a->d_k);
    d.dv_out = reinterpret_cast<bf16_t*>(a->d_v); d.dbeta = a->d_beta; d.dg = a->d_g; d.ds0 = a->d_initial_state;
    rc = lnx_direct_bwd(d, a->dk, a->gate, nstate, st);
    if (rc != LNX_OK) return rc;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "chunk backward launch: %s", hipGetErrorString(e));
    return LNX_OK;
  }
  if (a->dtype == LNX_BF16)  // dk <= 128 without a per-channel gate went to the direct-solve kernels above
    rc = (a->dk == 256)   ? launch_bwd_gate<bf16_t, 256>(a->gate, p, nstate, st)
         : (a->dk == 128) ? launch_bwd<bf16_t, 128, LNX_GATE_VECTOR>(p, nstate, st)
                          : launch_bwd<bf16_t, 64, LNX_GATE_VECTOR>(p, nstate, st);
  else
    rc = (a->dk == 256)   ? launch_bwd_gate<float, 256>(a->gate, p, nstate, st)
         : (a->dk == 128) ? launch_bwd_gate<float, 128>(a->gate, p, nstate, st)
                          : launch_bwd_gate<float, 64>(a->gate, p, nstate, st);
  if (rc != LNX_OK) return rc;
  if (raw_gate && (a->d_gate_A_log || a->d_gate_bias)) {
    lnx_gate_finish_sums(p.gpart, p.gprows, a->H, a->dk, a->d_gate_A_log, a->d_gate_bias, st);
    lnx_profile_mark(nullptr, st);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lnx_set_error(LNX_ERR_LAUNCH, "chunk backward launch: %s", hipGetErrorString(e));
  return LNX_OK;
}
