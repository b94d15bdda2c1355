// Geometry and workspace layout shared by the chunk forward and backward kernels.
//
// A "row" is one (batch, head) pair -- or one head of the packed batch; a row owns N chunk
// slots of 64 tokens.  Dense batch: N = ceil(T / 64), slot n covers tokens [64 n, 64 n + 64).
// Packed batch: chunks restart at every sequence boundary, so N = T / 64 + nseq slots are
// reserved and a table built on the device maps slot -> (first token, length, sequence);
// unused slots have length 0.
//
// Per-slot tensors kept in the workspace (element type T = bf16 or fp32 unless noted), all
// row-major with the token index first; kernels that contract over tokens read them through
// the transposing LDS loads of mma_tiles.h, so no transposed copies are stored:
//   G    fp32 [64] or [64][dk]   cumulative gate inside the chunk
//   P    [64][64]   scale * <q_i, k_j> * exp(G_i - G_j), i >= j
//   W    [64][dk]   (I + A)^-1 diag(beta) (K * exp(G))
//   U    [64][dv]   (I + A)^-1 diag(beta) V
//   TmT  [64][64]   ((I + A)^-1)^T, used by the backward pass
//   D    [64][dv]   U - W S
//   SnT  [dv][dk]   transpose of the state entering the chunk
//   vector gate only:  X [64][64] = <k_i, k_j>_E (i > j),  Kr [64][dk] = K * exp(G_last - G),
//                      Qg [64][dk] = scale * Q * exp(G)
// Backward adds dD [64][dv], dSn [dv][dk] (gradient of the state leaving the chunk, transposed), dW [64][dk]
// and dG (fp32 partial gradient of the cumulative gate).
#pragma once

#include "mma_tiles.h"

struct ChunkGeom {
  int H, T, N, nseq, rows;       // rows = B * H (dense) or H (packed); N = chunk slots per row
  int ts;                        // distance between consecutive tokens of a row, in tokens: 1 ([B,H,T,.]) or H ([B,T,H,.])
  const int32_t* cu;             // device cu_seqlens or nullptr
  const int32_t* tab;            // packed only: [N][2] (token0, len), seq_chunk0[nseq + 1], order[nseq]
};

__device__ __forceinline__ void chunk_span(const ChunkGeom& g, int n, int& tok0, int& len) {
  if (g.tab) {
    tok0 = g.tab[2 * n];
    len = g.tab[2 * n + 1];
  } else {
    tok0 = n * LNX_C;
    len = min(LNX_C, g.T - tok0);
  }
}

// Position of token `tok` of (batch, head) row `row` in units of one token's vector (dk or dv elements, or one
// scalar for beta / g); token tok + 1 of the same row is g.ts further on.
__device__ __forceinline__ int64_t tok_index(const ChunkGeom& g, int row, int tok) {
  return g.ts == 1 ? (int64_t)row * g.T + tok : ((int64_t)(row / g.H) * g.T + tok) * g.H + row % g.H;
}

// The sequential kernels take one workgroup per (state, head): blockIdx.x -> state index and row.
// Packed batches hand the sequences out longest first (order[] of the table), so that the longest
// chains start first when there are more workgroups than fit the chip at once.
__device__ __forceinline__ void scan_state(const ChunkGeom& g, int bx, int& sidx, int& row, int& seq) {
  if (g.tab) {
    seq = g.tab[2 * g.N + g.nseq + 1 + bx / g.H];
    row = bx % g.H;
    sidx = seq * g.H + row;
  } else {
    seq = 0;
    sidx = row = bx;
  }
}

// Chunk-slot range [c0, c1) of state index `s` (batch element or sequence).
__device__ __forceinline__ void seq_chunks(const ChunkGeom& g, int s, int& c0, int& c1) {
  if (g.tab) {
    c0 = g.tab[2 * g.N + s];
    c1 = g.tab[2 * g.N + s + 1];
  } else {
    c0 = 0;
    c1 = g.N;
  }
}

// Token range [t0, t1) of the sequence (or batch row) a sequential kernel works on.  Its chunk slots c0, c0 + 1, ...
// start 64 tokens apart from t0, so the span of a chunk is arithmetic on these three numbers -- the movers of the
// sequential kernels must not read the chunk table per chunk: a load in the address computation of a fetch makes
// the fetch wait for every load issued before it.
struct SeqSpan {
  int t0, t1, c0;
};
__device__ __forceinline__ SeqSpan seq_span(const ChunkGeom& g, int seq, int c0) {
  SeqSpan s;
  s.t0 = g.cu ? seq_first(g.cu, seq, g.T) : 0;
  s.t1 = g.cu ? seq_end(g.cu, seq, g.T) : g.T;
  s.c0 = c0;
  return s;
}
__device__ __forceinline__ void chunk_span(const SeqSpan& s, int n, int& tok0, int& len) {
  tok0 = s.t0 + (n - s.c0) * LNX_C;
  len = min(LNX_C, s.t1 - tok0);
}

// 1-D launch of `parts` workgroups per chunk slot such that the parts of one slot run on the same
// XCD (workgroups are dealt round-robin to the 8 XCDs, each with its own L2) and back to back, so
// the tiles they share are read from HBM once.  Grid size: lnx_xcd_grid(slots, parts).
__device__ __forceinline__ bool xcd_slot_part(int64_t slots, int parts, int64_t& slot, int& part) {
  const int64_t bid = blockIdx.x, rest = bid >> 3;
  part = (int)(rest % parts);
  slot = (rest / parts) * 8 + (bid & 7);
  return slot < slots;
}
inline unsigned lnx_xcd_grid(int64_t slots, int parts) { return (unsigned)(((slots + 7) / 8) * 8 * parts); }

struct ChunkWs {
  uint64_t tab, G, P, X, W, U, Kr, Qg, Tm, Nq, Nk, Fq, TmT, D, SnT, dD, dSn, dW, dG, gpart, total;
};

// kda_gate.hip: partial rows of the fused gate activation's parameter gradients and their reduction
uint64_t lnx_gate_part_bytes(int64_t nrows, int D);
void lnx_gate_finish_sums(float* part, int64_t nrows, int H, int dk, float* d_A_log, float* d_bias, hipStream_t st);

// log(1 + e^x) in the overflow-free form max(x, 0) + log1p(e^-|x|); x itself above the threshold (kda.py:157-163)
__device__ __forceinline__ float lnx_softplus_thr(float x, float thr) {
  return x > thr ? x : fmaxf(x, 0.f) + __logf(1.f + __expf(-fabsf(x)));
}

// 2-byte inputs with dk <= 128 and no per-channel gate take the kernels of chunk_direct.hip, which keep G, Pm, Tm, the
// per-chunk states and state gradients, D and dR in the workspace (no W, U, dW); every other shape takes the WY-split
// kernels.  The choice reads only fields that the forward and the backward call of one step necessarily share (element
// type, dk, gate kind), so both calls lay the workspace out the same way; there is one set of kernels per shape.
inline bool lnx_chunk_direct(const lnx_scan_args* a) {
  return a->dtype == LNX_BF16 && a->dk <= 128 && a->gate != LNX_GATE_VECTOR;
}

inline uint64_t lnx_align256(uint64_t x) { return (x + 255) & ~uint64_t(255); }

inline int lnx_chunk_slots(const lnx_scan_args* a) {
  return a->cu_seqlens ? a->T / LNX_C + a->nseq : (a->T + LNX_C - 1) / LNX_C;
}

// With forward_only the tensors only the backward pass reads (Tm^T, X, D, the entering states for 2-byte inputs,
// whose outputs leave the scan kernel itself) and the backward pass's own scratch are not reserved.
inline ChunkWs lnx_chunk_ws_layout(const lnx_scan_args* a) {
  ChunkWs w;
  const uint64_t es = (a->dtype == LNX_BF16) ? 2 : 4;
  const uint64_t rows = a->cu_seqlens ? (uint64_t)a->H : (uint64_t)a->B * a->H;
  const uint64_t N = (uint64_t)lnx_chunk_slots(a);
  const uint64_t slots = rows * N, dk = a->dk, dv = a->dv, C = LNX_C;
  const bool vec = a->gate == LNX_GATE_VECTOR;
  const bool bwd = !a->forward_only;                      // a backward pass will follow
  const bool saved = bwd || a->dtype != LNX_BF16;         // the forward pass writes its per-chunk tensors
  uint64_t off = 0;
  auto take = [&](uint64_t bytes) { uint64_t o = off; off = lnx_align256(off + bytes); return o; };
  w.tab = take(a->cu_seqlens ? (2 * N + 2 * (uint64_t)a->nseq + 1) * 4 : 0);
  if (lnx_chunk_direct(a)) {
    w.X = w.W = w.U = w.Kr = w.Qg = w.TmT = w.dW = w.dG = w.gpart = 0;
    w.G = take(slots * C * 4);
    w.Nq = take(slots * C * 4);  // 1 / (|q_t| + eps), or 1 when the inputs come normalised
    w.Nk = take(slots * C * 4);
    w.Fq = take(slots * C * 4);  // scale e^{G_t} / (|q_t| + eps): what the scans multiply their Q rows with
    w.P = take(slots * C * C * es);
    w.Tm = take(slots * C * C * es);
    w.SnT = take(bwd ? slots * dv * dk * es : 0);   // states entering the chunks, [v][k]
    w.dSn = take(bwd ? slots * dk * dv * es : 0);   // state gradients leaving the chunks, [v][k]
    w.D = take(bwd ? slots * dv * C * es : 0);      // D^T  [v][token]
    w.dD = take(bwd ? slots * dv * C * es : 0);     // dR^T [v][token]
    w.total = off;
    return w;
  }
  w.Tm = w.Nq = w.Nk = w.Fq = 0;
  w.G = take(vec ? slots * C * dk * 4 : slots * C * 4);
  w.P = take(slots * C * C * es);
  w.X = take(vec && saved ? slots * C * C * es : 0);
  w.W = take(slots * C * dk * es);
  w.U = take(slots * C * dv * es);
  w.Kr = take(vec ? slots * C * dk * es : 0);
  w.Qg = take(vec ? slots * C * dk * es : 0);
  w.TmT = take(saved ? slots * C * C * es : 0);
  w.D = take(saved ? slots * C * dv * es : 0);
  w.SnT = take(saved ? slots * dv * dk * es : 0);
  w.dD = take(bwd ? slots * C * dv * es : 0);
  w.dSn = take(bwd ? slots * dk * dv * es : 0);
  w.dW = take(bwd ? slots * C * dk * es : 0);
  w.dG = take(bwd ? (vec ? slots * C * dk * 4 : slots * C * 4 * (dk / 64)) : 0);  // scalar gate: one slot per 64-channel part
  // fused gate activation: one partial row of its parameter gradients per chunk slot of a (batch element, head)
  w.gpart = take(bwd && vec && a->gate_raw ? lnx_gate_part_bytes((int64_t)(slots / a->H), a->H * a->dk) : 0);
  w.total = off;
  return w;
}

// Slab width of the two sequential kernels: 32 columns when 64-column slabs would give workgroups to at
// most half of the 256 CUs.  `forced` is lnx_scan_args.test_scan_slab: 32 or 64 overrides the choice (the
// tests cover both variants at small shapes with it; the workspace layout does not depend on the width).
inline bool lnx_narrow_slabs(int64_t wide_workgroups, int forced) {
  if (forced == 32) return true;
  if (forced == 64) return false;
  return wide_workgroups <= 128;
}

// Arguments of the kernels of chunk_direct.hip (2-byte inputs).
struct DirectParams {
  ChunkGeom geom;
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  const float* beta;
  const float* s0;
  float* sT_out;
  void* o;
  int dv, o_dtype;
  int save;   // forward scan: write the state entering every chunk (the backward pass reads it)
  int vcols;  // leading value columns present in v (its row length); the rest of the dv columns are zero
  int gate;
  int l2norm;  // q and k rows are normalised inside the kernels (factors from the prepare kernel in Nq, Nk)
  int slab;    // lnx_scan_args.test_scan_slab
  float scale;
  char* ws;
  ChunkWs off;
  // backward only
  const bf16_t* d_o;
  const float* d_sT;
  bf16_t* dq;
  bf16_t* dk;
  bf16_t* dv_out;
  float* dbeta;
  float* dg;
  float* ds0;
};
int lnx_direct_scan_fwd(const DirectParams& p, int dk, int gate, int nstate, hipStream_t st);
int lnx_direct_bwd(const DirectParams& p, int dk, int gate, int nstate, hipStream_t st);

// Shared argument validation of the chunk entry points; returns LNX_OK or an error status.
int lnx_chunk_check(const lnx_scan_args* a, bool backward);


// ---------------------------------------------------------------------------------------
// Vector-gate (KDA) helpers.  The per-channel decays E_ij[c] = exp(G_i[c] - G_j[c]) (i >= j, G the
// cumulative gate inside the chunk, non-increasing along i) sit inside the token sums.  Wherever a
// reference token r with j <= r <= i exists for a whole group of rows, the decay factors as
// E_ij = exp(G_i - G_r) * exp(G_r - G_j), both factors <= 1 (the splitting kda.py:504-523 uses for
// its forward matrices), and the group's sum over j becomes a small matrix product on
// v_mfma_f32_16x16x4_f32 with one operand scaled on the fly (fp32 operands: nothing is rounded to
// bf16 on the way).  Two levels of it: 16-token blocks against everything before (after) them,
// and the 4-token groups inside a block against the earlier (later) groups of that block -- one
// accumulator row group of the MFMA is exactly one such group.  Only the 4x4 triangles on the
// diagonal are left to the VALU (exponents of non-positive numbers).
// Tiles live in LDS: M [64][LNX_LDA] fp32 (already masked to the lower triangle), G and out
// [64][ldf] fp32, operands [64][ldb] in T.  All 256 threads must call; each helper contains one
// workgroup barrier between its two phases (they update `out` with different thread mappings).
// ---------------------------------------------------------------------------------------

// out[i][c] += mul * sum_{j <= i (j < i if STRICT)} M[i][j] * E_ij[c] * b[j][c]
template <typename T, int CH, bool STRICT>
__device__ __forceinline__ void pair_row(float* out, const float* M, const float* G, int ldf, const T* b, int ldb,
                                         float mul, int tid) {
  const int wave = tid >> 6, lane = tid & 63, l16 = lane & 15, kq = lane >> 4;
  for (int cb = wave; cb < CH / 16; cb += 4) {
    const int c = 16 * cb + l16;
#pragma unroll
    for (int I = 0; I < 4; ++I) {
      floatx4 tot = {0.f, 0.f, 0.f, 0.f};
      float gi[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) gi[e] = G[(16 * I + 4 * kq + e) * ldf + c];
      // reference 16 I: all tokens before the block; reference 16 I + 4 a: the block's tokens before group a
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        if (I == 0 && a == 0) continue;
        const int ref = 16 * I + 4 * a, jlo = (a == 0) ? 0 : 16 * I;
        const float gref = G[ref * ldf + c];
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j0 = jlo; j0 < ref; j0 += 4) {
          const int j = j0 + kq;
          const float av = M[(16 * I + l16) * LNX_LDA + j];
          const float bv = to_f32(b[j * ldb + c]) * __expf(fminf(gref - G[j * ldf + c], 0.f));
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc, 0, 0, 0);
        }
        if (a == 0 || kq == a) {  // a > 0: only the rows of group a are meaningful
#pragma unroll
          for (int e = 0; e < 4; ++e) tot[e] += acc[e] * __expf(fminf(gi[e] - gref, 0.f));
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) out[(16 * I + 4 * kq + e) * ldf + c] += mul * tot[e];
    }
  }
  lds_barrier();
  for (int i = wave; i < 64; i += 4) {
    const int jb = i & ~3;
    for (int c = lane; c < CH; c += 64) {
      const float gi = G[i * ldf + c];
      float m[4], gv[4], bv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {  // unconditional loads, masks applied after
        m[u] = M[i * LNX_LDA + jb + u];
        gv[u] = G[(jb + u) * ldf + c];
        bv[u] = to_f32(b[(jb + u) * ldb + c]);
      }
      float acc = 0.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool on = STRICT ? (jb + u < i) : (jb + u <= i);
        acc += on ? m[u] * __expf(fminf(gi - gv[u], 0.f)) * bv[u] : 0.f;
      }
      out[i * ldf + c] += mul * acc;
    }
  }
}

// out[j][c] += mul * sum_{i >= j (i > j if STRICT)} M[i][j] * E_ij[c] * a[i][c]
template <typename T, int CH, bool STRICT>
__device__ __forceinline__ void pair_col(float* out, const float* M, const float* G, int ldf, const T* a, int lda,
                                         float mul, int tid) {
  const int wave = tid >> 6, lane = tid & 63, l16 = lane & 15, kq = lane >> 4;
  for (int cb = wave; cb < CH / 16; cb += 4) {
    const int c = 16 * cb + l16;
#pragma unroll
    for (int J = 0; J < 4; ++J) {
      floatx4 tot = {0.f, 0.f, 0.f, 0.f};
      float gj[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) gj[e] = G[(16 * J + 4 * kq + e) * ldf + c];
      // later 16-token blocks (reference: their first token)
#pragma unroll
      for (int I = J + 1; I < 4; ++I) {
        const float gref = G[16 * I * ldf + c];
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i0 = 16 * I; i0 < 16 * I + 16; i0 += 4) {
          const int i = i0 + kq;
          const float mv = M[i * LNX_LDA + 16 * J + l16];
          const float av = to_f32(a[i * lda + c]) * __expf(fminf(G[i * ldf + c] - gref, 0.f));
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(mv, av, acc, 0, 0, 0);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) tot[e] += acc[e] * __expf(fminf(gref - gj[e], 0.f));
      }
      // later 4-token groups of the same block (reference: the group's first token); only the
      // columns of earlier groups are meaningful
#pragma unroll
      for (int g4 = 1; g4 < 4; ++g4) {
        const int i = 16 * J + 4 * g4 + kq;
        const float gref = G[(16 * J + 4 * g4) * ldf + c];
        const float mv = M[i * LNX_LDA + 16 * J + l16];
        const float av = to_f32(a[i * lda + c]) * __expf(fminf(G[i * ldf + c] - gref, 0.f));
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(mv, av, acc, 0, 0, 0);
        if (kq < g4) {
#pragma unroll
          for (int e = 0; e < 4; ++e) tot[e] += acc[e] * __expf(fminf(gref - gj[e], 0.f));
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) out[(16 * J + 4 * kq + e) * ldf + c] += mul * tot[e];
    }
  }
  lds_barrier();
  for (int j = wave; j < 64; j += 4) {
    const int ib = j & ~3;
    for (int c = lane; c < CH; c += 64) {
      const float gj = G[j * ldf + c];
      float m[4], gv[4], av[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        m[u] = M[(ib + u) * LNX_LDA + j];
        gv[u] = G[(ib + u) * ldf + c];
        av[u] = to_f32(a[(ib + u) * lda + c]);
      }
      float acc = 0.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool on = STRICT ? (ib + u > j) : (ib + u >= j);
        acc += on ? m[u] * __expf(fminf(gv[u] - gj, 0.f)) * av[u] : 0.f;
      }
      out[j * ldf + c] += mul * acc;
    }
  }
}

// ---------------------------------------------------------------------------------------
// pair_levels: both pair sums of a 64-channel tile at once for 2-byte inputs, on the bf16 MFMA, with every decay taken
// once.  For i > j let h be the highest bit in which i and j differ; then m = (i with the bits below h cleared) lies
// in (j, i], and E_ij = exp(G_i - G_m) exp(G_m - G_j) with both factors <= 1.  At "level" h every token has exactly
// one role -- bit h set: a row token i with factor exp(G_i - G_m), clear: a column token j with factor
// exp(G_m - G_j), m = (token with the bits below 2h cleared) + h -- so one exponential per (token, channel, level)
// serves both sums:
//   ro[i][c] = sum_{j < i} X[i][j] E_ij[c] b[j][c] = sum_h  F_h[i][c] * sum_j X_h[i][j] (F_h b)[j][c]
//   co[j][c] = sum_{i > j} X[i][j] E_ij[c] a[i][c] = sum_h  F_h[j][c] * sum_i X_h[i][j] (F_h a)[i][c]
// with X_h the entries of X whose (i, j) belong to level h: whole 16x16 blocks for h = 32, 16, 8, lane-masked diagonal
// blocks for h = 4, 2, 1.  Wave w owns channels 16 w .. 16 w + 15; lane (c = lane % 16, kq = lane / 16) holds the
// sixteen tokens 16 t + 4 kq + e (t, e = 0..3) of its channel, which is at once the k-slot order of the scaled B
// operands of v_mfma_f32_16x16x16_bf16 and the accumulator rows of its results, so factors, operands and results
// never leave the lane.  Not STRICT: the diagonal X[i][i] (E = 1) is added to both sums.
// X [64][LNX_LDA] fp32, G [64][ldf] fp32, b / a [64][ld] bf16, all in LDS; results are per lane, index 4 t + e.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ floatx4 mfma16_bf16(bf16x4 a, bf16x4 b, floatx4 c) {
  typedef short short4_ __attribute__((ext_vector_type(4)));
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_, a), __builtin_bit_cast(short4_, b), c, 0, 0, 0);
}

// A operands from X: block (ti, t) with lane = (row l16, k-slots 4 kq + e), and the same block transposed,
// lane = (column l16, k-slots = rows 4 kq + e)
__device__ __forceinline__ bf16x4 pair_x_rows(const float* __restrict__ X, int ti, int t, int l16, int kq) {
  return pack_bf16x4(load4(X + (16 * ti + l16) * LNX_LDA + 16 * t + 4 * kq));
}
__device__ __forceinline__ bf16x4 pair_x_cols(const float* __restrict__ X, int ti, int t, int l16, int kq) {
  const float* p = X + (16 * ti + 4 * kq) * LNX_LDA + 16 * t + l16;
  return pack_bf16x4(floatx4{p[0], p[LNX_LDA], p[2 * LNX_LDA], p[3 * LNX_LDA]});
}

// Levels 32 and 16: whole 16x16 blocks of X, roles fixed per block -- row blocks (2, 3) against column blocks (0, 1)
// at level 32; (1) against (0) and (3) against (2) at level 16.
template <int H>
__device__ __forceinline__ void pair_cross(float (&ro)[16], float (&co)[16], const float (&g)[16], const float (&dec)[16],
                                           const float (&bv)[16], const float (&av)[16], const float* __restrict__ X,
                                           const float* __restrict__ G, int ldf, int c, int l16, int kq) {
  constexpr float LOG2E = 1.4426950408889634f;  // g arrives multiplied by log2(e): the factors are plain exp2
  const float m0 = LOG2E * G[H * ldf + c], m1 = H == 32 ? m0 : LOG2E * G[48 * ldf + c];
  float F[16];
  bf16x4 B[4];  // block t as B operand: F b of a column block (row sums), F a of a row block (column sums)
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const bool up = ((16 * t) & H) != 0;
    const float ref = (H == 32 || t < 2) ? m0 : m1;
    // one exponential per four tokens, the others by the single-step decays: away from the reference the factors shrink
    if (up) {
      F[4 * t] = __builtin_amdgcn_exp2f(fminf(g[4 * t] - ref, 0.f));
#pragma unroll
      for (int e = 1; e < 4; ++e) F[4 * t + e] = F[4 * t + e - 1] * dec[4 * t + e];
    } else {
      F[4 * t + 3] = __builtin_amdgcn_exp2f(fminf(ref - g[4 * t + 3], 0.f));
#pragma unroll
      for (int e = 2; e >= 0; --e) F[4 * t + e] = F[4 * t + e + 1] * dec[4 * t + e + 1];
    }
    floatx4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = F[4 * t + e] * (up ? av[4 * t + e] : bv[4 * t + e]);
    B[t] = pack_bf16x4(v);
  }
  const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ti = 1; ti < 4; ++ti) {
    if (H == 32 ? ti < 2 : !(ti & 1)) continue;
    floatx4 acc = zero;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      if (H == 32 ? t < 2 : t == ti - 1) acc = mfma16_bf16(pair_x_rows(X, ti, t, l16, kq), B[t], acc);
#pragma unroll
    for (int e = 0; e < 4; ++e) ro[4 * ti + e] += F[4 * ti + e] * acc[e];
  }
#pragma unroll
  for (int tj = 0; tj < 3; ++tj) {
    if (H == 32 ? tj >= 2 : (tj & 1)) continue;
    floatx4 acc = zero;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      if (H == 32 ? t >= 2 : t == tj + 1) acc = mfma16_bf16(pair_x_cols(X, t, tj, l16, kq), B[t], acc);
#pragma unroll
    for (int e = 0; e < 4; ++e) co[4 * tj + e] += F[4 * tj + e] * acc[e];
  }
}

// Levels 8, 4, 2, 1 of one diagonal 16x16 block: lane = (row l16 of the block, k-slots 4 kq + e), and a row and a
// k-slot only meet inside the same 2H-token segment.  g, b, a, ro, co: the lane's four tokens of this block.
__device__ __forceinline__ void pair_diag(floatx4& ro, floatx4& co, const floatx4 g, const floatx4 dec, const floatx4 bv, const floatx4 av,
                                          const float* __restrict__ X, const float* __restrict__ G, int ldf, int c, int t,
                                          int l16, int kq) {
  typedef unsigned uint2_ __attribute__((ext_vector_type(2)));
  constexpr float LOG2E = 1.4426950408889634f;
  const uint2_ xr = __builtin_bit_cast(uint2_, pair_x_rows(X, t, t, l16, kq)), xc = __builtin_bit_cast(uint2_, pair_x_cols(X, t, t, l16, kq));
  const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int H = 8; H >= 1; H >>= 1) {
    floatx4 fu, fl;  // the factor of each token in its role at this level (row token: fu, column token: fl), 0 in the other
    if (H >= 4) {  // all four tokens share the role and the reference: one exponential, the rest by the single-step decays
      const bool up = H == 8 ? (kq & 2) != 0 : (kq & 1) != 0;
      const float ref = LOG2E * G[(16 * t + (H == 8 ? 8 : 8 * (kq >> 1) + 4)) * ldf + c];
      const float f = __builtin_amdgcn_exp2f(fminf(up ? g[0] - ref : ref - g[3], 0.f));
      floatx4 F;
      F[0] = up ? f : f * dec[3] * dec[2] * dec[1];
      F[1] = up ? f * dec[1] : f * dec[3] * dec[2];
      F[2] = up ? F[1] * dec[2] : f * dec[3];
      F[3] = up ? F[2] * dec[3] : f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        fu[e] = up ? F[e] : 0.f;
        fl[e] = up ? 0.f : F[e];
      }
    } else if (H == 2) {  // reference: token 2 of the four
      fl = floatx4{dec[1] * dec[2], dec[2], 0.f, 0.f};
      fu = floatx4{0.f, 0.f, 1.f, dec[3]};
    } else {  // references: tokens 1 and 3
      fl = floatx4{dec[1], 0.f, dec[3], 0.f};
      fu = floatx4{0.f, 1.f, 0.f, 1.f};
    }
    // k-slots (0, 1) and (2, 3) each share a 2-token segment, so the masks act on whole dwords of the packed operand
    uint2_ mk;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const bool on = H == 8 ? true : H == 4 ? (l16 >> 3) == (kq >> 1) : H == 2 ? (l16 >> 2) == kq : (l16 >> 1) == 2 * kq + w;
      mk[w] = on ? 0xffffffffu : 0u;
    }
    const floatx4 r = mfma16_bf16(__builtin_bit_cast(bf16x4, xr & mk), pack_bf16x4(fl * bv), zero);
    const floatx4 q = mfma16_bf16(__builtin_bit_cast(bf16x4, xc & mk), pack_bf16x4(fu * av), zero);
    ro += fu * r;
    co += fl * q;
  }
}

template <bool STRICT>
__device__ __forceinline__ void pair_levels(float (&ro)[16], float (&co)[16], const float* __restrict__ X,
                                            const float* __restrict__ G, int ldf, const bf16_t* __restrict__ b, int ldb,
                                            const bf16_t* __restrict__ a, int lda, int tid) {
  const int wave = tid >> 6, lane = tid & 63, l16 = lane & 15, kq = lane >> 4;
  const int c = 16 * wave + l16;
  float g[16], bv[16], av[16];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int tok = 16 * t + 4 * kq + e, x = 4 * t + e;
      g[x] = 1.4426950408889634f * G[tok * ldf + c];
      bv[x] = (float)b[tok * ldb + c];
      av[x] = (float)a[tok * lda + c];
      const float d = STRICT ? 0.f : X[tok * LNX_LDA + tok];
      ro[x] = d * bv[x];
      co[x] = d * av[x];
    }
  float dec[16];  // single-step decays exp(G_tok - G_{tok-1}) inside each group of four (the first entry of a group is unused)
#pragma unroll
  for (int x = 0; x < 16; ++x) dec[x] = (x & 3) ? __builtin_amdgcn_exp2f(fminf(g[x] - g[x - 1], 0.f)) : 1.f;
  pair_cross<32>(ro, co, g, dec, bv, av, X, G, ldf, c, l16, kq);
  __builtin_amdgcn_sched_barrier(0);  // one part at a time: interleaving them multiplies the live factors
  pair_cross<16>(ro, co, g, dec, bv, av, X, G, ldf, c, l16, kq);
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    __builtin_amdgcn_sched_barrier(0);
    floatx4 r4 = {ro[4 * t], ro[4 * t + 1], ro[4 * t + 2], ro[4 * t + 3]}, c4 = {co[4 * t], co[4 * t + 1], co[4 * t + 2], co[4 * t + 3]};
    pair_diag(r4, c4, floatx4{g[4 * t], g[4 * t + 1], g[4 * t + 2], g[4 * t + 3]},
              floatx4{1.f, dec[4 * t + 1], dec[4 * t + 2], dec[4 * t + 3]}, floatx4{bv[4 * t], bv[4 * t + 1], bv[4 * t + 2], bv[4 * t + 3]},
              floatx4{av[4 * t], av[4 * t + 1], av[4 * t + 2], av[4 * t + 3]}, X, G, ldf, c, t, l16, kq);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ro[4 * t + e] = r4[e];
      co[4 * t + e] = c4[e];
    }
  }
}
