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
  const int32_t* cu;             // device cu_seqlens or nullptr
  const int32_t* tab;            // packed only: [N][2] (token0, len) then seq_chunk0[nseq + 1]
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
  uint64_t tab, G, P, X, W, U, Kr, Qg, TmT, D, SnT, dD, dSn, dW, dG, total;
};

inline uint64_t lnx_align256(uint64_t x) { return (x + 255) & ~uint64_t(255); }

inline int lnx_chunk_slots(const lnx_scan_args* a) {
  return a->cu_seqlens ? a->T / LNX_C + a->nseq : (a->T + LNX_C - 1) / LNX_C;
}

inline ChunkWs lnx_chunk_ws_layout(const lnx_scan_args* a) {
  ChunkWs w;
  const uint64_t es = (a->dtype == LNX_BF16) ? 2 : 4;
  const uint64_t rows = a->cu_seqlens ? (uint64_t)a->H : (uint64_t)a->B * a->H;
  const uint64_t N = (uint64_t)lnx_chunk_slots(a);
  const uint64_t slots = rows * N, dk = a->dk, dv = a->dv, C = LNX_C;
  uint64_t off = 0;
  auto take = [&](uint64_t bytes) { uint64_t o = off; off = lnx_align256(off + bytes); return o; };
  w.tab = take(a->cu_seqlens ? (2 * N + a->nseq + 1) * 4 : 0);
  w.G = take(a->gate == LNX_GATE_VECTOR ? slots * C * dk * 4 : slots * C * 4);
  w.P = take(slots * C * C * es);
  w.X = take(a->gate == LNX_GATE_VECTOR ? slots * C * C * es : 0);
  w.W = take(slots * C * dk * es);
  w.U = take(slots * C * dv * es);
  w.Kr = take(a->gate == LNX_GATE_VECTOR ? slots * C * dk * es : 0);
  w.Qg = take(a->gate == LNX_GATE_VECTOR ? slots * C * dk * es : 0);
  w.TmT = take(slots * C * C * es);
  w.D = take(slots * C * dv * es);
  w.SnT = take(slots * dv * dk * es);
  w.dD = take(slots * C * dv * es);
  w.dSn = take(slots * dk * dv * es);
  w.dW = take(slots * C * dk * es);
  w.dG = take(a->gate == LNX_GATE_VECTOR ? slots * C * dk * 4 : slots * C * 4);
  w.total = off;
  return w;
}

// Shared argument validation of the chunk entry points; returns LNX_OK or an error status.
int lnx_chunk_check(const lnx_scan_args* a, bool backward);

// Builds the packed-batch chunk table (no-op for dense batches).
void lnx_chunk_build_table(const lnx_scan_args* a, const ChunkWs& w, hipStream_t st);

// ---------------------------------------------------------------------------------------
// Vector-gate (KDA) helpers: per-channel decays E_ij[c] = prod_{m=j+1..i} alpha_m[c] are applied
// with a multiplicative recurrence along the token index, so no exponent of a positive number
// is ever taken (the property kda.py:426-434 protects with its blocked factorisation).
// Tiles live in LDS: M [64][LNX_LDA] fp32, al (alpha) and out [64][ldf] fp32, operands [64][ldb].
// A wavefront owns a token row (or column), its lanes the channels.
// ---------------------------------------------------------------------------------------

// out[i][c] += mul * sum_{j <= i (j < i if STRICT)} M[i][j] * E_ij[c] * b[j][c]
// The token loop runs in blocks of 8 whose LDS reads are issued together (the loop is latency
// bound otherwise); blocks are aligned so that masked tokens multiply by M = 0 / alpha = 1.
template <typename T, int DK, bool STRICT>
__device__ __forceinline__ void pair_row(float* out, const float* M, const float* al, int ldf, const T* b, int ldb,
                                         float mul, int tid) {
  const int wave = tid >> 6, lane = tid & 63;
  for (int i = wave; i < 64; i += 4)
    for (int c = lane; c < DK; c += 64) {
      float e = 1.f, acc = 0.f;
      for (int j0 = i | 7; j0 >= 7; j0 -= 8) {  // tokens j0, j0-1, ..., j0-7
        float m[8], bv[8], av[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int j = j0 - u;  // always a valid row: loads are unconditional, masks applied after
          m[u] = M[i * LNX_LDA + j];
          bv[u] = to_f32(b[j * ldb + c]);
          av[u] = al[j * ldf + c];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int j = j0 - u;
          const bool on = j <= i;
          m[u] = (on && !(STRICT && j == i)) ? m[u] : 0.f;
          av[u] = on ? av[u] : 1.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          acc += m[u] * e * bv[u];
          e *= av[u];
        }
      }
      out[i * ldf + c] += mul * acc;
    }
}

// out[j][c] += mul * sum_{i >= j (i > j if STRICT)} M[i][j] * E_ij[c] * a[i][c]
template <typename T, int DK, bool STRICT>
__device__ __forceinline__ void pair_col(float* out, const float* M, const float* al, int ldf, const T* a, int lda,
                                         float mul, int tid) {
  const int wave = tid >> 6, lane = tid & 63;
  for (int j = wave; j < 64; j += 4)
    for (int c = lane; c < DK; c += 64) {
      float e = 1.f, acc = 0.f;
      for (int i0 = j & ~7; i0 < 64; i0 += 8) {  // tokens i0 .. i0+7
        float m[8], xv[8], av[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = i0 + u;
          m[u] = M[i * LNX_LDA + j];
          xv[u] = to_f32(a[i * lda + c]);
          av[u] = al[i * ldf + c];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int i = i0 + u;
          m[u] = (i > j || (!STRICT && i == j)) ? m[u] : 0.f;
          av[u] = (i > j) ? av[u] : 1.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          e *= av[u];
          acc += m[u] * e * xv[u];
        }
      }
      out[j * ldf + c] += mul * acc;
    }
}
