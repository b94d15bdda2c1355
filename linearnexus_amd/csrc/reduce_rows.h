// Column sums of a [n x d] fp32 matrix of partial results in a caller-owned workspace: how the streaming backward
// kernels finish their per-channel parameter gradients without atomics (deterministic results).
#pragma once

#include "lnx_common.h"

#define LNX_SUM_SLICES 64  // first-level slices of the partial rows

// out[y][c] = sum of part[r][c] over the rows r of slice y = blockIdx.y (`per` rows each, `n` rows in all; d a
// multiple of 4); 256 threads = 16 groups of four columns x 16 interleaved row sets, eight independent loads in
// flight per thread.  Run twice -- many slices, then one -- so that no single CU has to read all partial rows.
static __global__ __launch_bounds__(256) void lnx_sum_rows_kernel(const float* part, int64_t n, int64_t per, int d, float* out) {
  part += (int64_t)blockIdx.y * per * d;
  out += (int64_t)blockIdx.y * d;
  n = min(per, n - (int64_t)blockIdx.y * per);
  __shared__ floatx4 red[16][16];
  const int cg = threadIdx.x & 15, rs = threadIdx.x >> 4;
  const int c = (blockIdx.x * 16 + cg) * 4;
  floatx4 acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
  if (c < d) {
    for (int64_t r = rs; r < n; r += 16 * 8) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (r + 16 * u < n) acc[u] += load4(part + (r + 16 * u) * d + c);
    }
  }
  red[rs][cg] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
  __syncthreads();
  if (rs == 0 && c < d) {
    floatx4 t = red[0][cg];
#pragma unroll
    for (int q = 1; q < 16; ++q) t += red[q][cg];
    store4(out + c, t);
  }
}


// Bytes of workspace for `n` partial rows of `d` floats plus the first-level sums behind them.
static inline uint64_t lnx_sum_rows_bytes(int64_t n, int d) { return (uint64_t)(n + LNX_SUM_SLICES) * d * sizeof(float); }

// out[c] = sum_r part[r][c]; `part` must have room for lnx_sum_rows_bytes(n, d).  Two levels (many slices, then
// one) so that no single CU has to read all partial rows.
static inline void lnx_sum_rows(float* part, int64_t n, int d, float* out, hipStream_t st) {
  const int64_t per = (n + LNX_SUM_SLICES - 1) / LNX_SUM_SLICES;
  if (per > 1) {
    float* part2 = part + n * d;
    const int slices = (int)((n + per - 1) / per);
    lnx_sum_rows_kernel<<<dim3((d + 63) / 64, slices), 256, 0, st>>>(part, n, per, d, part2);
    lnx_sum_rows_kernel<<<dim3((d + 63) / 64, 1), 256, 0, st>>>(part2, slices, slices, d, out);
  } else {
    lnx_sum_rows_kernel<<<dim3((d + 63) / 64, 1), 256, 0, st>>>(part, n, n > 0 ? n : 1, d, out);
  }
}
