/*
 * Plain-C caller of liblinearnexus_hip.so: no Python, no torch -- device memory from hipMalloc,
 * the argument block filled by hand, results checked against closed forms of the delta rule
 * (beta = 0 and no gate: S_T = S0 and o_t = scale * S0^T q_t; test_deltanet.py:281-297 uses the
 * same special case -- it exercises the boundary, not the arithmetic: the WY inverse and W, U, D are trivial there;
 * then one key direction e repeated for every token with random beta in (0.1, 1): the state stays e u_t^T with
 * u_t = (1 - beta_t) u_{t-1} + beta_t v_t, o_t = scale <q_t, e> u_t, and the chunk's triangular system is the dense
 * all-ones lower triangle scaled by beta, so its inverse and every product of the chunk path carry weight).
 * Built by linearnexus_amd/build.py (gcc) next to this file; tests/test_c_abi_gpu.py runs it.  Exit status 0 = every
 * check passed.
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/linearnexus_hip.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)
#define CHECK_LNX(x) do { int s_ = (x); if (s_ != LNX_OK) { fprintf(stderr, "%s -> %d: %s\n", #x, s_, lnx_last_error()); return 3; } } while (0)

static float frand(unsigned* s) {  /* uniform in [-1, 1) */
  *s = *s * 1664525u + 1013904223u;
  return (float)((*s >> 8) & 0xFFFFFF) / 8388608.0f - 1.0f;
}

static float* to_device(const float* h, size_t n) {
  float* d = NULL;
  if (hipMalloc((void**)&d, n * sizeof(float)) != hipSuccess) return NULL;
  if (hipMemcpy(d, h, n * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) return NULL;
  return d;
}

int main(void) {
  enum { B = 2, H = 2, T = 96, D = 64 };
  const size_t nq = (size_t)B * H * T * D, ns = (size_t)B * H * D * D, nb = (size_t)B * H * T;
  const float scale = 1.0f / sqrtf((float)D);
  unsigned seed = 12345u;
  float *q = malloc(nq * 4), *k = malloc(nq * 4), *v = malloc(nq * 4), *beta = calloc(nb, 4), *s0 = malloc(ns * 4);
  float *o = malloc(nq * 4), *sT = malloc(ns * 4), *oref = malloc(nq * 4);
  for (size_t i = 0; i < nq; ++i) { q[i] = frand(&seed); k[i] = frand(&seed); v[i] = frand(&seed); }
  for (size_t i = 0; i < ns; ++i) s0[i] = 0.1f * frand(&seed);
  for (int bh = 0; bh < B * H; ++bh)
    for (int t = 0; t < T; ++t)
      for (int c = 0; c < D; ++c) {
        double acc = 0;
        for (int r = 0; r < D; ++r) acc += (double)s0[((size_t)bh * D + r) * D + c] * q[((size_t)bh * T + t) * D + r];
        oref[((size_t)bh * T + t) * D + c] = (float)(scale * acc);
      }

  printf("abi version %d\n", lnx_abi_version());
  float *dq = to_device(q, nq), *dk = to_device(k, nq), *dv = to_device(v, nq), *dbeta = to_device(beta, nb);
  float *ds0 = to_device(s0, ns), *dO = NULL, *dsT = NULL;
  if (!dq || !dk || !dv || !dbeta || !ds0) { fprintf(stderr, "device allocation failed\n"); return 2; }
  CHECK_HIP(hipMalloc((void**)&dO, nq * 4));
  CHECK_HIP(hipMalloc((void**)&dsT, ns * 4));
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));

  lnx_scan_args a;
  memset(&a, 0, sizeof a);
  a.B = B; a.H = H; a.T = T; a.dk = D; a.dv = D; a.chunk = 64;
  a.dtype = LNX_F32; a.o_dtype = LNX_F32; a.gate = LNX_GATE_NONE; a.scale = scale;
  a.q = dq; a.k = dk; a.v = dv; a.beta = dbeta; a.initial_state = ds0; a.o = dO; a.final_state = dsT;

  double worst = 0;
  for (int pass = 0; pass < 2; ++pass) {  /* 0: chunked (MFMA) path, 1: token-by-token path */
    CHECK_HIP(hipMemsetAsync(dO, 0xFF, nq * 4, st));
    CHECK_HIP(hipMemsetAsync(dsT, 0xFF, ns * 4, st));
    if (pass == 0) {
      a.workspace_bytes = lnx_chunk_workspace_bytes(&a);
      if (a.workspace_bytes == 0) { fprintf(stderr, "workspace query failed: %s\n", lnx_last_error()); return 3; }
      CHECK_HIP(hipMalloc(&a.workspace, a.workspace_bytes));
      CHECK_LNX(lnx_chunk_fwd(&a, st));
    } else {
      CHECK_LNX(lnx_recurrent_fwd(&a, st));
    }
    CHECK_HIP(hipStreamSynchronize(st));
    CHECK_HIP(hipMemcpy(o, dO, nq * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(sT, dsT, ns * 4, hipMemcpyDeviceToHost));
    double eo = 0, es = 0, mo = 0, ms = 0;
    for (size_t i = 0; i < nq; ++i) { eo = fmax(eo, fabs((double)o[i] - oref[i])); mo = fmax(mo, fabs((double)oref[i])); }
    for (size_t i = 0; i < ns; ++i) { es = fmax(es, fabs((double)sT[i] - s0[i])); ms = fmax(ms, fabs((double)s0[i])); }
    printf("%s: o err %.3g, state err %.3g (relative to the maximum)\n", pass ? "lnx_recurrent_fwd" : "lnx_chunk_fwd", eo / mo, es / ms);
    worst = fmax(worst, fmax(eo / mo, es / ms));
  }

  /* one repeated key direction, beta in (0.1, 1), zero initial state */
  {
    float* e = malloc((size_t)B * H * D * 4);
    for (int bh = 0; bh < B * H; ++bh) {
      double n2 = 0;
      for (int c = 0; c < D; ++c) { e[bh * D + c] = frand(&seed); n2 += (double)e[bh * D + c] * e[bh * D + c]; }
      for (int c = 0; c < D; ++c) e[bh * D + c] = (float)(e[bh * D + c] / sqrt(n2));
    }
    float* sref = malloc(ns * 4);
    for (int bh = 0; bh < B * H; ++bh) {
      double u[D];
      for (int c = 0; c < D; ++c) u[c] = 0;
      double ee = 0;  /* <e, e> as the kernels see it (fp32 entries) */
      for (int c = 0; c < D; ++c) ee += (double)e[bh * D + c] * e[bh * D + c];
      for (int t = 0; t < T; ++t) {
        const size_t row = ((size_t)bh * T + t) * D;
        beta[(size_t)bh * T + t] = 0.55f + 0.45f * frand(&seed);
        const double b = beta[(size_t)bh * T + t];
        double qe = 0;
        for (int c = 0; c < D; ++c) { k[row + c] = e[bh * D + c]; qe += (double)q[row + c] * e[bh * D + c]; }
        for (int c = 0; c < D; ++c) u[c] = u[c] + b * (v[row + c] - ee * u[c]);
        for (int c = 0; c < D; ++c) oref[row + c] = (float)(scale * qe * u[c]);
      }
      for (int r = 0; r < D; ++r)
        for (int c = 0; c < D; ++c) sref[((size_t)bh * D + r) * D + c] = (float)(e[bh * D + r] * u[c]);
    }
    CHECK_HIP(hipMemcpy(dk, k, nq * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dbeta, beta, nb * 4, hipMemcpyHostToDevice));
    a.initial_state = NULL;
    for (int pass = 0; pass < 2; ++pass) {
      CHECK_HIP(hipMemsetAsync(dO, 0xFF, nq * 4, st));
      CHECK_HIP(hipMemsetAsync(dsT, 0xFF, ns * 4, st));
      if (pass == 0) CHECK_LNX(lnx_chunk_fwd(&a, st));
      else CHECK_LNX(lnx_recurrent_fwd(&a, st));
      CHECK_HIP(hipStreamSynchronize(st));
      CHECK_HIP(hipMemcpy(o, dO, nq * 4, hipMemcpyDeviceToHost));
      CHECK_HIP(hipMemcpy(sT, dsT, ns * 4, hipMemcpyDeviceToHost));
      double eo = 0, es = 0, mo = 0, ms = 0;
      for (size_t i = 0; i < nq; ++i) { eo = fmax(eo, fabs((double)o[i] - oref[i])); mo = fmax(mo, fabs((double)oref[i])); }
      for (size_t i = 0; i < ns; ++i) { es = fmax(es, fabs((double)sT[i] - sref[i])); ms = fmax(ms, fabs((double)sref[i])); }
      printf("repeated key, %s: o err %.3g, state err %.3g (relative to the maximum)\n", pass ? "lnx_recurrent_fwd" : "lnx_chunk_fwd", eo / mo, es / ms);
      worst = fmax(worst, fmax(eo / mo, es / ms));
    }
    a.initial_state = ds0;
    /* the checks below are the beta = 0 case again */
    memset(beta, 0, nb * 4);
    CHECK_HIP(hipMemcpy(dbeta, beta, nb * 4, hipMemcpyHostToDevice));
    for (int c = 0; c < D; ++c) {
      double acc = 0;
      for (int r = 0; r < D; ++r) acc += (double)s0[(size_t)r * D + c] * q[r];
      oref[c] = (float)(scale * acc);
    }
    free(e);
    free(sref);
  }

  /* decode step on the last token, state in place */
  a.T = 1; a.final_state = ds0;
  a.q = dq; a.k = dk; a.v = dv; a.o = dO;  /* token 0 of row 0 only when B = H = 1; use a one-row view */
  a.B = 1; a.H = 1;
  CHECK_LNX(lnx_decode_step(&a, st));
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipMemcpy(o, dO, D * 4, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(sT, ds0, (size_t)D * D * 4, hipMemcpyDeviceToHost));
  double eo = 0, es = 0;
  for (int c = 0; c < D; ++c) eo = fmax(eo, fabs((double)o[c] - oref[c]));
  for (int i = 0; i < D * D; ++i) es = fmax(es, fabs((double)sT[i] - s0[i]));
  printf("lnx_decode_step: o err %.3g, state err %.3g (absolute)\n", eo, es);
  worst = fmax(worst, fmax(eo, es));

  /* error path: a required pointer is missing */
  a.q = NULL;
  if (lnx_decode_step(&a, st) != LNX_ERR_NULL || !strstr(lnx_last_error(), "required")) { fprintf(stderr, "error path\n"); return 4; }

  printf("worst %.3g\n", worst);
  return worst < 1e-4 ? 0 : 1;
}
