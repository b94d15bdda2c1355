/*
 * C-ABI of the MI355X (gfx950) delta-rule scan library, liblinearnexus_hip.so.
 *
 * The reference (saran-gangster/linearnexus) is pure Python/JAX and has no native
 * interface of its own; these entry points are what an XLA-FFI / ctypes binding for
 * its layer ops would bind.  Every function returns 0 on success and a negative
 * lnx_status otherwise; lnx_last_error() gives the thread-local message.  Nothing
 * here allocates or frees device memory or synchronises the device, and the compute
 * entry points keep no state between calls: the caller owns all buffers (workspace
 * included) and the stream.  The two exceptions are documented where they are declared:
 * lnx_chunk_fwd_static works on a scratch array the library holds per GPU, and the
 * optional timing of lnx_profile_enable keeps a process-wide list of HIP events.
 *
 * Tensor conventions (the reference's, linearnexus/modules/linear_attn/delta_net.py:126-134):
 *   q, k  [B, H, T, dk]   v, o  [B, H, T, dv]   beta [B, H, T]   state [B, H, dk, dv] fp32
 *   gate  g: none | [B, H, T] (Gated DeltaNet) | [B, H, T, dk] (KDA), fp32 log-decay <= 0
 * All tensors are dense, last dimension contiguous.  q/k/v (and dO, dq, dk, dv) share
 * one element type `dtype` (fp32 or bf16); beta, g, states and their gradients are fp32.
 * With cu_seqlens != NULL the batch is packed: B must be 1, sequences are
 * [cu[s], cu[s+1]) along T, states are [nseq, H, dk, dv] and reset at every boundary.
 * Contract: cu[0] = 0, cu non-decreasing, cu[nseq] = T.  The table is device memory the host
 * side cannot inspect, so the kernels clamp its entries to [0, T] and read a decreasing pair as
 * an empty sequence -- a malformed table never causes an access outside the tensors -- but
 * tokens outside every sequence then keep unspecified outputs and gradients.
 */
#ifndef LINEARNEXUS_HIP_H
#define LINEARNEXUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { LNX_F32 = 0, LNX_BF16 = 1 } lnx_dtype;
typedef enum { LNX_GATE_NONE = 0, LNX_GATE_SCALAR = 1, LNX_GATE_VECTOR = 2 } lnx_gate;

typedef enum {
  LNX_OK = 0,
  LNX_ERR_NULL = -1,        /* a required pointer is NULL */
  LNX_ERR_SHAPE = -2,       /* unsupported or inconsistent dimensions */
  LNX_ERR_DTYPE = -3,       /* unsupported element type */
  LNX_ERR_WORKSPACE = -4,   /* workspace missing or too small */
  LNX_ERR_LAUNCH = -5,      /* HIP reported a launch error */
  LNX_ERR_DEVICE = -6       /* not a gfx950 device / no device */
} lnx_status;

/* One argument block for every entry point; fields an entry point does not use are ignored. */
typedef struct lnx_scan_args {
  int32_t B, H, T, dk, dv;
  int32_t chunk;            /* chunk length; 64 is the only supported value (must be % 16 == 0) */
  int32_t dtype;            /* lnx_dtype of q, k, v, dO, dq, dk, dv */
  int32_t o_dtype;          /* lnx_dtype of o */
  int32_t gate;             /* lnx_gate */
  int32_t use_qk_l2norm;    /* normalise q, k rows as x / (|x|_2 + 1e-6) inside the op: always honoured by the decode step
                               and the token-by-token scan; by the chunk entry points where lnx_chunk_fuses_l2norm
                               says so (ABI version 6), d_q and d_k are then the gradients of the raw q and k */
  int32_t nseq;             /* number of packed sequences; 0 for a dense batch */
  float scale;              /* multiplies q (after normalisation) */
  int32_t forward_only;     /* lnx_chunk_fwd: no backward pass will follow, do not write the per-chunk tensors
                               only lnx_chunk_bwd reads (inference / prefill); the workspace is still needed */
  int32_t token_first;      /* 0: q, k, v, o, beta, g and their gradients are [B,H,T,.] (the reference's layout);
                               1: they are [B,T,H,.] (what the reference's blocks hold before they transpose,
                               delta_net.py:645-647) -- packed batches [1,T,H,.]; states are [B,H,dk,dv] either way */

  const void* q;
  const void* k;
  const void* v;
  const float* beta;
  const float* g;               /* NULL when gate == LNX_GATE_NONE */
  const float* initial_state;   /* NULL = zeros */
  const int32_t* cu_seqlens;    /* NULL for a dense batch; device pointer, nseq + 1 entries */
  void* o;
  float* final_state;           /* may alias initial_state for the decode step (in place) */

  /* backward only */
  const void* d_o;              /* [B,H,T,dv] in dtype */
  const float* d_final_state;   /* NULL = zeros */
  void* d_q;                    /* gradient outputs, same shapes/dtypes as q, k, v */
  void* d_k;
  void* d_v;
  float* d_beta;
  float* d_g;                   /* NULL when gate == LNX_GATE_NONE */
  float* d_initial_state;       /* NULL = not wanted */

  void* workspace;
  uint64_t workspace_bytes;

  int32_t value_cols;           /* lnx_chunk_fwd with forward_only (ABI version 4): v holds only the first value_cols
                                   of the dv value columns (its rows are value_cols long); the others are zero and
                                   are not read.  0 = all dv.  With forward_only, o may also be NULL: only the final
                                   states are wanted.  (Transition matrices of sequence segments: value columns
                                   [v | 0], initial states [0 | I].) */

  /* The per-channel gate's activation inside the chunk op (ABI version 8; gate == LNX_GATE_VECTOR only).  With
     gate_raw != NULL, g is ignored and lnx_chunk_fwd forms the log-decay itself from the block's raw gate projection,
       g[b, h, t, c] = -exp(gate_A_log[h]) * softplus(gate_raw[b, h, t, c] + gate_bias[h * dk + c])
     (kda_gate, kda.py:153-165; softplus(x) = x above gate_threshold), in the prepare kernel's gate load: the fp32
     log-decay tensor never exists in memory.  gate_raw has the layout and element type of q ([B,H,T,dk] or, with
     token_first, [B,T,H,dk] = the projection's [B,T,H*dk]).  lnx_chunk_bwd then needs the same fields again, writes
     d_gate_raw (element type of q) in place of d_g and returns the parameter gradients d_gate_A_log [H] and
     d_gate_bias [H*dk] (either may be NULL), summed without atomics through partial rows in the workspace. */
  const void* gate_raw;
  const float* gate_A_log;
  const float* gate_bias;       /* NULL = no bias */
  float gate_threshold;
  void* d_gate_raw;
  float* d_gate_A_log;
  float* d_gate_bias;

  /* Test hooks (ABI version 8); a binding leaves both 0 = the library's choice.  Neither changes results or the
     workspace layout, only which of two tilings of the same kernel runs, so that tests reach both at small shapes. */
  int32_t test_scan_slab;       /* 32 or 64: value columns per workgroup of the sequential kernels */
  int32_t test_out_slabs;       /* > 0: value slabs per workgroup of the fp32 output kernel */
} lnx_scan_args;

/* Library identification; also the symbol a loader probes first. */
int lnx_abi_version(void);
const char* lnx_last_error(void);

/*
 * Single-token decode step, state updated in place when final_state == initial_state.
 * q,k [B,H,dk], v,o [B,H,dv], beta [B,H], g [B,H] or [B,H,dk]; T is ignored.
 * Replaces delta_rule_step (delta_net.py:357-397), gated_delta_rule_step
 * (gated_deltanet.py:539-597) and kda_step (kda.py:286-347).
 */
int lnx_decode_step(const lnx_scan_args* a, void* hip_stream);

/*
 * Token-by-token scan in fp32 with the state held in registers.
 * Replaces delta_rule_recurrent (delta_net.py:126-213; also the Pallas kernel
 * kernels/pallas/delta_rule.py:47-281), gated_delta_rule_recurrent
 * (gated_deltanet.py:136-229) and kda_recurrent (kda.py:179-283).
 */
int lnx_recurrent_fwd(const lnx_scan_args* a, void* hip_stream);

/*
 * Chunked (WY) forward on MFMA.  Replaces delta_rule_chunkwise (delta_net.py:216-354),
 * gated_delta_rule_chunkwise (gated_deltanet.py:232-534), kda_chunkwise (kda.py:350-655).
 * The workspace keeps the per-chunk tensors the backward pass re-uses; pass the same
 * workspace, unchanged, to lnx_chunk_bwd (unless forward_only was set), with the same shape, dtype, gate, nseq,
 * token_first, scale and use_qk_l2norm fields: the layout of the workspace follows from B, H, T, dk, dv, dtype, gate
 * and nseq alone (o_dtype does not enter it), and there is exactly one set of kernels per such shape.
 * Shapes: dk in {64, 128, 256} (256 is the head_dim of the reference's Gated DeltaNet presets,
 * models.py:142-143), dv a multiple of 64.  q, k, v, o, a per-channel gate (g or gate_raw), the states, the workspace
 * and the gradients of all of these must be 16-byte aligned (the kernels move their rows as 16-byte vectors);
 * LNX_ERR_SHAPE otherwise (LNX_ERR_WORKSPACE for the workspace).  beta, a scalar gate and their gradients only need their element's alignment.
 */
uint64_t lnx_chunk_workspace_bytes(const lnx_scan_args* a);
int lnx_chunk_fwd(const lnx_scan_args* a, void* hip_stream);
/*
 * 1 when lnx_chunk_fwd / lnx_chunk_bwd apply the in-op normalisation of q and k themselves for these arguments
 * (use_qk_l2norm = 1: gated_deltanet.py:273-275, kda.py:379-381 normalise inside the op, and it is their default):
 * q, k, v in bf16, dk <= 128, no per-channel gate.  The rows are scaled where the kernels stage them and the
 * backward pass carries d_q, d_k through the normalisation, so no normalised copies of q and k exist.  0: the chunk
 * entry points refuse use_qk_l2norm for these arguments; normalise with lnx_l2norm_fwd first.
 */
int lnx_chunk_fuses_l2norm(const lnx_scan_args* a);

/*
 * lnx_chunk_fwd for callers that cannot allocate device memory or bring a workspace (code under HIP graph
 * capture, tight serving loops): same arguments and results as lnx_chunk_fwd with forward_only = 1 (required),
 * but a->workspace / a->workspace_bytes are ignored and the per-chunk tensors go to a scratch array of
 * LNX_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process ends.  Shapes whose
 * lnx_chunk_workspace_bytes exceeds that size are refused with LNX_ERR_WORKSPACE.  It calls no hipMalloc / hipFree
 * or other allocating routine.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (two streams, two threads) race and must be serialised by the caller.  No counterpart in the reference, whose
 * JAX ops leave allocation to XLA.
 * For bf16 inputs with dk <= 128 and no per-channel gate the scratch takes 17 KiB per 64-token chunk of every
 * (batch, head) row, so B * H * ceil(T / 64) <= 3855 chunks fit (8 heads of 30720 tokens; a packed batch counts
 * T / 64 + nseq chunks per head); the other shapes also keep W and U there, (dk + dv) * 128 bytes more per chunk (twice
 * that for fp32); lnx_chunk_workspace_bytes with forward_only = 1 gives the exact figure.  The address of the array on the current device is looked up on the first call on
 * that device; a caller that will make its first call while its stream is capturing calls lnx_chunk_fwd_static_init()
 * once per device beforehand, outside the capture (it launches nothing).
 */
#define LNX_STATIC_SCRATCH_BYTES (64u << 20)
int lnx_chunk_fwd_static_init(void);
int lnx_chunk_fwd_static(const lnx_scan_args* a, void* hip_stream);

/*
 * Chunked backward: gradients of <o, dO> + <final_state, d_final_state>.  The reference
 * has no backward code (gradients come from JAX autodiff through lax.scan,
 * linearnexus/train/sft.py:126-127); this entry point is what its jax.custom_vjp
 * rule would call.  Needs the workspace filled by lnx_chunk_fwd on the same inputs.
 */
int lnx_chunk_bwd(const lnx_scan_args* a, void* hip_stream);

/*
 * Row-wise x / (|x|_2 + 1e-6) over the last dimension and its vector-Jacobian product,
 * the normalisation the reference applies inside its ops when use_qk_l2norm is set
 * (gated_deltanet.py:193-195, :273-275).  x, y, dy, dx: [rows, d] in `dtype`.
 */
int lnx_l2norm_fwd(const void* x, void* y, int64_t rows, int32_t d, int32_t dtype, void* hip_stream);
int lnx_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t d, int32_t dtype,
                   void* hip_stream);

/*
 * Short causal depthwise convolution over [B, T, D] activations, kernel width K <= 4, with the SiLU the
 * reference's blocks apply right after it fused in (activation: 0 = none, 1 = SiLU).  Replaces
 * depthwise_conv1d_causal (linearnexus/core/conv.py:13-68) + jax.nn.silu (gated_deltanet.py:765-779):
 *   xin = concat(cache, x) along T;  y[t] = act(bias + sum_j weight[j] * xin[t + j]);  new_cache = last K-1 rows of xin.
 * x, y, dy, dx [B,T,D] and cache, new_cache [B,K-1,D] in `dtype` (D a multiple of 16 bytes of elements);
 * weight [K,D], bias [D] and their gradients fp32.  bias, cache, new_cache, d_weight, d_bias may be NULL
 * (cache NULL = zeros).  new_cache may alias cache for T <= 32 (decode).  lnx_conv1d_bwd overwrites d_weight / d_bias
 * (it clears them with a fill kernel, then accumulates atomically); lnx_conv1d_cache_bwd gives the gradient with respect
 * to the carry-in cache, d_cache [B,K-1,D] in `dtype` (JAX autodiff of conv.py:56-67 differentiates the concatenation).
 * A width-1 kernel is the identity plus bias and ignores its weight (conv.py:39-44; d_weight is then zero).
 * Packed batches (the layout the chunk ops take with cu_seqlens; the reference has no packed convolution, this is one
 * call of conv.py:13-68 per sequence with a zero cache): x, y, dy, dx [1,T,D], cu_seqlens [nseq+1] device int32 under
 * the contract stated at the top; the taps stop at the first token of each token's sequence, new_cache (may be NULL)
 * receives the last K-1 rows of the last sequence.
 */
int lnx_conv1d_fwd(const void* x, const float* weight, const float* bias, const void* cache, void* y, void* new_cache,
                   int32_t B, int32_t T, int32_t D, int32_t K, int32_t dtype, int32_t activation, void* hip_stream);
int lnx_conv1d_bwd(const void* x, const float* weight, const float* bias, const void* cache, const void* dy, void* dx,
                   float* d_weight, float* d_bias, int32_t B, int32_t T, int32_t D, int32_t K, int32_t dtype,
                   int32_t activation, void* hip_stream);
int lnx_conv1d_cache_bwd(const void* x, const float* weight, const float* bias, const void* cache, const void* dy,
                         void* d_cache, int32_t B, int32_t T, int32_t D, int32_t K, int32_t dtype, int32_t activation,
                         void* hip_stream);
int lnx_conv1d_packed_fwd(const void* x, const float* weight, const float* bias, const int32_t* cu_seqlens, int32_t nseq,
                          void* y, void* new_cache, int32_t T, int32_t D, int32_t K, int32_t dtype, int32_t activation,
                          void* hip_stream);
int lnx_conv1d_packed_bwd(const void* x, const float* weight, const float* bias, const int32_t* cu_seqlens, int32_t nseq,
                          const void* dy, void* dx, float* d_weight, float* d_bias, int32_t T, int32_t D, int32_t K,
                          int32_t dtype, int32_t activation, void* hip_stream);

/*
 * RWKV-7's diagonal-plus-low-rank delta rule (linearnexus/modules/linear_attn/rwkv7.py:114-265), the sibling
 * recurrence of the delta rule:  u = h^T a;  h <- exp(gk) (.) h + b u^T + k v^T;  o = h^T (scale * q).
 * q, k, a, b [B,H,T,dk] and v, o [B,H,T,dv] in `dtype` / `o_dtype`; gk [B,H,T,dk] and the states [B,H,dk,dv] fp32.
 * lnx_dplr_recurrent_fwd replaces dplr_delta_rule_recurrent (rwkv7.py:114-213; initial_state NULL = zeros),
 * lnx_dplr_step replaces dplr_delta_rule_step (rwkv7.py:216-265; token tensors [B,H,d], T ignored, the state is
 * updated in place when final_state == initial_state).  dk in {8,16,32,64,128}, dv a multiple of 4.
 */
typedef struct lnx_dplr_args {
  int32_t B, H, T, dk, dv;
  int32_t dtype;            /* lnx_dtype of q, k, v, a, b */
  int32_t o_dtype;          /* lnx_dtype of o */
  float scale;              /* multiplies q */
  const void* q;
  const void* k;
  const void* v;
  const void* a;
  const void* b;
  const float* gk;
  const float* initial_state;
  void* o;
  float* final_state;
} lnx_dplr_args;
int lnx_dplr_recurrent_fwd(const lnx_dplr_args* a, void* hip_stream);
int lnx_dplr_step(const lnx_dplr_args* a, void* hip_stream);

/*
 * Backward pass of lnx_dplr_recurrent_fwd: the gradients of <o, d_o> + <final state, d_final_state>, what jax.grad of
 * the reference's scan returns (the reference has no backward code of its own: its blocks train through autodiff of
 * dplr_delta_rule_recurrent, rwkv7.py:148-213).  `fwd` holds the forward call's inputs (its o and final_state are not
 * read); d_o [B,H,T,dv] in fwd.o_dtype; d_final_state [B,H,dk,dv] fp32 or NULL (zero).  Outputs, all fp32: dq, dk,
 * da, db, dgk [B,H,T,dk], dv [B,H,T,dv], d_initial_state [B,H,dk,dv] (may be NULL).  The states the tokens start from
 * are recomputed from checkpoints every 64 tokens kept in a caller-owned workspace of
 * lnx_dplr_recurrent_bwd_workspace_bytes bytes.  dk in {8,16,32,64,128}, dv a multiple of 4, at most 256.  No
 * atomics: the result is the same from run to run.
 */
typedef struct lnx_dplr_bwd_args {
  lnx_dplr_args fwd;
  const void* d_o;
  const float* d_final_state;
  float* dq;
  float* dk;
  float* dv;
  float* da;
  float* db;
  float* dgk;
  float* d_initial_state;
  void* workspace;
  uint64_t workspace_bytes;
} lnx_dplr_bwd_args;
uint64_t lnx_dplr_recurrent_bwd_workspace_bytes(int32_t B, int32_t H, int32_t T, int32_t dk, int32_t dv);
int lnx_dplr_recurrent_bwd(const lnx_dplr_bwd_args* a, void* hip_stream);

/*
 * RMSNorm with an optional sigmoid gate over the rows of [rows, d] matrices, the output epilogue of the reference's
 * blocks: y = x * rsqrt(mean(x^2) + eps) * weight * sigmoid(gate).  Replaces FusedRMSNormGated.__call__
 * (linearnexus/modules/linear_attn/kda.py:664-700) and o_norm(o) * sigmoid(g_out) (gated_deltanet.py:854-862).
 * x, gate, y, dy, dx, d_gate in `dtype`; weight, d_weight [d] fp32; gate NULL = no gate; d a whole number of
 * 16-byte vectors, at most 256 of them (rows of 4, 8, 16, 32 or 64 vectors take the faster kernels).  d_weight (may be NULL) is summed without atomics through partial rows
 * in a caller-owned workspace of lnx_rmsnorm_gated_bwd_workspace_bytes bytes.
 */
int lnx_rmsnorm_gated_fwd(const void* x, const void* gate, const float* weight, void* y, int64_t rows, int32_t d,
                          float eps, int32_t dtype, void* hip_stream);
uint64_t lnx_rmsnorm_gated_bwd_workspace_bytes(int64_t rows, int32_t d, int32_t dtype);
int lnx_rmsnorm_gated_bwd(const void* x, const void* gate, const float* weight, const void* dy, void* dx, void* d_gate,
                          float* d_weight, int64_t rows, int32_t d, float eps, int32_t dtype, void* workspace,
                          uint64_t workspace_bytes, void* hip_stream);

/*
 * Gated DeltaNet's gate and learning-rate activations (the block computes them between its projections and the scan,
 * gated_deltanet.py:804-815) and their gradient:
 *   g[r, h] = -exp(A_log[h]) * softplus(a[r, h] + dt_bias[h])        beta[r, h] = beta_scale * sigmoid(b[r, h])
 * a, b, d_a, d_b [rows, H] in `dtype` (b, beta, d_beta, d_b may be NULL together: gate only); g, beta and their
 * gradients d_g, d_beta fp32 -- what lnx_chunk_fwd and lnx_decode_step read; A_log, dt_bias [H] fp32 (dt_bias may be
 * NULL).  beta_scale = 2 for allow_neg_eigval (gated_deltanet.py:806-807), else 1.  d_A_log, d_dt_bias (may be NULL)
 * are summed over the rows without atomics through a caller-owned workspace.
 */
int lnx_gdn_gate_fwd(const void* a, const void* b, const float* A_log, const float* dt_bias, float* g, float* beta,
                     int64_t rows, int32_t H, float beta_scale, int32_t dtype, void* hip_stream);
uint64_t lnx_gdn_gate_bwd_workspace_bytes(int64_t rows, int32_t H);
int lnx_gdn_gate_bwd(const void* a, const void* b, const float* A_log, const float* dt_bias, const float* d_g,
                     const float* d_beta, void* d_a, void* d_b, float* d_A_log, float* d_dt_bias, int64_t rows, int32_t H,
                     float beta_scale, int32_t dtype, void* workspace, uint64_t workspace_bytes, void* hip_stream);

/*
 * KDA's gate activation (kda_gate, linearnexus/modules/linear_attn/kda.py:120-172) and its gradient:
 *   g_out[r, h, c] = -exp(A_log[h]) * softplus(g[r, h*dk + c] + g_bias[h*dk + c]),  softplus(x) = x for x > threshold
 * g, d_g [rows, H*dk] in `dtype`; g_out, d_out [rows, H, dk] in `out_dtype` (fp32 feeds lnx_chunk_fwd's vector gate
 * without a cast; the reference returns the input dtype, kda.py:172); A_log [H], g_bias [H*dk] (may be NULL) and their
 * gradients fp32 (may be NULL; they are summed without atomics through a caller-owned workspace).  dk % 4 == 0.
 * lnx_sigmoid_fwd / lnx_sigmoid_bwd are the beta = sigmoid(.) of the same function (kda.py:168-170) on fp32 vectors.
 */
int lnx_kda_gate_fwd(const void* g, const float* A_log, const float* g_bias, void* g_out, int64_t rows, int32_t H,
                     int32_t dk, float threshold, int32_t dtype, int32_t out_dtype, void* hip_stream);
uint64_t lnx_kda_gate_bwd_workspace_bytes(int64_t rows, int32_t H, int32_t dk);
int lnx_kda_gate_bwd(const void* g, const float* A_log, const float* g_bias, const void* d_out, void* d_g, float* d_A_log,
                     float* d_bias, int64_t rows, int32_t H, int32_t dk, float threshold, int32_t dtype, int32_t out_dtype,
                     void* workspace, uint64_t workspace_bytes, void* hip_stream);
int lnx_sigmoid_fwd(const float* x, float* y, int64_t n, void* hip_stream);
int lnx_sigmoid_bwd(const float* y, const float* dy, float* dx, int64_t n, void* hip_stream);

/*
 * Optional per-kernel timing for benchmarks (no counterpart in the reference; its micro-benchmark
 * times whole jitted ops, bench_kda_kernels.py:216-249).  While enabled (process-wide),
 * every entry point records HIP events around each kernel it launches, on the caller's stream.
 * lnx_profile_read waits for them, returns the number of kernels timed since the last read and
 * fills up to `capacity` (name, milliseconds) pairs.  At most 8192 marks (one per kernel plus one
 * per entry-point call) are kept between reads.  This is the one piece of process-wide mutable state in the
 * library (a mutex-guarded list of events, created on first use); it is off unless enabled, and calls on a
 * stream that is being captured into a graph take no marks, so the compute entry points stay capturable.
 */
int lnx_profile_enable(int on);
int lnx_profile_read(int capacity, const char** names, float* ms);

#ifdef __cplusplus
}
#endif
#endif /* LINEARNEXUS_HIP_H */
