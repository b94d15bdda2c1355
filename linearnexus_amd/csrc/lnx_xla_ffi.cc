// XLA FFI handlers over the C-ABI of liblinearnexus_hip.so: what a JAX caller registers with
// jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(symbol), platform="ROCM") in place of the reference's
// `try accelerated -> except -> fallback` seam (linearnexus/kernels/backend.py:38-60,
// linearnexus/modules/linear_attn/delta_net.py:150-156).  One file, no state: every handler unpacks its buffers and
// attributes into an lnx_scan_args block and calls one entry point on the stream XLA hands over.
//
// Built by linearnexus_amd/build.py only where the XLA FFI headers exist (jax.ffi.include_dir(), or the directory
// named by XLA_FFI_INCLUDE_DIR): the image this library is developed in has neither JAX nor the headers, so this file
// is compiled on the installation that has them.
//
// Conventions shared by the four handlers:
//   * q, k, v are [B, H, T, d] (token_first = 0, the reference's layout) or [B, T, H, d] (token_first = 1); the decode
//     step takes [B, H, d].  dtype is q's element type (F32 or BF16), o_dtype the output buffer's.
//   * An optional operand (g, initial_state, cu_seqlens, d_final_state) is passed as a buffer with zero elements when
//     absent -- XLA FFI has no optional operands -- and reaches the C-ABI as NULL.
//   * gate: 0 none, 1 scalar g [B,H,T], 2 per-channel g [B,H,T,dk] (lnx_gate).
//   * The chunk workspace is a U8 result of LnxChunkFwd sized by lnx_chunk_workspace_bytes at trace time; LnxChunkBwd
//     takes it as an operand aliased to a result of the same shape (input_output_aliases), because the backward kernels
//     write their own per-chunk tensors into it.
//   * LnxDecodeStep's state result is meant to alias its state operand ({5: 1} in input_output_aliases with the state
//     donated): the 512 MiB state of the decode configuration is then updated in place; without the alias XLA passes
//     two buffers and the kernel reads one and writes the other.

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "../../include/linearnexus_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

struct Attrs {
  int32_t gate, token_first, forward_only, use_qk_l2norm, nseq;
  float scale;
};

const void* ptr_or_null(const ffi::AnyBuffer& b) { return b.element_count() == 0 ? nullptr : b.untyped_data(); }

bool dtype_of(ffi::DataType t, int32_t* out) {
  if (t == ffi::DataType::F32) { *out = LNX_F32; return true; }
  if (t == ffi::DataType::BF16) { *out = LNX_BF16; return true; }
  return false;
}

ffi::Error status(int rc, const char* what) {
  if (rc == LNX_OK) return ffi::Error::Success();
  return ffi::Error(rc == LNX_ERR_LAUNCH || rc == LNX_ERR_DEVICE ? ffi::ErrorCode::kInternal : ffi::ErrorCode::kInvalidArgument,
                    std::string(what) + ": " + lnx_last_error());
}

// Shapes and element types of the token tensors into `a`; false if q is not a rank-4 (rank-3: decode) F32/BF16 buffer.
bool fill_shapes(lnx_scan_args* a, const ffi::AnyBuffer& q, const ffi::AnyBuffer& v, const Attrs& at, bool decode) {
  const auto qd = q.dimensions();
  const auto vd = v.dimensions();
  if (decode) {
    if (qd.size() != 3 || vd.size() != 3) return false;
    a->B = (int32_t)qd[0]; a->H = (int32_t)qd[1]; a->T = 1; a->dk = (int32_t)qd[2]; a->dv = (int32_t)vd[2];
  } else {
    if (qd.size() != 4 || vd.size() != 4) return false;
    a->B = (int32_t)qd[0];
    a->H = (int32_t)qd[at.token_first ? 2 : 1];
    a->T = (int32_t)qd[at.token_first ? 1 : 2];
    a->dk = (int32_t)qd[3];
    a->dv = (int32_t)vd[3];
  }
  a->chunk = 64;
  a->gate = at.gate;
  a->scale = at.scale;
  a->token_first = at.token_first;
  a->forward_only = at.forward_only;
  a->use_qk_l2norm = at.use_qk_l2norm;
  a->nseq = at.nseq;
  return dtype_of(q.element_type(), &a->dtype);
}

void fill_inputs(lnx_scan_args* a, const ffi::AnyBuffer& q, const ffi::AnyBuffer& k, const ffi::AnyBuffer& v,
                 const ffi::AnyBuffer& beta, const ffi::AnyBuffer& g, const ffi::AnyBuffer& s0,
                 const ffi::AnyBuffer& cu) {
  a->q = q.untyped_data();
  a->k = k.untyped_data();
  a->v = v.untyped_data();
  a->beta = static_cast<const float*>(beta.untyped_data());
  a->g = static_cast<const float*>(ptr_or_null(g));
  a->initial_state = static_cast<const float*>(ptr_or_null(s0));
  a->cu_seqlens = static_cast<const int32_t*>(ptr_or_null(cu));
}

#define LNX_BAD_SHAPES() ffi::Error(ffi::ErrorCode::kInvalidArgument, "q, v must be rank-4 (decode: rank-3) F32 or BF16 buffers")

// ---- lnx_chunk_fwd: delta_rule_chunkwise / gated_delta_rule_chunkwise / kda_chunkwise ----
ffi::Error ChunkFwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer beta,
                        ffi::AnyBuffer g, ffi::AnyBuffer s0, ffi::AnyBuffer cu, ffi::Result<ffi::AnyBuffer> o,
                        ffi::Result<ffi::AnyBuffer> final_state, ffi::Result<ffi::AnyBuffer> workspace, int32_t gate,
                        float scale, int32_t token_first, int32_t forward_only, int32_t use_qk_l2norm, int32_t nseq) {
  lnx_scan_args a = {};
  const Attrs at = {gate, token_first, forward_only, use_qk_l2norm, nseq, scale};
  if (!fill_shapes(&a, q, v, at, false) || !dtype_of(o->element_type(), &a.o_dtype)) return LNX_BAD_SHAPES();
  fill_inputs(&a, q, k, v, beta, g, s0, cu);
  a.o = o->untyped_data();
  a.final_state = static_cast<float*>(final_state->untyped_data());
  a.workspace = workspace->untyped_data();
  a.workspace_bytes = workspace->size_bytes();
  return status(lnx_chunk_fwd(&a, stream), "lnx_chunk_fwd");
}

// ---- lnx_chunk_bwd: the custom_vjp backward rule of the three chunk ops ----
ffi::Error ChunkBwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer beta,
                        ffi::AnyBuffer g, ffi::AnyBuffer s0, ffi::AnyBuffer cu, ffi::AnyBuffer d_o,
                        ffi::AnyBuffer d_final_state, ffi::AnyBuffer workspace_in, ffi::Result<ffi::AnyBuffer> d_q,
                        ffi::Result<ffi::AnyBuffer> d_k, ffi::Result<ffi::AnyBuffer> d_v, ffi::Result<ffi::AnyBuffer> d_beta,
                        ffi::Result<ffi::AnyBuffer> d_g, ffi::Result<ffi::AnyBuffer> d_s0,
                        ffi::Result<ffi::AnyBuffer> workspace, int32_t gate, float scale, int32_t token_first,
                        int32_t use_qk_l2norm, int32_t nseq) {
  lnx_scan_args a = {};
  const Attrs at = {gate, token_first, 0, use_qk_l2norm, nseq, scale};
  if (!fill_shapes(&a, q, v, at, false)) return LNX_BAD_SHAPES();
  a.o_dtype = a.dtype;
  fill_inputs(&a, q, k, v, beta, g, s0, cu);
  a.d_o = d_o.untyped_data();
  a.d_final_state = static_cast<const float*>(ptr_or_null(d_final_state));
  a.d_q = d_q->untyped_data();
  a.d_k = d_k->untyped_data();
  a.d_v = d_v->untyped_data();
  a.d_beta = static_cast<float*>(d_beta->untyped_data());
  a.d_g = d_g->element_count() == 0 ? nullptr : static_cast<float*>(d_g->untyped_data());
  a.d_initial_state = d_s0->element_count() == 0 ? nullptr : static_cast<float*>(d_s0->untyped_data());
  // the forward's workspace, aliased: without the alias XLA hands over a fresh result buffer and the saved per-chunk
  // tensors are not in it
  if (workspace->untyped_data() != workspace_in.untyped_data())
    return ffi::Error(ffi::ErrorCode::kFailedPrecondition,
                      "LnxChunkBwd: the workspace result must alias the workspace operand (input_output_aliases)");
  a.workspace = workspace->untyped_data();
  a.workspace_bytes = workspace->size_bytes();
  return status(lnx_chunk_bwd(&a, stream), "lnx_chunk_bwd");
}

// ---- lnx_recurrent_fwd: delta_rule_recurrent / gated_delta_rule_recurrent / kda_recurrent ----
ffi::Error RecurrentFwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer beta,
                            ffi::AnyBuffer g, ffi::AnyBuffer s0, ffi::AnyBuffer cu, ffi::Result<ffi::AnyBuffer> o,
                            ffi::Result<ffi::AnyBuffer> final_state, int32_t gate, float scale, int32_t token_first,
                            int32_t use_qk_l2norm, int32_t nseq) {
  lnx_scan_args a = {};
  const Attrs at = {gate, token_first, 1, use_qk_l2norm, nseq, scale};
  if (!fill_shapes(&a, q, v, at, false) || !dtype_of(o->element_type(), &a.o_dtype)) return LNX_BAD_SHAPES();
  fill_inputs(&a, q, k, v, beta, g, s0, cu);
  a.o = o->untyped_data();
  a.final_state = static_cast<float*>(final_state->untyped_data());
  return status(lnx_recurrent_fwd(&a, stream), "lnx_recurrent_fwd");
}

// ---- lnx_decode_step: delta_rule_step / gated_delta_rule_step / kda_step ----
ffi::Error DecodeStepImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer beta,
                          ffi::AnyBuffer g, ffi::AnyBuffer state, ffi::Result<ffi::AnyBuffer> o,
                          ffi::Result<ffi::AnyBuffer> state_out, int32_t gate, float scale, int32_t use_qk_l2norm) {
  lnx_scan_args a = {};
  const Attrs at = {gate, 0, 1, use_qk_l2norm, 0, scale};
  if (!fill_shapes(&a, q, v, at, true) || !dtype_of(o->element_type(), &a.o_dtype)) return LNX_BAD_SHAPES();
  a.q = q.untyped_data();
  a.k = k.untyped_data();
  a.v = v.untyped_data();
  a.beta = static_cast<const float*>(beta.untyped_data());
  a.g = static_cast<const float*>(ptr_or_null(g));
  a.initial_state = static_cast<const float*>(state.untyped_data());
  a.final_state = static_cast<float*>(state_out->untyped_data());  // the same address when XLA honoured the alias
  a.o = o->untyped_data();
  return status(lnx_decode_step(&a, stream), "lnx_decode_step");
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(LnxChunkFwd, ChunkFwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v
                                  .Arg<ffi::AnyBuffer>()   // beta  f32
                                  .Arg<ffi::AnyBuffer>()   // g     f32, zero elements when gate == 0
                                  .Arg<ffi::AnyBuffer>()   // initial_state f32, zero elements = zeros
                                  .Arg<ffi::AnyBuffer>()   // cu_seqlens s32 [nseq + 1], zero elements = dense batch
                                  .Ret<ffi::AnyBuffer>()   // o
                                  .Ret<ffi::AnyBuffer>()   // final_state f32
                                  .Ret<ffi::AnyBuffer>()   // workspace u8 [lnx_chunk_workspace_bytes]
                                  .Attr<int32_t>("gate")
                                  .Attr<float>("scale")
                                  .Attr<int32_t>("token_first")
                                  .Attr<int32_t>("forward_only")
                                  .Attr<int32_t>("use_qk_l2norm")
                                  .Attr<int32_t>("nseq"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(LnxChunkBwd, ChunkBwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v
                                  .Arg<ffi::AnyBuffer>()   // beta
                                  .Arg<ffi::AnyBuffer>()   // g
                                  .Arg<ffi::AnyBuffer>()   // initial_state
                                  .Arg<ffi::AnyBuffer>()   // cu_seqlens
                                  .Arg<ffi::AnyBuffer>()   // d_o (q's element type)
                                  .Arg<ffi::AnyBuffer>()   // d_final_state f32, zero elements = zeros
                                  .Arg<ffi::AnyBuffer>()   // workspace from LnxChunkFwd (aliased to the last result)
                                  .Ret<ffi::AnyBuffer>()   // d_q
                                  .Ret<ffi::AnyBuffer>()   // d_k
                                  .Ret<ffi::AnyBuffer>()   // d_v
                                  .Ret<ffi::AnyBuffer>()   // d_beta f32
                                  .Ret<ffi::AnyBuffer>()   // d_g f32, zero elements when gate == 0
                                  .Ret<ffi::AnyBuffer>()   // d_initial_state f32, zero elements = not wanted
                                  .Ret<ffi::AnyBuffer>()   // workspace
                                  .Attr<int32_t>("gate")
                                  .Attr<float>("scale")
                                  .Attr<int32_t>("token_first")
                                  .Attr<int32_t>("use_qk_l2norm")
                                  .Attr<int32_t>("nseq"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(LnxRecurrentFwd, RecurrentFwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v
                                  .Arg<ffi::AnyBuffer>()   // beta
                                  .Arg<ffi::AnyBuffer>()   // g
                                  .Arg<ffi::AnyBuffer>()   // initial_state
                                  .Arg<ffi::AnyBuffer>()   // cu_seqlens
                                  .Ret<ffi::AnyBuffer>()   // o
                                  .Ret<ffi::AnyBuffer>()   // final_state
                                  .Attr<int32_t>("gate")
                                  .Attr<float>("scale")
                                  .Attr<int32_t>("token_first")
                                  .Attr<int32_t>("use_qk_l2norm")
                                  .Attr<int32_t>("nseq"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(LnxDecodeStep, DecodeStepImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()   // q [B,H,dk]
                                  .Arg<ffi::AnyBuffer>()   // k
                                  .Arg<ffi::AnyBuffer>()   // v [B,H,dv]
                                  .Arg<ffi::AnyBuffer>()   // beta [B,H]
                                  .Arg<ffi::AnyBuffer>()   // g [B,H] | [B,H,dk] | zero elements
                                  .Arg<ffi::AnyBuffer>()   // state [B,H,dk,dv] f32 (donated)
                                  .Ret<ffi::AnyBuffer>()   // o [B,H,dv]
                                  .Ret<ffi::AnyBuffer>()   // state, aliased to operand 5
                                  .Attr<int32_t>("gate")
                                  .Attr<float>("scale")
                                  .Attr<int32_t>("use_qk_l2norm"));
