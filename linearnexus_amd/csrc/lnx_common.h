// Shared device helpers for the gfx950 delta-rule kernels: element types, conversions,
// wavefront reductions and the error channel of the C-ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/linearnexus_hip.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define LNX_WAVE 64
#define LNX_L2_EPS 1e-6f

// Host side: records a message for lnx_last_error() and returns `code`.
int lnx_set_error(int code, const char* fmt, ...);

// Host side: when per-kernel timing is enabled (lnx_profile_enable), records a HIP event on
// `st` before the kernel named `kernel_name`; a NULL name closes the current entry point.
#define LNX_PROFILE_MAX 8192
void lnx_profile_mark(const char* kernel_name, hipStream_t st);

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

// Four consecutive elements as they lie in memory: what a prefetch keeps in registers until the value is used.
template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef floatx4 V; };
template <> struct Vec4<bf16_t> { typedef bf16x4 V; };

// Loads 4 consecutive elements as fp32.
__device__ __forceinline__ floatx4 load4(const float* p) { return *reinterpret_cast<const floatx4*>(p); }
__device__ __forceinline__ floatx4 load4(const bf16_t* p) {
  bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
  floatx4 r = {(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
  return r;
}
// Four fp32 -> four bf16 (round to nearest even) as two v_cvt_pk_bf16_f32 joined as integers: written as a four-element
// conversion, or element by element, hipcc takes the vector apart -- one conversion per element and a v_perm_b32 per
// pair to put them back together, three instructions where one does.
__device__ __forceinline__ bf16x4 pack_bf16x4(floatx4 v) {
  typedef unsigned uint2_ __attribute__((ext_vector_type(2)));
  const uint2_ r = {__builtin_bit_cast(unsigned, __builtin_convertvector((floatx2{v[0], v[1]}), bf16x2)),
                    __builtin_bit_cast(unsigned, __builtin_convertvector((floatx2{v[2], v[3]}), bf16x2))};
  return __builtin_bit_cast(bf16x4, r);
}
__device__ __forceinline__ void store4(float* p, floatx4 x) { *reinterpret_cast<floatx4*>(p) = x; }
__device__ __forceinline__ void store4(bf16_t* p, floatx4 x) { *reinterpret_cast<bf16x4*>(p) = pack_bf16x4(x); }

// Token range [seq_first, seq_end) of packed sequence s, read defensively: cu_seqlens lives in device memory where the
// host cannot check it, so entries are clamped to [0, T] and an end before its start reads as an empty sequence.  A
// well-formed table (cu[0] = 0, non-decreasing, cu[nseq] = T) is unchanged by this.
__device__ __forceinline__ int seq_first(const int32_t* cu, int s, int T) { return min(max(cu[s], 0), T); }
__device__ __forceinline__ int seq_end(const int32_t* cu, int s, int T) { return max(min(max(cu[s + 1], 0), T), seq_first(cu, s, T)); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits until every global
// load and store of the wave has completed, which puts the full memory latency of a register
// prefetch (and of streamed-out results) on the critical path of each loop iteration.  Use this
// one wherever the data exchanged between the waves lives in LDS; global memory written by one
// wave and read back by another in the same kernel still needs __syncthreads().
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Sum over all 64 lanes; every lane gets the total.
// Sum over the four lanes of a quad (lanes 4q .. 4q+3), in every lane: two DPP quad permutes, no LDS crossbar.
__device__ __forceinline__ float quad_sum(float x) {
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));  // lanes [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));  // lanes [2,3,0,1]
  return x;
}

// x + (x of lane ^ 16) and x + (x of lane ^ 32), in every lane, on the VALU: v_permlane16_swap exchanges the odd rows
// (16 lanes) of its first operand with the even rows of its second, v_permlane32_swap the upper half of the first
// with the lower half of the second; fed the same value twice they return it with the even rows / lower half
// repeated and with the odd rows / upper half repeated.  (A shuffle would go through the LDS crossbar.)
__device__ __forceinline__ float xor16_sum(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor32_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float wave_sum(float x) {
  // inside a row of 16 lanes with DPP (no LDS crossbar): quads, the two quads of a half row, the two half rows
  x = quad_sum(x);
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xF, 0xF, true));  // row_half_mirror: lane i <-> 7 - i
  x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x128, 0xF, 0xF, true));  // row_ror:8 = lane ^ 8
  return xor32_sum(xor16_sum(x));
}
