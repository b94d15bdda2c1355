// MFMA tile primitives for gfx950 shared by the chunk kernels.
//
// All block-level products have the "NT" form C[M x N] += A[M x K] * B[N x K]^T with both
// operands K-contiguous in LDS, which is the native operand layout of the 32x32 MFMA
// instructions: lane = (row r = lane & 31, k-group kg = lane >> 5) holds VEC consecutive
// k-elements of row r.  bf16 uses v_mfma_f32_32x32x16_bf16 (8 elements per lane), fp32 uses
// four v_mfma_f32_32x32x2_f32 per 8-wide k-step (4 elements per lane).
//
// Accumulator fragment (floatx16) of one 32x32 tile: element e of lane l is
//   row = 8 * (e / 4) + 4 * (l >> 5) + (e % 4),  col = l & 31.
// Four consecutive e share a column and cover four consecutive rows, so a fragment can be
// written transposed ([col][row]) with 4-element vector stores.
#pragma once

#include "lnx_common.h"

#define LNX_C 64  // chunk length (tokens)

template <typename T> struct Mma;

template <> struct Mma<bf16_t> {
  static constexpr int KS = 16;   // k per step
  static constexpr int VEC = 8;   // elements per lane per step == elements per 16-byte vector
  static constexpr int PAD = 8;   // LDS row padding (elements) = 16 bytes
  typedef bf16x8 Frag;
  typedef bf16x4 Quad;
  static __device__ __forceinline__ Frag load(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
  static __device__ __forceinline__ void mma(floatx16& c, const Frag& a, const Frag& b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // Operand fragment whose contraction index runs along the ROWS of a row-major LDS tile:
  // lane (r = lane & 31, kg = lane >> 5) gets tile[k0 + 8 kg + 0..7][c0 + r].  Two
  // ds_read_b64_tr_b16: inside a 16-lane group, result element j of lane L is element (L % 4) of
  // what lane 4 j + L / 4 addressed, so source lane s = 4 j + q points at row j, columns 4 q .. 4 q + 3.
  static __device__ __forceinline__ Frag load_t(const bf16_t* tile, int ld, int k0, int c0, int lane) {
    typedef short short4_ __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) short4_ lds_short4;
    const int s = lane & 15, grp = lane >> 4;
    const bf16_t* p = tile + (k0 + 8 * (grp >> 1) + (s >> 2)) * ld + c0 + 16 * (grp & 1) + 4 * (s & 3);
    const short4_ lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p));
    const short4_ hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p + 4 * ld));
    typedef short short8_ __attribute__((ext_vector_type(8)));
    const short8_ v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(Frag, v);
  }

  // ---- chaining products through registers ----
  // A 32x32 accumulator fragment can be the B operand of the next product without a trip through LDS when the
  // contraction runs over the fragment's rows: lane (n = lane & 31, kg = lane >> 5) holds, as elements 8 h .. 8 h + 7
  // of the fragment (h = 0, 1), the rows  16 h + 4 kg + (0..3)  and  16 h + 8 + 4 kg + (0..3)  of column n.  The MFMA
  // only needs both operands to agree on which contraction index sits in which slot, so the A operand is loaded in
  // that same order ("chain order") with two 8-byte reads instead of one 16-byte read.
  static __device__ __forceinline__ Frag from_acc(const floatx16& c, int h) {
    typedef unsigned uint4_ __attribute__((ext_vector_type(4)));
    typedef unsigned uint2_ __attribute__((ext_vector_type(2)));
    const uint2_ lo = __builtin_bit_cast(uint2_, pack_bf16x4(floatx4{c[8 * h], c[8 * h + 1], c[8 * h + 2], c[8 * h + 3]}));
    const uint2_ hi = __builtin_bit_cast(uint2_, pack_bf16x4(floatx4{c[8 * h + 4], c[8 * h + 5], c[8 * h + 6], c[8 * h + 7]}));
    return __builtin_bit_cast(Frag, (uint4_{lo[0], lo[1], hi[0], hi[1]}));
  }
  // A operand in chain order from a [rows][k] tile: p points at (this lane's row, first k of the 16-wide step)
  static __device__ __forceinline__ Frag load_chain(const bf16_t* p, int lane) {
    const bf16_t* q = p + 4 * (lane >> 5);
    const bf16x4 lo = *reinterpret_cast<const bf16x4*>(q), hi = *reinterpret_cast<const bf16x4*>(q + 8);
    Frag v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return v;
  }
  // A operand in chain order from a row-major [k][rows] tile (contraction along the tile's rows), like load_t
  static __device__ __forceinline__ Frag load_t_chain(const bf16_t* tile, int ld, int k0, int c0, int lane) {
    typedef short short4_ __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) short4_ lds_short4;
    const int s = lane & 15, grp = lane >> 4;
    const bf16_t* p = tile + (k0 + 4 * (grp >> 1) + (s >> 2)) * ld + c0 + 16 * (grp & 1) + 4 * (s & 3);
    const short4_ lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p));
    const short4_ hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p + 8 * ld));
    typedef short short8_ __attribute__((ext_vector_type(8)));
    const short8_ v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(Frag, v);
  }
  // Four consecutive rows of this lane's column of a row-major tile, i.e. elements 4 q .. 4 q + 3 of an accumulator
  // fragment's position: tile[r0 + 8 q + 4 (lane >> 5) + (0..3)][c0 + (lane & 31)], one transposing read.
  static __device__ __forceinline__ bf16x4 load_acc_rows_raw(const bf16_t* tile, int ld, int r0, int q, int c0, int lane) {
    typedef short short4_ __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) short4_ lds_short4;
    const int s = lane & 15, grp = lane >> 4;
    const bf16_t* p = tile + (r0 + 8 * q + 4 * (grp >> 1) + (s >> 2)) * ld + c0 + 16 * (grp & 1) + 4 * (s & 3);
    return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p)));
  }
  static __device__ __forceinline__ floatx4 load_acc_rows(const bf16_t* tile, int ld, int r0, int q, int c0, int lane) {
    typedef short short4_ __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) short4_ lds_short4;
    const int s = lane & 15, grp = lane >> 4;
    const bf16_t* p = tile + (r0 + 8 * q + 4 * (grp >> 1) + (s >> 2)) * ld + c0 + 16 * (grp & 1) + 4 * (s & 3);
    const short4_ x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p));
    const bf16x4 y = __builtin_bit_cast(bf16x4, x);
    floatx4 r = {(float)y[0], (float)y[1], (float)y[2], (float)y[3]};
    return r;
  }
};

template <> struct Mma<float> {
  static constexpr int KS = 8;
  static constexpr int VEC = 4;
  static constexpr int PAD = 4;
  typedef floatx4 Frag;
  typedef floatx4 Quad;
  static __device__ __forceinline__ Frag load(const float* p) { return *reinterpret_cast<const floatx4*>(p); }
  static __device__ __forceinline__ void mma(floatx16& c, const Frag& a, const Frag& b) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
  }
  // fp32: one element per MFMA, so the transposed-source fragment is four conflict-free scalar reads
  static __device__ __forceinline__ Frag load_t(const float* tile, int ld, int k0, int c0, int lane) {
    const float* p = tile + (k0 + 4 * (lane >> 5)) * ld + c0 + (lane & 31);
    Frag v = {p[0], p[ld], p[2 * ld], p[3 * ld]};
    return v;
  }
};

template <int MT, int NT>
__device__ __forceinline__ void frag_zero(floatx16 (&acc)[MT][NT]) {
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
}

// acc[i][j] += A[32 i .. , :K] * B[32 j .. , :K]^T ; A, B point at this wave's first rows.
template <typename T, int MT, int NT>
__device__ __forceinline__ void mma_nt(floatx16 (&acc)[MT][NT], const T* A, int lda, const T* B, int ldb, int K,
                                       int lane) {
  typedef Mma<T> M;
  const int r = lane & 31, ko = (lane >> 5) * M::VEC;
  const T* ap = A + r * lda + ko;
  const T* bp = B + r * ldb + ko;
  for (int k0 = 0; k0 < K; k0 += M::KS) {
    typename M::Frag a[MT], b[NT];
#pragma unroll
    for (int i = 0; i < MT; ++i) a[i] = M::load(ap + i * 32 * lda + k0);
#pragma unroll
    for (int j = 0; j < NT; ++j) b[j] = M::load(bp + j * 32 * ldb + k0);
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) M::mma(acc[i][j], a[i], b[j]);
  }
}

// General form: TA / TB say that the operand is given as a row-major [K][rows] tile (contraction
// index along the tile's rows; A / B then point at the tile's first used column) instead of the
// native [rows][K] layout.
template <typename T, int MT, int NT, bool TA, bool TB>
__device__ __forceinline__ void mma_x(floatx16 (&acc)[MT][NT], const T* A, int lda, const T* B, int ldb, int K,
                                      int lane) {
  typedef Mma<T> M;
  const int r = lane & 31, ko = (lane >> 5) * M::VEC;
  for (int k0 = 0; k0 < K; k0 += M::KS) {
    typename M::Frag a[MT], b[NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
      a[i] = TA ? M::load_t(A, lda, k0, 32 * i, lane) : M::load(A + (r + 32 * i) * lda + ko + k0);
#pragma unroll
    for (int j = 0; j < NT; ++j)
      b[j] = TB ? M::load_t(B, ldb, k0, 32 * j, lane) : M::load(B + (r + 32 * j) * ldb + ko + k0);
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) M::mma(acc[i][j], a[i], b[j]);
  }
}

// ---------------------------------------------------------------------------------------
// Loads that go straight to LDS (global_load_lds_dwordx4): one wave instruction fetches 16 bytes per lane from per-lane
// global addresses and writes them to 1 KB of consecutive LDS, lane l at `dst` + 16 l; no registers hold the data, so
// whole slabs can be in flight behind the one being multiplied.  The LDS layout of a tile is therefore unpadded; which
// 16-byte granule a lane fetches is free, so the granules of a row are permuted by an XOR of the row index instead
// (SwzTile) -- rows that an access pattern reads together land in different banks.  The compiler does not know that
// these instructions write LDS or count towards vmcnt: the callers wait with dma_wait<N>() (all but the N youngest of
// this wave's memory instructions have completed; the counter retires in order) and a workgroup barrier before reading.
// ---------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) char lds_char_t;
__device__ __forceinline__ unsigned lds_byte_addr(const void* p) { return (unsigned)(uintptr_t)(lds_char_t*)p; }
__device__ __forceinline__ void dma16(const void* src, unsigned dst) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(__builtin_amdgcn_readfirstlane(dst)) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// A [ROWS][COLS] bf16 tile in LDS without padding, COLS * 2 bytes per row, granule g (16 bytes) of row r at granule
// position g ^ x(r).  x is chosen so that both ways of reading the tile touch every bank once per access:
//   a row read (16 lanes = 16 consecutive rows, one granule each) needs 16 rows on 16 different 16-byte slots of the
//   256 bytes of bank space, a transposing read (half a wave = 4 consecutive rows r0 % 4 == 0 times 4 aligned granules)
//   needs the 4 rows on different 64-byte quarters:
//   256-byte rows: x = 4 (r % 4) + r / 4 % 4;  128-byte rows: x = 4 (r / 2 % 2) + r / 4 % 4;  64-byte rows: x = r / 4 % 4.
// Tiles of 256- or 128-byte rows that are only read through transposing reads (ROW_READS = false) drop the second
// term: fewer address instructions.
template <int ROWS, int COLS, bool ROW_READS = true> struct SwzTile {
  typedef bf16_t T;
  typedef Mma<bf16_t> M;
  typedef short short4_ __attribute__((ext_vector_type(4)));
  typedef short short8_ __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) short4_ lds_short4;
  static constexpr int G = COLS / 8, BYTES = ROWS * COLS * 2, NINSTR = BYTES / 1024;
  static_assert(G == 16 || G == 8 || G == 4, "rows of 256, 128 or 64 bytes");
  static __device__ __forceinline__ int x(int r) {
    const int lo = ROW_READS || G == 4 ? (r >> 2) & 3 : 0;
    return G == 16 ? ((r & 3) << 2) | lo : G == 8 ? (((r >> 1) & 1) << 2) | lo : lo;
  }
  // element offset of (row r, column c)
  static __device__ __forceinline__ int at(int r, int c) { return r * COLS + ((((c >> 3) ^ x(r)) << 3) | (c & 7)); }
  // instruction j of the tile's load: the row and the column of the granule this lane fetches
  static __device__ __forceinline__ void src(int j, int lane, int& r, int& c) {
    const int p = 64 * j + lane;
    r = p / G;
    c = ((p % G) ^ x(r)) << 3;
  }
  // the four consecutive rows r0 .. r0 + 3 (r0 % 4 == 0) of column c0 + (this lane's column): one transposing read
  static __device__ __forceinline__ short4_ tr4(const T* tile, int r0, int c0, int lane) {
    const int s = lane & 15;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(tile + at(r0 + (s >> 2), c0 + 4 * (s & 3))));
  }
  // Mma::load_t on the swizzled tile: contraction index along the tile's rows k0 .. k0 + 15, columns c0 .. c0 + 31
  static __device__ __forceinline__ typename M::Frag load_t(const T* tile, int k0, int c0, int lane) {
    const int grp = lane >> 4;
    const short4_ lo = tr4(tile, k0 + 8 * (grp >> 1), c0 + 16 * (grp & 1), lane);
    const short4_ hi = tr4(tile, k0 + 8 * (grp >> 1) + 4, c0 + 16 * (grp & 1), lane);
    const short8_ v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(typename M::Frag, v);
  }
  // Mma::load on the swizzled tile: eight consecutive elements of row r from column c (c % 8 == 0)
  static __device__ __forceinline__ typename M::Frag load(const T* tile, int r, int c) {
    return *reinterpret_cast<const typename M::Frag*>(tile + at(r, c));
  }
};

__device__ __forceinline__ int frag_row(int e, int lane) { return 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3); }
__device__ __forceinline__ int frag_col(int lane) { return lane & 31; }

// dst[row][col] = acc (row-major tile with leading dimension ld); dst points at the tile origin.
template <typename T, int MT, int NT>
__device__ __forceinline__ void frag_store(const floatx16 (&acc)[MT][NT], T* dst, int64_t ld, int lane,
                                           int row_limit = 1 << 30) {
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = 32 * i + frag_row(e, lane);
        if (row < row_limit) dst[row * ld + 32 * j + frag_col(lane)] = from_f32<T>(acc[i][j][e]);
      }
}

// dst[col][row] = acc: transposed store, four consecutive rows per vector.
template <typename T, int MT, int NT>
__device__ __forceinline__ void frag_store_t(const floatx16 (&acc)[MT][NT], T* dst, int64_t ld, int lane) {
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = 32 * i + 8 * q + 4 * (lane >> 5);
        const int col = 32 * j + frag_col(lane);
        floatx4 x = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        store4(dst + col * ld + row, x);
      }
}

// ---------------------------------------------------------------------------------------
// global <-> LDS staging of [rows x cols] tiles by a 256-thread block
// ---------------------------------------------------------------------------------------

template <typename T> struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  typedef typename Mma<T>::Frag V;
};

template <typename T>
__device__ __forceinline__ typename Vec16<T>::V vec_zero() {
  typename Vec16<T>::V z;
#pragma unroll
  for (int e = 0; e < Vec16<T>::N; ++e) z[e] = (T)0.f;
  return z;
}

// A [ROWS x COLS] tile held in registers between its global loads and its LDS stores, so that a
// kernel can issue the loads of all tiles of a phase before it waits for any of them.
// Rows >= valid read as zero (valid <= 0: the whole tile).  COLS % VEC == 0.
// The loads are buffer loads through a descriptor that covers exactly the valid rows: the hardware's range check
// returns zeros past the end, the per-thread offsets do not depend on the chunk (no address arithmetic in vector
// registers per load), and no load sits behind a branch or a select -- either would keep the compiler from
// counting the loads in flight exactly, and it would then make the next tile store wait for (nearly) all of
// them, younger prefetches included.
template <typename T, int ROWS, int COLS> struct TileRegs {
  static constexpr int N = Vec16<T>::N, VPR = COLS / N, TOTAL = ROWS * VPR, IT = (TOTAL + 255) / 256;
  typename Vec16<T>::V x[IT];
  __device__ __forceinline__ void load(const T* src, int64_t stride, int valid, int tid) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const int bytes = valid > 0 ? (int)(valid * stride * (int64_t)sizeof(T)) : 0;
    // raw buffer (no stride, no swizzle) of `bytes` bytes; 0x00020000: 32-bit data format, as untyped loads need
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(src), 0, bytes, 0x00020000);
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
      const u32x4 raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)((r * stride + c) * (int64_t)sizeof(T)), 0, 0);
      x[it] = __builtin_bit_cast(typename Vec16<T>::V, raw);
    }
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int it = 0; it < IT; ++it) x[it] = vec_zero<T>();
  }
  __device__ __forceinline__ typename Vec16<T>::V get(int it, int) const { return x[it]; }
  __device__ __forceinline__ void store(T* dst, int ld, int tid) const {
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
      if (idx < TOTAL) *reinterpret_cast<typename Vec16<T>::V*>(dst + r * ld + c) = x[it];
    }
  }
};

// A lower-triangular [64 x 64] 2-byte tile travels packed: of its 512 eight-element vectors (row r, columns 8 c .. 8 c + 7)
// only the 288 with 8 c <= r can hold a non-zero.  Rows come in groups of eight; group g has g + 1 vectors per row and starts
// at packed index 4 g (g + 1); a slot of the workspace keeps its 64 x 64 elements and uses the first 288 x 16 bytes.
constexpr int LNX_TRI_VECS = 288;
__device__ __forceinline__ void tri_vec_pos(int idx, int& r, int& c) {  // idx < LNX_TRI_VECS
  int g = 0;
#pragma unroll
  for (int h = 1; h < 8; ++h) g += (4 * h * (h + 1) <= idx) ? 1 : 0;
  const int o = idx - 4 * g * (g + 1);  // < 64
  // o / (g + 1) without an integer division: (o + 0.5) / (g + 1) is at least 1/16 away from every integer
  const int q = (int)(((float)o + 0.5f) * __builtin_amdgcn_rcpf((float)(g + 1)));
  r = 8 * g + q;
  c = o - q * (g + 1);
}
// The packed tile in the registers of 256 threads (vector tid, and vector 256 + tid for tid < 32) between its global
// loads and its LDS stores, like TileRegs; the LDS tile's upper part is zeroed once by the caller and never written.
template <typename T> struct TriRegs {
  static_assert(sizeof(T) == 2, "packed triangles are a 2-byte format");
  typename Vec16<T>::V x[2];
  int o0, o1;  // LDS element offsets of this thread's two vectors for a leading dimension fixed at init
  bool second;
  __device__ __forceinline__ void init(int ld, int tid) {
    int r, c;
    tri_vec_pos(tid, r, c);
    o0 = r * ld + 8 * c;
    second = tid < LNX_TRI_VECS - 256;
    tri_vec_pos(second ? 256 + tid : LNX_TRI_VECS - 1, r, c);
    o1 = r * ld + 8 * c;
  }
  __device__ __forceinline__ void load(const T* src, int tid) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(src), 0, LNX_TRI_VECS * 16, 0x00020000);
    x[0] = __builtin_bit_cast(typename Vec16<T>::V, __builtin_amdgcn_raw_buffer_load_b128(rsrc, 16 * tid, 0, 0));
    // threads without a second vector read past the end: the range check returns zeros, nothing sits behind a branch
    x[1] = __builtin_bit_cast(typename Vec16<T>::V, __builtin_amdgcn_raw_buffer_load_b128(rsrc, 16 * (256 + tid), 0, 0));
  }
  __device__ __forceinline__ void store(T* dst) const {
    *reinterpret_cast<typename Vec16<T>::V*>(dst + o0) = x[0];
    if (second) *reinterpret_cast<typename Vec16<T>::V*>(dst + o1) = x[1];
  }
};

// One-shot form (load, then store) for a single tile.
template <typename T, int ROWS, int COLS>
__device__ __forceinline__ void stage_tile(T* dst, int ld, const T* src, int64_t stride, int valid, int tid) {
  TileRegs<T, ROWS, COLS> t;
  t.load(src, stride, valid, tid);
  t.store(dst, ld, tid);
}

// LDS tile [ROWS][COLS] (leading dimension ld) -> global, 16-byte vectors, rows < valid only.
// FULL: every row is written and the tile is a whole number of 256-thread passes, so the loads
// and stores are unconditional and issued as two batches.
template <typename T, int ROWS, int COLS, bool FULL = false>
__device__ __forceinline__ void unstage_tile(T* dst, int64_t stride, const T* src, int ld, int valid, int tid) {
  typedef typename Vec16<T>::V V;
  constexpr int N = Vec16<T>::N, VPR = COLS / N, TOTAL = ROWS * VPR, IT = (TOTAL + 255) / 256;
  if constexpr (FULL) {
    static_assert(TOTAL % 256 == 0, "whole passes only");
    V x[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
      x[it] = *reinterpret_cast<const V*>(src + r * ld + c);
    }
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
      *reinterpret_cast<V*>(dst + r * stride + c) = x[it];
    }
  } else {
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
      if (idx < TOTAL && r < valid) *reinterpret_cast<V*>(dst + r * stride + c) = *reinterpret_cast<const V*>(src + r * ld + c);
    }
  }
}

// The same through a buffer descriptor that covers rows < valid only: the hardware drops the stores past the end, so
// no store sits behind a branch and a loop that also prefetches can count its memory instructions exactly.
template <typename T, int ROWS, int COLS>
__device__ __forceinline__ void unstage_tile_checked(T* dst, int64_t stride, const T* src, int ld, int valid, int tid) {
  typedef typename Vec16<T>::V V;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  constexpr int N = Vec16<T>::N, VPR = COLS / N, TOTAL = ROWS * VPR, IT = TOTAL / 256;
  static_assert(TOTAL % 256 == 0, "whole passes only");
  const int bytes = valid > 0 ? (int)(valid * stride * (int64_t)sizeof(T)) : 0;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(dst, 0, bytes, 0x00020000);
  V x[IT];
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
    x[it] = *reinterpret_cast<const V*>(src + r * ld + c);
  }
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * N;
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, x[it]), rsrc, (int)((r * stride + c) * (int64_t)sizeof(T)), 0, 0);
  }
}

// A bf16 LDS tile written out as fp32 rows (same range check): the direct-solve forward scan stages its outputs in
// bf16 -- the precision the reference returns them in for bf16 inputs -- and widens them here when the caller asked
// for fp32 outputs.
template <int ROWS, int COLS>
__device__ __forceinline__ void unstage_tile_checked_widen(float* dst, int64_t stride, const bf16_t* src, int ld, int valid, int tid) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  constexpr int VPR = COLS / 8, TOTAL = ROWS * VPR, IT = TOTAL / 256;
  static_assert(TOTAL % 256 == 0, "whole passes only");
  const int bytes = valid > 0 ? (int)(valid * stride * (int64_t)sizeof(float)) : 0;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(dst, 0, bytes, 0x00020000);
  bf16x8 x[IT];
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * 8;
    x[it] = *reinterpret_cast<const bf16x8*>(src + r * ld + c);
  }
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + 256 * it, r = idx / VPR, c = (idx - r * VPR) * 8;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const floatx4 y = {(float)x[it][4 * h], (float)x[it][4 * h + 1], (float)x[it][4 * h + 2], (float)x[it][4 * h + 3]};
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, y), rsrc, (int)((r * stride + c + 4 * h) * (int64_t)sizeof(float)), 0, 0);
    }
  }
}

// Sums f(e) * acc[i][0][e] over the 32 lanes that share rows, for all 16*MT rows of a wave's
// fragments at once, by a transpose-reduce (31 shuffles per 32 values instead of 160), then adds
// the row totals into rows[] (LDS) with one atomic per row and wave.  Callers zero rows[] and have at most two waves
// per row, so the result does not depend on the order of arrival (0 + a + b = 0 + b + a in floating point).
template <int MT>
__device__ __forceinline__ void rows_reduce_add(float (&v)[16 * MT], int row0, int lane, float* rows) {
  // after the step with mask m, v[t] (t < n/2) holds the partial for value index t + (lane & m ? n/2 : 0)
  static_assert(MT == 1 || MT == 2, "one or two row tiles");
  constexpr int NV = 16 * MT;
  int n = NV;
  // reduce value count down to 1 using lane bits 4,3,2,1 (and 0 when NV == 32); remaining lane bits by plain xor-adds
  constexpr int STEPS = (MT == 2) ? 5 : 4;
  int masks[5] = {16, 8, 4, 2, 1};
#pragma unroll
  for (int s_ = 0; s_ < STEPS; ++s_) {
    const int m = masks[s_];
    const int half = NV >> (s_ + 1);
    const bool hi = (lane & m) != 0;
#pragma unroll
    for (int t = 0; t < half; ++t) {
      const float a = v[t], b = v[t + half];
      const float send = hi ? a : b, keep = hi ? b : a;
      v[t] = keep + __shfl_xor(send, m, LNX_WAVE);
    }
  }
  (void)n;
  float total = v[0];
  if (MT == 1) total += __shfl_xor(total, 1, LNX_WAVE);  // 16 values: lane bit 0 still unreduced
  // value index owned by this lane: bits (4,3,2,1[,0]) of the lane select the halves kept
  int idx = 0;
#pragma unroll
  for (int s_ = 0; s_ < STEPS; ++s_) idx |= ((lane & masks[s_]) ? (NV >> (s_ + 1)) : 0);
  const int i = idx >> 4, e = idx & 15;
  if (MT == 2 || (lane & 1) == 0) atomicAdd(&rows[row0 + 32 * i + frag_row(e, lane)], total);
}

// ---------------------------------------------------------------------------------------
// 16x16 fp32 products on v_mfma_f32_16x16x4_f32, operands row-major in LDS
//   returns C[i][j] = sum_k A[i][k] * B[k][j];  fragment: c[e] is row 4*(lane>>4)+e, col lane&15
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ floatx4 mm16_f32(const float* A, int lda, const float* B, int ldb, int K, int lane) {
  floatx4 c = {0.f, 0.f, 0.f, 0.f};
  const int i = lane & 15, kq = lane >> 4;
  for (int k0 = 0; k0 < K; k0 += 4) {
    const float a = A[i * lda + k0 + kq];
    const float b = B[(k0 + kq) * ldb + i];
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  return c;
}

__device__ __forceinline__ void mm16_store(float* dst, int ld, floatx4 c, int lane, float sign) {
#pragma unroll
  for (int e = 0; e < 4; ++e) dst[(4 * (lane >> 4) + e) * ld + (lane & 15)] = sign * c[e];
}

#define LNX_LDA 68  // leading dimension of the fp32 64x64 matrices in LDS

// In-LDS inverse of the unit lower-triangular matrix I + A (A strictly lower, 64x64, fp32,
// leading dimension LNX_LDA):  Tm = (I + A)^-1.  `sA` is read only; `sT` receives the full
// matrix (upper triangle zero); `sX` is a [32][36] fp32 scratch.  Must be called by all 256
// threads.  Diagonal 16x16 blocks by forward substitution, then two levels of block merges
//   [[L0, 0], [B, L1]]^-1 = [[L0^-1, 0], [-L1^-1 B L0^-1, L1^-1]].
// In place (sT == sA, INPLACE): A's upper triangle and diagonal must hold zeros; every block of A is read for the last
// time before the barrier that precedes the write of the same block of Tm.
template <bool INPLACE = false>
__device__ __forceinline__ void tri_inverse_64(const float* sA, float* sT, float* sX, int tid) {
  const int wave = tid >> 6, lane = tid & 63;
  if (!INPLACE) {
    for (int idx = tid; idx < 64 * LNX_LDA; idx += 256) sT[idx] = 0.f;
    lds_barrier();
  }
  if (lane < 16) {
    const int r0 = 16 * wave, c = lane;
    float d[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float s = (i == c) ? 1.f : 0.f;
#pragma unroll
      for (int m = 0; m < i; ++m) s -= sA[(r0 + i) * LNX_LDA + r0 + m] * d[m];
      d[i] = s;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) sT[(r0 + i) * LNX_LDA + r0 + c] = d[i];
  }
  lds_barrier();
  // level 1: blocks (1,0) and (3,2) of the 16x16 grid, one per wave 0/1
  float* sXw = sX + (wave & 1) * 16 * 36;
  const int b = 32 * (wave & 1);  // super-block origin
  if (wave < 2) {
    floatx4 x = mm16_f32(sA + (b + 16) * LNX_LDA + b, LNX_LDA, sT + b * LNX_LDA + b, LNX_LDA, 16, lane);
    mm16_store(sXw, 36, x, lane, 1.f);
  }
  lds_barrier();
  if (wave < 2) {
    floatx4 y = mm16_f32(sT + (b + 16) * LNX_LDA + b + 16, LNX_LDA, sXw, 36, 16, lane);
    mm16_store(sT + (b + 16) * LNX_LDA + b, LNX_LDA, y, lane, -1.f);
  }
  lds_barrier();
  // level 2: the 32x32 lower-left block, one 16x16 output per wave
  const int bi = 16 * (wave >> 1), bj = 16 * (wave & 1);
  {
    floatx4 x = mm16_f32(sA + (32 + bi) * LNX_LDA, LNX_LDA, sT + bj, LNX_LDA, 32, lane);
    mm16_store(sX + bi * 36 + bj, 36, x, lane, 1.f);
  }
  lds_barrier();
  {
    floatx4 y = mm16_f32(sT + (32 + bi) * LNX_LDA + 32, LNX_LDA, sX + bj, 36, 32, lane);
    mm16_store(sT + (32 + bi) * LNX_LDA + bj, LNX_LDA, y, lane, -1.f);
  }
  lds_barrier();
}
