// Shared device helpers for the gfx950 kernels: vector types, bf16 packing, MFMA wrappers,
// wave-half exchange, the global->register->LDS staging of rotated / copied tiles and the transposing LDS read.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

// The attention kernels are written once for "the 16-bit element type" of q, k, v, dO and of every matrix-core operand:
// bf16 in the normal build of a source file, fp16 when the same file is compiled with -DCOROPE_F16, which also moves
// everything into the namespace corope_f16 so that both builds link into one library.
#ifdef COROPE_F16
#define COROPE_NS corope_f16
#else
#define COROPE_NS corope
#endif

namespace COROPE_NS {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int kWave = 64;

// ---- bf16 <-> fp32 --------------------------------------------------------------------------
// A 32-bit word holds two bf16: element 0 in the low half, element 1 in the high half.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// Round-to-nearest-even pack of two floats into one bf16x2 word (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}

// ---- MFMA ------------------------------------------------------------------------------------
// D(32x32) += A(32x16) * B(16x32), 16-bit elements in (bf16, or fp16 in the COROPE_F16 build), fp32 accumulate.
//   A operand: lane l holds row (l % 32), contraction slots 8*(l / 32) .. +7
//   B operand: lane l holds column (l % 32), contraction slots 8*(l / 32) .. +7
//   D/C      : lane l holds column (l % 32); register i holds row 8*(i / 4) + 4*(l / 32) + (i % 4)
__device__ __forceinline__ f32x16 mfma32_bf16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                 0, 0, 0);
}
#ifndef COROPE_F16
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) { return mfma32_bf16(a, b, c); }
#endif

// The same tile shape with fp16 operands (11 significant bits instead of 8).
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
__device__ __forceinline__ f32x16 mfma32_f16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
// Two floats -> packed fp16 (lo in bits 0..15), round to nearest even (v_cvt_pk_f16_f32).
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, f16x2));
}

#ifdef COROPE_F16
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) { return mfma32_f16(a, b, c); }
#endif

// D(16x16) += A(16x32) * B(32x16): half the matrix-pipe time of the 32x32x16 form, for products that need few rows.
//   A operand: lane l holds row (l % 16), contraction slots 8*(l / 16) .. +7
//   B operand: lane l holds column (l % 16), contraction slots 8*(l / 16) .. +7
//   D/C      : lane l holds column (l % 16); register i holds row 4*(l / 16) + i
__device__ __forceinline__ f32x4 mfma16_f16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
#ifdef COROPE_F16
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) { return mfma16_f16(a, b, c); }
#else
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
#endif

// ---- the element type of the attention kernels: two elements per 32-bit word, element 0 in the low half -------------
#ifdef COROPE_F16
__device__ __forceinline__ float elt_lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
__device__ __forceinline__ float elt_hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
__device__ __forceinline__ uint32_t pack_elts(float lo, float hi) { return pack_f16(lo, hi); }
#else
__device__ __forceinline__ float elt_lo(uint32_t w) { return bf16_lo(w); }
__device__ __forceinline__ float elt_hi(uint32_t w) { return bf16_hi(w); }
__device__ __forceinline__ uint32_t pack_elts(float lo, float hi) { return pack_bf16(lo, hi); }
#endif

// D = A * B + C with D in registers of its own (C stays intact): the form the score products start from, C holding minus
// the reference value of the exponentials in every register.  Written as an asm statement because the compiler, given
// the builtin, copies C into D first.  The only readers of D that may follow are further mfma32 that accumulate into it
// (same registers as C and D: no wait states needed) -- the vector units must not touch D before one of those has run, and the
// compiler, to which this statement is opaque, inserts no wait states behind it: the build checks the generated assembly
// of every kernel for that (check_isa.py).
__device__ __forceinline__ f32x16 mfma32_from(u32x4 a, u32x4 b, const f32x16& c) {
  f32x16 d;
#ifdef COROPE_F16
  asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
#else
  asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
#endif
  return d;
}

// With one wave per SIMD (head dim 256) the compiler gives every MFMA it selects its accumulator in the accumulation half
// of the register file, and a product whose result the vector units read next (scores, dP) then costs a copy per element
// each way.  The same products as asm statements with every operand in the vector half: mfma32_zero_v starts a chain from
// zero, mfma32_acc_v accumulates in place, and mfma32_settle behind the last of a chain waits the 12 states after which the
// vector units may touch the result (the compiler inserts none behind an asm statement; check_isa.py verifies).
__device__ __forceinline__ f32x16 mfma32_zero_v(u32x4 a, u32x4 b) {
  f32x16 d;
#ifdef COROPE_F16
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
#else
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
#endif
  return d;
}
__device__ __forceinline__ void mfma32_acc_v(f32x16& d, u32x4 a, u32x4 b) {
#ifdef COROPE_F16
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
#else
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
#endif
}
// ... and with the B operand in the accumulation half (where a wave's per-item operand rows live when it has 512 registers):
// Score products with the query operand in the accumulation half of the register file (the matrix cores read A and B
// operands from either half; the vector units only the other one, which the scores, probabilities and staging fill).
// As asm statements: the compiler, given the builtin, copies such an operand over before every use.  `from`: the result
// lands in registers of its own, C stays intact; `acc`: accumulates in place.  The compiler inserts no wait states behind
// an asm statement: the first vector instruction that reads the scores follows at least two further MFMAs (or one and
// an explicit s_nop) behind the last of these, which the build checks in the generated assembly (check_isa.py).
// mfma32_zero_aq starts a chain from zero.
__device__ __forceinline__ f32x16 mfma32_from_aq(u32x4 a, const u32x4& b, const f32x16& c) {
  f32x16 d;
#ifdef COROPE_F16
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "a"(b), "v"(c));
#else
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "a"(b), "v"(c));
#endif
  return d;
}
__device__ __forceinline__ void mfma32_acc_aq(f32x16& d, u32x4 a, const u32x4& b) {
#ifdef COROPE_F16
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
#else
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
#endif
}
__device__ __forceinline__ f32x16 mfma32_zero_aq(u32x4 a, const u32x4& b) {
  f32x16 d;
#ifdef COROPE_F16
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
#else
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
#endif
  return d;
}

__device__ __forceinline__ void mfma32_settle(f32x16& d) { asm volatile("s_nop 7\n\ts_nop 3" : "+v"(d)); }

// Row index (0..31) held by accumulator register i of lane-half h in a 32x32 MFMA result.
__device__ __forceinline__ constexpr int acc_row(int i, int h) { return 8 * (i / 4) + 4 * h + (i % 4); }

// ---- exchange between the two 32-lane halves of a wave ---------------------------------------------
__device__ __forceinline__ float half_max(float x) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float half_sum(float x) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---- addressing ------------------------------------------------------------------------------------
// base + a 32-bit unsigned byte offset.  With a wave-uniform base this is the "scalar base + 32-bit vector offset"
// form of the global load, which needs one address register per lane instead of two and no 64-bit arithmetic.
// Callers guarantee that one (batch, head) slice and the cos/sin tables stay below 4 GiB.
template <typename T>
__device__ __forceinline__ const T* byte_offset(const T* base, uint32_t bytes) {
  return reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + bytes);
}
template <typename T>
__device__ __forceinline__ T* byte_offset(T* base, uint32_t bytes) {
  return reinterpret_cast<T*>(reinterpret_cast<char*>(base) + bytes);
}

// Grouped-query attention: slab (batch, query head) -> slab (batch, key/value head) of tensors with Hkv heads.
__device__ __forceinline__ int kv_slab(int bh, int H, int Hkv) {
  return H == Hkv ? bh : (bh / H) * Hkv + (bh % H) / (H / Hkv);
}

// Waves per SIMD the attention kernels are built for: two up to D = 128 (256 registers per lane each); at D = 256 the
// operand rows and accumulators of a wave need more than that, so one wave per SIMD, with 512.
template <int D>
constexpr int kWavesPerSimd = D > 128 ? 1 : 2;

// ---- LDS tile layouts -----------------------------------------------------------------------------
// Row-major tile [rows][D] of bf16 with PAD elements of padding per row.
//   PAD = 8  (16 bytes): 16 consecutive rows read at the same column with 16-byte reads land in 16 different
//                        bank groups -- the layout for tiles read row-wise as MFMA operands;
//   PAD = 32 (64 bytes): the row stride is 16 dwords past a multiple of 64, so the 4 rows x 32 bytes a 16-lane
//                        block touches in a transposing read (and the 8 rows of a whole wave) spread over all
//                        banks -- the layout for tiles read only through load_a_trans;
//   PAD = kStaggerPad:   for tiles read both ways: 64 bytes of padding as with PAD = 32, and every fourth row another 16
//                        bytes.  Row r then starts 4 * r + r / 4 sixteen-byte groups past a multiple of 16 groups: 16
//                        consecutive rows sit in 16 different groups (row-wise reads), and the 4 rows x 64 bytes that
//                        two 16-lane blocks of a transposing read touch still cover every bank once.  The extra 16 bytes
//                        per 4 rows are the same for rows 4 apart in lane terms (lane part + compile-time constant).
constexpr int kStaggerPad = 9;
template <int D, int PAD = 8>
struct RowTile {
  static constexpr bool kStaggered = PAD == kStaggerPad;
  static constexpr int kStride = D + (kStaggered ? 32 : PAD);  // elements
  static constexpr int bytes(int rows) { return (rows * kStride + (kStaggered ? 8 * ((rows + 3) / 4) : 0)) * 2; }
  __device__ static __forceinline__ int stagger(int row) { return kStaggered ? 8 * (row >> 2) : 0; }
  __device__ static __forceinline__ int off(int row, int col) { return row * kStride + stagger(row) + col; }
};

// ---- staging: a ROWS x D tile with the half-layout rotation applied on the way -----------------------
// Work unit = one row x 8 rotation pairs: columns [8c, 8c+8) and [D/2 + 8c, D/2 + 8c + 8) of the same row
// are loaded by the same thread, so the rotation is thread-local.  cos/sin come from fp32 tables of which
// only the first D/2 columns are used.  SCALED: the rotated values are multiplied by out_scale before the one rounding
// (the query side of QK^T carries sm_scale * log2(e), so that scores leave the matrix cores in base-2 units).
template <int D, int ROWS, int NT, bool SCALED = false, int PAD = 8>
struct RotStage {
  static constexpr int kChunks = D / 16;              // units per row
  static constexpr int kUnits = ROWS * kChunks;
  static constexpr int kIters = (kUnits + NT - 1) / NT;
  u32x4 x1[kIters], x2[kIters];
  f32x4 c[kIters][2], s[kIters][2];
  float out_scale = 1.f;

  // src: first row of the (n, D) bf16 matrix; row0: first tile row; rows >= n_rows are clamped.
  // row_bytes: bytes between rows of src (D * 2 for a contiguous matrix)
  __device__ __forceinline__ void load(const uint16_t* __restrict__ src, const float* __restrict__ cosp,
                                       const float* __restrict__ sinp, int64_t fstride, int row0, int n_rows,
                                       uint32_t row_bytes = D * 2) {
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      int u = threadIdx.x + it * NT;
      if (kUnits % NT != 0 && u >= kUnits) u = kUnits - 1;
      int r = u / kChunks, ch = u % kChunks;
      int row = min(row0 + r, n_rows - 1);
      const uint16_t* p = byte_offset(src, (uint32_t)row * row_bytes + ch * 16);
      x1[it] = *reinterpret_cast<const u32x4*>(p);
      x2[it] = *reinterpret_cast<const u32x4*>(p + D / 2);
      const uint32_t foff = ((uint32_t)row * (uint32_t)fstride + ch * 8) * 4;
      const float* cp = byte_offset(cosp, foff);
      const float* sp = byte_offset(sinp, foff);
      c[it][0] = *reinterpret_cast<const f32x4*>(cp);
      c[it][1] = *reinterpret_cast<const f32x4*>(cp + 4);
      s[it][0] = *reinterpret_cast<const f32x4*>(sp);
      s[it][1] = *reinterpret_cast<const f32x4*>(sp + 4);
    }
  }

  // Rotates unit `it`: y1 = x1 c - x2 s, y2 = x2 c + x1 s (fp32), rounds to bf16.
  __device__ __forceinline__ void rotate(int it, u32x4& y1, u32x4& y2) const {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float a0 = elt_lo(x1[it][w]), a1 = elt_hi(x1[it][w]);
      float b0 = elt_lo(x2[it][w]), b1 = elt_hi(x2[it][w]);
      float c0 = c[it][w / 2][(2 * w) % 4], c1 = c[it][w / 2][(2 * w) % 4 + 1];
      float s0 = s[it][w / 2][(2 * w) % 4], s1 = s[it][w / 2][(2 * w) % 4 + 1];
      if constexpr (SCALED) {
        y1[w] = pack_elts((a0 * c0 - b0 * s0) * out_scale, (a1 * c1 - b1 * s1) * out_scale);
        y2[w] = pack_elts((b0 * c0 + a0 * s0) * out_scale, (b1 * c1 + a1 * s1) * out_scale);
      } else {
        y1[w] = pack_elts(a0 * c0 - b0 * s0, a1 * c1 - b1 * s1);
        y2[w] = pack_elts(b0 * c0 + a0 * s0, b1 * c1 + a1 * s1);
      }
    }
  }

  // Row-major store of the rotated tile.
  __device__ __forceinline__ void store_rows(uint16_t* lds) const {
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      int u = threadIdx.x + it * NT;
      if (kUnits % NT != 0 && u >= kUnits) continue;
      int r = u / kChunks, ch = u % kChunks;
      u32x4 y1, y2;
      rotate(it, y1, y2);
      *reinterpret_cast<u32x4*>(lds + RowTile<D, PAD>::off(r, ch * 8)) = y1;
      *reinterpret_cast<u32x4*>(lds + RowTile<D, PAD>::off(r, D / 2 + ch * 8)) = y2;
    }
  }
};

// ---- staging: a ROWS x D tile copied row-major (no rotation) -------------------------------------------
template <int D, int ROWS, int NT, int PAD = 8>
struct CopyStage {
  static constexpr int kChunks = D / 8;  // 16-byte units per row
  static constexpr int kUnits = ROWS * kChunks;
  static constexpr int kIters = (kUnits + NT - 1) / NT;
  u32x4 x[kIters];

  __device__ __forceinline__ void load(const uint16_t* __restrict__ src, int row0, int n_rows, uint32_t row_bytes = D * 2) {
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      int u = threadIdx.x + it * NT;
      if (kUnits % NT != 0 && u >= kUnits) u = kUnits - 1;
      int row = min(row0 + u / kChunks, n_rows - 1);
      x[it] = *reinterpret_cast<const u32x4*>(byte_offset(src, (uint32_t)row * row_bytes + (u % kChunks) * 16));
    }
  }
  __device__ __forceinline__ void store_rows(uint16_t* lds) const {
#pragma unroll
    for (int it = 0; it < kIters; ++it) {
      int u = threadIdx.x + it * NT;
      if (kUnits % NT != 0 && u >= kUnits) continue;
      *reinterpret_cast<u32x4*>(lds + RowTile<D, PAD>::off(u / kChunks, (u % kChunks) * 8)) = x[it];
    }
  }
};

// Staging of a tile whose rows take part in QK^T: rotated on the way to LDS (PREROT = false), or copied from a tensor
// that rope_rotate_kernel rotated beforehand (PREROT = true; the tables are then not touched).
template <int D, int ROWS, int NT, bool PREROT, bool SCALED = false, int PAD = 8>
struct RopeStage : RotStage<D, ROWS, NT, SCALED, PAD> {};
template <int D, int ROWS, int NT, bool SCALED, int PAD>
struct RopeStage<D, ROWS, NT, true, SCALED, PAD> : CopyStage<D, ROWS, NT, PAD> {
  float out_scale = 1.f;   // unused: the copy was scaled when it was rotated
  __device__ __forceinline__ void load(const uint16_t* __restrict__ src, const float*, const float*, int64_t, int row0,
                                       int n_rows, uint32_t row_bytes = D * 2) {
    CopyStage<D, ROWS, NT, PAD>::load(src, row0, n_rows, row_bytes);
  }
};

// ---- transposing LDS read (ds_read_b64_tr_b16) ------------------------------------------------------------
// The instruction works on blocks of 16 lanes: source lane s supplies 8 bytes E[s][0..3]; result lane L
// receives { E[4j + L/4][L % 4] : j = 0..3 }.
//
// load_a_trans builds the A operand of mfma32 (32 rows m x 16 contraction slots) from a ROW-MAJOR tile
// T[k][m] whose rows are the contraction index, i.e. it reads the tile transposed.  The contraction slots
// follow the order in which a 32x32 accumulator hands out its rows when it is re-used as a B operand:
//   slot j of lane-half h  <->  k = kbase + 8*(j / 4) + 4*h + (j % 4).
typedef __attribute__((ext_vector_type(4))) short s16x4;
__device__ __forceinline__ u32x4 load_a_trans(const uint16_t* tile, int stride, int kbase, int m0) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  const int l = threadIdx.x % kWave;
  const int blk = l / 16, s = l % 16, h = blk / 2;
  const uint16_t* p = tile + (kbase + 4 * h + s / 4) * stride + m0 + 16 * (blk % 2) + 4 * (s % 4);
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * stride));
  u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a[0], a[1], b[0], b[1]};
}

// The same read from a tile of layout T (a RowTile); kbase: a multiple of 4.
template <typename T>
__device__ __forceinline__ u32x4 load_a_trans_of(const uint16_t* tile, int kbase, int m0) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  const int l = threadIdx.x % kWave;
  const int blk = l / 16, s = l % 16, h = blk / 2;
  // rows kbase + 4h + s/4 and, 8 further, the second half
  const uint16_t* p = tile + T::off(kbase, 0) + T::off(4 * h + s / 4, m0 + 16 * (blk % 2) + 4 * (s % 4));
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + T::off(8, 0)));
  u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a[0], a[1], b[0], b[1]};
}

// The same read with the address split into its per-lane part and the rest: a_trans_lane_offset(stride) elements are
// added to the tile once (per lane), load_a_trans_at then needs only compile-time offsets on top of that pointer.
__device__ __forceinline__ int a_trans_lane_offset(int stride) {
  const int l = threadIdx.x % kWave;
  const int blk = l / 16, s = l % 16, h = blk / 2;
  return (4 * h + s / 4) * stride + 16 * (blk % 2) + 4 * (s % 4);
}
__device__ __forceinline__ u32x4 load_a_trans_at(const uint16_t* lane_tile, int stride, int kbase, int m0) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  const uint16_t* p = lane_tile + kbase * stride + m0;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * stride));
  u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a[0], a[1], b[0], b[1]};
}

// Loads 32 rows x D of a (rows, D) bf16 matrix as the B operand chunks of mfma32 (lane = row, 8 columns per
// chunk and lane-half), optionally applying the half-layout rotation first.  KC = D / 16 chunks.
template <int D, bool ROTATE>
__device__ __forceinline__ void load_b_rows(u32x4 (&out)[D / 16], const uint16_t* __restrict__ src,
                                            const float* __restrict__ cosp, const float* __restrict__ sinp,
                                            int64_t fstride, int row) {
  constexpr int KC = D / 16;
  const int lh = (threadIdx.x % kWave) / 32;
  const uint16_t* xp = src + (int64_t)row * D + 8 * lh;
  if constexpr (!ROTATE) {
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) out[kc] = *reinterpret_cast<const u32x4*>(xp + 16 * kc);
  } else {
    const float* cp = cosp + (int64_t)row * fstride + 8 * lh;
    const float* sp = sinp + (int64_t)row * fstride + 8 * lh;
#pragma unroll
    for (int kc = 0; kc < KC / 2; ++kc) {
      u32x4 x1 = *reinterpret_cast<const u32x4*>(xp + 16 * kc);
      u32x4 x2 = *reinterpret_cast<const u32x4*>(xp + D / 2 + 16 * kc);
      f32x4 c[2] = {*reinterpret_cast<const f32x4*>(cp + 16 * kc), *reinterpret_cast<const f32x4*>(cp + 16 * kc + 4)};
      f32x4 s[2] = {*reinterpret_cast<const f32x4*>(sp + 16 * kc), *reinterpret_cast<const f32x4*>(sp + 16 * kc + 4)};
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float a0 = elt_lo(x1[w]), a1 = elt_hi(x1[w]), b0 = elt_lo(x2[w]), b1 = elt_hi(x2[w]);
        float c0 = c[w / 2][(2 * w) % 4], c1 = c[w / 2][(2 * w) % 4 + 1];
        float s0 = s[w / 2][(2 * w) % 4], s1 = s[w / 2][(2 * w) % 4 + 1];
        out[kc][w] = pack_elts(a0 * c0 - b0 * s0, a1 * c1 - b1 * s1);
        out[kc + KC / 2][w] = pack_elts(b0 * c0 + a0 * s0, b1 * c1 + a1 * s1);
      }
    }
  }
}

// A wave's LDS instructions execute in program order, so LDS bytes that only this wave touches can be written and read
// back by it without a barrier or a wait; all that is needed is that the compiler keeps the accesses in program order.
// (A workgroup barrier would also wait for the global loads issued ahead of time.)
__device__ __forceinline__ void lds_order() { asm volatile("" ::: "memory"); }

// ---- a wave's 32 rows through LDS: coalesced global accesses on one side, lane = row on the other ---------------------
// The MFMA layouts make a lane own a row (a query or a key), so loading B operands or storing transposed accumulators
// straight from / to global memory touches 32 different rows per instruction, 16 or 32 bytes of each.  These helpers go
// through a wave-private LDS tile instead: global memory sees whole 128- or 256-byte row segments per instruction.  A wave's
// LDS instructions execute in program order, so no barrier is needed between the two halves of a helper; the caller only
// has to make sure that no other wave uses the same LDS bytes at the same time.

// B operand chunks (as load_b_rows) of rows row0 .. row0 + 31 of a (n_rows, D) bf16 matrix, rows clamped to n_rows - 1,
// in two steps so that a kernel can issue all its prologue loads before it waits for any of them: load() starts the
// global loads, park() writes the rows (ROTATE: after the half-layout rotation, fp32, one rounding) into the wave's LDS
// tile and reads them back as B operands; rot_out (may be null) receives the rotated rows that lie inside the matrix.
// wave_tile: 32 * RowTile<D>::kStride elements of LDS.
template <int D, bool ROTATE>
struct WaveRows;

template <int D>
struct WaveRows<D, false> {
  static constexpr int CPR = D / 8;            // 16-byte chunks per row
  static constexpr int RPI = kWave / CPR;      // rows per load instruction
  static constexpr int IT = 32 / RPI;
  u32x4 x[IT];
  __device__ __forceinline__ void load(const uint16_t* __restrict__ src, const float*, const float*, int64_t, int row0,
                                       int n_rows, int l = threadIdx.x % kWave, uint32_t row_bytes = D * 2) {
#pragma unroll
    for (int i = 0; i < IT; ++i)
      x[i] = *reinterpret_cast<const u32x4*>(
          byte_offset(src, (uint32_t)min(row0 + RPI * i + l / CPR, n_rows - 1) * row_bytes + (l % CPR) * 16));
  }
  __device__ __forceinline__ void park(u32x4 (&out)[D / 16], uint16_t* wave_tile, uint16_t* = nullptr, int = 0, int = 0,
                                       float = 1.f) {
    const int l = threadIdx.x % kWave;
    lds_order();
#pragma unroll
    for (int i = 0; i < IT; ++i)
      *reinterpret_cast<u32x4*>(wave_tile + RowTile<D>::off(RPI * i + l / CPR, (l % CPR) * 8)) = x[i];
    lds_order();
#pragma unroll
    for (int kc = 0; kc < D / 16; ++kc)
      out[kc] = *reinterpret_cast<const u32x4*>(wave_tile + RowTile<D>::off(l % 32, 16 * kc + 8 * (l / 32)));
    lds_order();
  }
};

template <int D>
struct WaveRows<D, true> {
  static constexpr int UPR = D / 16;           // units (8 rotation pairs) per row
  static constexpr int RPI = kWave / UPR;
  static constexpr int IT = 32 / RPI;
  u32x4 x1[IT], x2[IT];
  f32x4 c[IT][2], s[IT][2];
  // l: the lane (callers inside a loop over work items pass a value the optimiser cannot see through, so that the
  // per-lane address parts are recomputed per item instead of being kept in registers across the whole loop)
  __device__ __forceinline__ void load(const uint16_t* __restrict__ src, const float* __restrict__ cosp,
                                       const float* __restrict__ sinp, int64_t fstride, int row0, int n_rows,
                                       int l = threadIdx.x % kWave, uint32_t row_bytes = D * 2) {
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      const int row = min(row0 + RPI * i + l / UPR, n_rows - 1), u = l % UPR;
      const uint16_t* xp = byte_offset(src, (uint32_t)row * row_bytes + u * 16);
      x1[i] = *reinterpret_cast<const u32x4*>(xp);
      x2[i] = *reinterpret_cast<const u32x4*>(xp + D / 2);
      const uint32_t foff = ((uint32_t)row * (uint32_t)fstride + u * 8) * 4;
      const float* cp = byte_offset(cosp, foff);
      const float* sp = byte_offset(sinp, foff);
      c[i][0] = *reinterpret_cast<const f32x4*>(cp);
      c[i][1] = *reinterpret_cast<const f32x4*>(cp + 4);
      s[i][0] = *reinterpret_cast<const f32x4*>(sp);
      s[i][1] = *reinterpret_cast<const f32x4*>(sp + 4);
    }
  }
  __device__ __forceinline__ void park(u32x4 (&out)[D / 16], uint16_t* wave_tile, uint16_t* __restrict__ rot_out = nullptr,
                                       int row0 = 0, int n_rows = 0, float out_scale = 1.f) {
    const int l = threadIdx.x % kWave;
    lds_order();
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      const int r = RPI * i + l / UPR, u = l % UPR;
      u32x4 y1, y2;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float a0 = elt_lo(x1[i][w]), a1 = elt_hi(x1[i][w]), b0 = elt_lo(x2[i][w]), b1 = elt_hi(x2[i][w]);
        float c0 = c[i][w / 2][(2 * w) % 4], c1 = c[i][w / 2][(2 * w) % 4 + 1];
        float s0 = s[i][w / 2][(2 * w) % 4], s1 = s[i][w / 2][(2 * w) % 4 + 1];
        y1[w] = pack_elts((a0 * c0 - b0 * s0) * out_scale, (a1 * c1 - b1 * s1) * out_scale);
        y2[w] = pack_elts((b0 * c0 + a0 * s0) * out_scale, (b1 * c1 + a1 * s1) * out_scale);
      }
      *reinterpret_cast<u32x4*>(wave_tile + RowTile<D>::off(r, u * 8)) = y1;
      *reinterpret_cast<u32x4*>(wave_tile + RowTile<D>::off(r, D / 2 + u * 8)) = y2;
      if (rot_out != nullptr && row0 + r < n_rows) {
        uint16_t* dst = byte_offset(rot_out, (uint32_t)(row0 + r) * (D * 2) + u * 16);
        *reinterpret_cast<u32x4*>(dst) = y1;
        *reinterpret_cast<u32x4*>(dst + D / 2) = y2;
      }
    }
    lds_order();
#pragma unroll
    for (int kc = 0; kc < D / 16; ++kc)
      out[kc] = *reinterpret_cast<const u32x4*>(wave_tile + RowTile<D>::off(l % 32, 16 * kc + 8 * (l / 32)));
    lds_order();
  }
};

// ---- a wave's private 32 x D tile of 16-bit elements without row padding ---------------------------------------------
// 16-byte chunk c of row r is kept at chunk c ^ swz(r) of the row: sixteen consecutive rows read at one chunk index (the
// B-operand read, lane = row) then touch sixteen different bank groups, and so do the chunks of one row.  8 KB at D = 128.
template <int D>
struct WaveTile {
  static constexpr int CPR = D / 8;                      // 16-byte chunks per row
  static constexpr int RP = 16 / CPR > 0 ? 16 / CPR : 1;  // rows per 256 bytes
  static constexpr int kBytes = 32 * D * 2;
  __device__ static __forceinline__ int swz(int r) { return (r / RP) & (CPR - 1); }
  __device__ static __forceinline__ int off(int r, int c) { return r * (D * 2) + ((c ^ swz(r)) << 4); }   // bytes
};

// WaveRows<D, true>::load's rows, rotated, scaled and rounded, through a WaveTile: rot_out (may be null) receives the rows
// that lie inside the matrix, `out` the B operand chunks.
template <int D>
__device__ __forceinline__ void park_rotated_rows(const WaveRows<D, true>& w, u32x4 (&out)[D / 16], uint8_t* tile,
                                                  uint16_t* __restrict__ rot_out, int row0, int n_rows, float out_scale,
                                                  int l = threadIdx.x % kWave) {
  using WR = WaveRows<D, true>;
  using T = WaveTile<D>;
  lds_order();
#pragma unroll
  for (int i = 0; i < WR::IT; ++i) {
    const int r = WR::RPI * i + l / WR::UPR, u = l % WR::UPR;
    u32x4 y1, y2;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float a0 = elt_lo(w.x1[i][k]), a1 = elt_hi(w.x1[i][k]), b0 = elt_lo(w.x2[i][k]), b1 = elt_hi(w.x2[i][k]);
      float c0 = w.c[i][k / 2][(2 * k) % 4], c1 = w.c[i][k / 2][(2 * k) % 4 + 1];
      float s0 = w.s[i][k / 2][(2 * k) % 4], s1 = w.s[i][k / 2][(2 * k) % 4 + 1];
      y1[k] = pack_elts((a0 * c0 - b0 * s0) * out_scale, (a1 * c1 - b1 * s1) * out_scale);
      y2[k] = pack_elts((b0 * c0 + a0 * s0) * out_scale, (b1 * c1 + a1 * s1) * out_scale);
    }
    *reinterpret_cast<u32x4*>(tile + T::off(r, u)) = y1;
    *reinterpret_cast<u32x4*>(tile + T::off(r, u + T::CPR / 2)) = y2;
    if (rot_out != nullptr && row0 + r < n_rows) {
      uint16_t* dst = byte_offset(rot_out, (uint32_t)(row0 + r) * (D * 2) + u * 16);
      *reinterpret_cast<u32x4*>(dst) = y1;
      *reinterpret_cast<u32x4*>(dst + D / 2) = y2;
    }
  }
  lds_order();
#pragma unroll
  for (int kc = 0; kc < D / 16; ++kc) out[kc] = *reinterpret_cast<const u32x4*>(tile + T::off(l % 32, 2 * kc + l / 32));
  lds_order();
}

// WaveRows<D, false>::load's rows through a WaveTile, as B operand chunks.
template <int D>
__device__ __forceinline__ void park_plain_rows(const WaveRows<D, false>& w, u32x4 (&out)[D / 16], uint8_t* tile,
                                                int l = threadIdx.x % kWave) {
  using WR = WaveRows<D, false>;
  using T = WaveTile<D>;
  lds_order();
#pragma unroll
  for (int i = 0; i < WR::IT; ++i) *reinterpret_cast<u32x4*>(tile + T::off(WR::RPI * i + l / WR::CPR, l % WR::CPR)) = w.x[i];
  lds_order();
#pragma unroll
  for (int kc = 0; kc < D / 16; ++kc) out[kc] = *reinterpret_cast<const u32x4*>(tile + T::off(l % 32, 2 * kc + l / 32));
  lds_order();
}
template <int D>
__device__ __forceinline__ void park_rows(const WaveRows<D, false>& w, u32x4 (&out)[D / 16], uint8_t* tile, float, int l) {
  park_plain_rows<D>(w, out, tile, l);
}
template <int D>
__device__ __forceinline__ void park_rows(const WaveRows<D, true>& w, u32x4 (&out)[D / 16], uint8_t* tile, float out_scale,
                                          int l) {
  park_rotated_rows<D>(w, out, tile, nullptr, 0, 0, out_scale, l);
}

// Persistent launches: one workgroup per compute unit (or per item, if those are fewer), every workgroup walking a list
// of items that is fixed by arithmetic.  Items are numbered heaviest first and dealt to the workgroups in rounds,
// forwards in even rounds and backwards in odd ones, so that the workgroups end up with equal work when the rounds are
// full and the weights fall linearly (causal attention).  Workgroup ids are dealt round-robin to the 8 XCDs and both
// directions keep id % 8: with the slab index running fastest in the item number (and slabs a multiple of 8), all items
// of a slab stay on one XCD and share its L2.
struct ItemList {
  int G, fwd, back;
  __device__ __forceinline__ ItemList() {
    G = gridDim.x;
    fwd = blockIdx.x;
    back = (G % 8 == 0) ? (G - 8 - (fwd & ~7)) + (fwd & 7) : G - 1 - fwd;
  }
  __device__ __forceinline__ int at(int round) const { return round * G + ((round & 1) ? back : fwd); }
};

// Rows row0 .. row0 + 31 of a (n_rows, D) matrix of 16-bit elements from transposed fp32 accumulators (layout as for
// store_rows_via_lds below), every value multiplied by `scale` (per lane = per row), one rounding, through a WaveTile:
// 16-byte stores that cover whole rows.
template <int D>
__device__ __forceinline__ void store_rows_via_wave_tile(const f32x16 (&acc)[D / 32], uint16_t* __restrict__ dst, int row0,
                                                         int n_rows, float scale, uint8_t* tile,
                                                         int l = threadIdx.x % kWave) {
  using T = WaveTile<D>;
  const int lq = l % 32, lh = l / 32;
  lds_order();
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<u32x2*>(tile + T::off(lq, db * 4 + g) + 8 * lh) =
          u32x2{pack_elts(acc[db][4 * g] * scale, acc[db][4 * g + 1] * scale),
                pack_elts(acc[db][4 * g + 2] * scale, acc[db][4 * g + 3] * scale)};
  lds_order();
  constexpr int RPI = kWave / T::CPR;
#pragma unroll
  for (int i = 0; i < 32 / RPI; ++i) {
    const int r = RPI * i + l / T::CPR, c = l % T::CPR, row = row0 + r;
    const u32x4 x = *reinterpret_cast<const u32x4*>(tile + T::off(r, c));
    if (row < n_rows) *reinterpret_cast<u32x4*>(byte_offset(dst, (uint32_t)row * (D * 2) + c * 16)) = x;
  }
  lds_order();
}

// The same for accumulators of rotated rows (dQ_r, dK_r): the half-layout rotation is undone in fp32 before the one
// rounding, d1 = d1r c + d2r s, d2 = d2r c - d1r s.  A lane holds both partners of a pair (columns j and j + D/2 of its
// row), so this needs no exchange; its 2 x D/4 table values are read in 16-byte pieces, in a step of their own so that a
// kernel can request them ahead of other loads (loads return in the order they were issued).
template <int D>
struct UnrotateTables {
  static constexpr int NP = (D / 64) * 4;   // 16-byte pieces per table
  f32x4 c[NP], s[NP];
  __device__ __forceinline__ void load(const float* __restrict__ cosp, const float* __restrict__ sinp, int64_t fstride,
                                       int row0, int n_rows, int l = threadIdx.x % kWave) {
    const uint32_t frow = (uint32_t)min(row0 + l % 32, n_rows - 1) * (uint32_t)fstride;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const uint32_t foff = (frow + (i / 4) * 32 + 8 * (i % 4) + 4 * (l / 32)) * 4;
      c[i] = *reinterpret_cast<const f32x4*>(byte_offset(cosp, foff));
      s[i] = *reinterpret_cast<const f32x4*>(byte_offset(sinp, foff));
    }
  }
};
template <int D>
__device__ __forceinline__ void store_unrotated_rows_via_wave_tile(const f32x16 (&acc)[D / 32], const UnrotateTables<D>& tb,
                                                                   uint16_t* __restrict__ dst, int row0, int n_rows,
                                                                   float scale, uint8_t* tile, int l = threadIdx.x % kWave) {
  using T = WaveTile<D>;
  constexpr int NH = D / 64;   // 32-column blocks per half
  const int lq = l % 32, lh = l / 32;
  lds_order();
#pragma unroll
  for (int db = 0; db < NH; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 c = tb.c[db * 4 + g], s = tb.s[db * 4 + g];
      float o1[4], o2[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float r1 = acc[db][4 * g + e] * scale, r2 = acc[db + NH][4 * g + e] * scale;
        o1[e] = r1 * c[e] + r2 * s[e];
        o2[e] = r2 * c[e] - r1 * s[e];
      }
      *reinterpret_cast<u32x2*>(tile + T::off(lq, db * 4 + g) + 8 * lh) = u32x2{pack_elts(o1[0], o1[1]), pack_elts(o1[2], o1[3])};
      *reinterpret_cast<u32x2*>(tile + T::off(lq, (db + NH) * 4 + g) + 8 * lh) = u32x2{pack_elts(o2[0], o2[1]), pack_elts(o2[2], o2[3])};
    }
  lds_order();
  constexpr int RPI = kWave / T::CPR;
#pragma unroll
  for (int i = 0; i < 32 / RPI; ++i) {
    const int r = RPI * i + l / T::CPR, c = l % T::CPR, row = row0 + r;
    const u32x4 x = *reinterpret_cast<const u32x4*>(tile + T::off(r, c));
    if (row < n_rows) *reinterpret_cast<u32x4*>(byte_offset(dst, (uint32_t)row * (D * 2) + c * 16)) = x;
  }
  lds_order();
}

// Rows row0 .. row0 + 31 of a (n_rows, D) bf16 matrix from transposed fp32 accumulators (lane = row l % 32, acc[db][i] =
// column db*32 + 8*(i/4) + 4*(l/32) + i%4): every value is multiplied by `scale` (which may
// differ from lane to lane, i.e. from row to row), UNROTATE undoes the half-layout rotation in fp32 (d1 = d1r c + d2r s,
// d2 = d2r c - d1r s), one rounding to bf16, 16-byte stores that cover whole 128-byte row segments.
// wave_tile: 32 * kAccTileStride<D> floats of LDS.
template <int D>
constexpr int kAccTileStride = D + 4;
template <int D, bool UNROTATE>
__device__ __forceinline__ void store_rows_via_lds(const f32x16 (&acc)[D / 32], uint16_t* __restrict__ dst, int row0,
                                                   int n_rows, const float* __restrict__ cosp,
                                                   const float* __restrict__ sinp, int64_t fstride, float scale,
                                                   float* wave_tile) {
  constexpr int LS = kAccTileStride<D>;
  const int l = threadIdx.x % kWave, lq = l % 32, lh = l / 32;
  lds_order();
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<f32x4*>(wave_tile + lq * LS + db * 32 + 8 * g + 4 * lh) =
          f32x4{acc[db][4 * g] * scale, acc[db][4 * g + 1] * scale, acc[db][4 * g + 2] * scale, acc[db][4 * g + 3] * scale};
  lds_order();
  constexpr int UPR = D / 16, RPI = kWave / UPR;
#pragma unroll
  for (int i = 0; i < 32 / RPI; ++i) {
    const int r = RPI * i + l / UPR, u = l % UPR, row = row0 + r;
    const float* t = wave_tile + r * LS + u * 8;
    f32x4 a[2] = {*reinterpret_cast<const f32x4*>(t), *reinterpret_cast<const f32x4*>(t + 4)};
    f32x4 b[2] = {*reinterpret_cast<const f32x4*>(t + D / 2), *reinterpret_cast<const f32x4*>(t + D / 2 + 4)};
    if (row < n_rows) {
      float o1[8], o2[8];
      if constexpr (UNROTATE) {
        const uint32_t foff = ((uint32_t)row * (uint32_t)fstride + u * 8) * 4;
        const float* cp = byte_offset(cosp, foff);
        const float* sp = byte_offset(sinp, foff);
        f32x4 c[2] = {*reinterpret_cast<const f32x4*>(cp), *reinterpret_cast<const f32x4*>(cp + 4)};
        f32x4 s[2] = {*reinterpret_cast<const f32x4*>(sp), *reinterpret_cast<const f32x4*>(sp + 4)};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float r1 = a[e / 4][e % 4], r2 = b[e / 4][e % 4], ce = c[e / 4][e % 4], se = s[e / 4][e % 4];
          o1[e] = r1 * ce + r2 * se;
          o2[e] = r2 * ce - r1 * se;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          o1[e] = a[e / 4][e % 4];
          o2[e] = b[e / 4][e % 4];
        }
      }
      uint16_t* d = byte_offset(dst, (uint32_t)row * (D * 2) + u * 16);
      *reinterpret_cast<u32x4*>(d) = u32x4{pack_elts(o1[0], o1[1]), pack_elts(o1[2], o1[3]), pack_elts(o1[4], o1[5]), pack_elts(o1[6], o1[7])};
      *reinterpret_cast<u32x4*>(d + D / 2) = u32x4{pack_elts(o2[0], o2[1]), pack_elts(o2[2], o2[3]), pack_elts(o2[4], o2[5]), pack_elts(o2[6], o2[7])};
    }
  }
  lds_order();
}

// A operand of mfma16 (16 rows m x 32 contraction slots) read transposed from a row-major tile T[k][m]: lane l gets
// T[kbase + 8*(l / 16) + j][m0 + l % 16] for slots j = 0..7 (two transposing reads of 4 contraction rows each).
__device__ __forceinline__ u32x4 load_a_trans16(const uint16_t* tile, int stride, int kbase, int m0) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  const int l = threadIdx.x % kWave;
  const int g = l / 16, s = l % 16;
  const uint16_t* p = tile + (kbase + 8 * g + s / 4) * stride + m0 + 4 * (s % 4);
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * stride));
  u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a[0], a[1], b[0], b[1]};
}

// Natural-order variant of load_a_trans: slot j of lane-half h <-> k = kbase + 8*h + j.
__device__ __forceinline__ u32x4 load_a_trans_natural(const uint16_t* tile, int stride, int kbase, int m0) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  const int l = threadIdx.x % kWave;
  const int blk = l / 16, s = l % 16, h = blk / 2;
  const uint16_t* p = tile + (kbase + 8 * h + s / 4) * stride + m0 + 16 * (blk % 2) + 4 * (s % 4);
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * stride));
  u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
  return u32x4{a[0], a[1], b[0], b[1]};
}

// ---- wave-wide reductions and scans ---------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m);
  return x;
}
// Wave-wide scan and maximum with data-parallel-primitive moves (no LDS round trips): shifts by 1, 2, 4, 8 inside each
// row of 16 lanes, then lane 15 of rows 0 and 2 is broadcast into rows 1 and 3, then lane 31 into rows 2 and 3.  Lanes
// without a source take `identity`.  All 64 lanes must be active.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float identity, float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity), __builtin_bit_cast(int, x),
                                                               CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_prefix_sum(float x) {   // inclusive: lane l gets the sum over lanes 0..l
  x += dpp_move<0x111, 0xf>(0.f, x);
  x += dpp_move<0x112, 0xf>(0.f, x);
  x += dpp_move<0x114, 0xf>(0.f, x);
  x += dpp_move<0x118, 0xf>(0.f, x);
  x += dpp_move<0x142, 0xa>(0.f, x);
  x += dpp_move<0x143, 0xc>(0.f, x);
  return x;
}
// Sum over each row of 16 lanes, in every lane of the row (rotations within the row: no LDS round trips).
__device__ __forceinline__ float row16_sum(float x) {
  x += dpp_move<0x128, 0xf>(0.f, x);   // row_ror:8
  x += dpp_move<0x124, 0xf>(0.f, x);   // row_ror:4
  x += dpp_move<0x122, 0xf>(0.f, x);   // row_ror:2
  x += dpp_move<0x121, 0xf>(0.f, x);   // row_ror:1
  return x;
}
__device__ __forceinline__ float wave_last(float x) {          // lane 63's value, wave-uniform
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), kWave - 1));
}
__device__ __forceinline__ float wave_max(float x) {
  x = fmaxf(x, dpp_move<0x111, 0xf>(-INFINITY, x));
  x = fmaxf(x, dpp_move<0x112, 0xf>(-INFINITY, x));
  x = fmaxf(x, dpp_move<0x114, 0xf>(-INFINITY, x));
  x = fmaxf(x, dpp_move<0x118, 0xf>(-INFINITY, x));
  x = fmaxf(x, dpp_move<0x142, 0xa>(-INFINITY, x));
  x = fmaxf(x, dpp_move<0x143, 0xc>(-INFINITY, x));
  return wave_last(x);
}

__device__ __forceinline__ float bf16_to_f(uint16_t x) { return __builtin_bit_cast(float, (uint32_t)x << 16); }
__device__ __forceinline__ uint16_t f_to_bf16(float x) { return (uint16_t)(pack_bf16(x, 0.f) & 0xffffu); }
__device__ __forceinline__ uint16_t f_to_f16(float x) { return (uint16_t)(pack_f16(x, 0.f) & 0xffffu); }
__device__ __forceinline__ uint16_t f_to_elt(float x) { return (uint16_t)(pack_elts(x, 0.f) & 0xffffu); }
__device__ __forceinline__ float elt_to_f(uint16_t x) { return elt_lo((uint32_t)x); }

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>): a loop whose index is a compile-time constant
// in the body, so register arrays indexed with it never look dynamically indexed to the optimiser.
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

}  // namespace COROPE_NS
