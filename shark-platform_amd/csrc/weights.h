// Weight-format accessors: turn 16 consecutive reduction elements of one weight row into values of the
// activation type T, with the roundings of the reference's dequantize-then-cast
// (`unbox_tensor` -> layout.dequant() -> `.to(lhs.dtype)`, sharktank/sharktank/ops/default_impls.py:345-351):
//   Q8_0   w = T( f16(d * q) )                  sharktank/sharktank/types/layouts.py:274-290
//   Q4_1   w = T( f16( f16(d * q) + m ) )       layouts.py:302-357, layout_utils.py:67-86
//   FP8    w = T( DD( DD(q) * d ) ), DD = dtype of d   layouts.py:163-181
//   DENSE  w = T( element )
#pragma once
#include "stmoe_common.h"

namespace stmoe {

struct WeightView {
  const uint8_t* qs;
  const uint8_t* d;
  const uint8_t* m;
  int64_t rows;     // per expert
  int64_t cols;     // reduction length
  int64_t d_count;  // FP8: number of scales (1 or experts)
  int32_t dtype;    // DENSE element dtype / FP8 scale dtype
  int32_t experts;
};

static inline WeightView make_view(const stmoe_weight* w) {
  WeightView v;
  v.qs = (const uint8_t*)w->qs;
  v.d = (const uint8_t*)w->d;
  v.m = (const uint8_t*)w->m;
  v.rows = w->rows;
  v.cols = w->cols;
  v.d_count = w->d_count;
  v.dtype = w->dtype;
  v.experts = (int32_t)w->experts;
  return v;
}

// Formats as compile-time tags.  Dense weights are split by element type.
enum : int { WF_Q8_0 = 0, WF_Q4_1 = 1, WF_FP8_F32D = 2, WF_FP8_F16D = 3, WF_DENSE_F32 = 4, WF_DENSE_F16 = 5, WF_DENSE_BF16 = 6,
             // the same formats in the packed streaming order written by stmoe_prepack
             WF_Q8_0_P = 7, WF_Q4_1_P = 8, WF_FP8_F32D_P = 9 };

template <int WF> struct IsQ8 { static constexpr bool value = WF == WF_Q8_0 || WF == WF_Q8_0_P; };
template <int WF> struct IsQ4 { static constexpr bool value = WF == WF_Q4_1 || WF == WF_Q4_1_P; };

// pack two fp32 values, already rounded to T, into one dword of T bits
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float lo, float hi) {
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  const f16x2_t v = {(f16_t)lo, (f16_t)hi};  // a vector, so that both halves are written in place (no shift-and-or packing)
  return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float lo, float hi) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const bf16x2_t v = {(__bf16)lo, (__bf16)hi};  // one v_cvt_pk_bf16_f32 (round to nearest even)
  return __builtin_bit_cast(uint32_t, v);
}

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// Eight products a[i] * d, each rounded to fp32 and then to T, packed into four dwords.  For fp16 the mixed-precision
// fused multiply-add writes each half of a result dword in place (fp32 arithmetic, then the conversion): one instruction
// per element instead of a multiply per element and a packed conversion per pair.  These instructions write half a
// register, and on this ISA a read of such a register needs one wait state after the write; the compiler's hazard
// handling cannot see into inline assembly, so the sequence is ordered to keep every dependent pair at least three
// instructions apart and ends with an s_nop of two wait states, which covers the half-register read hazard and the
// wait a matrix-core instruction needs after a vector write of one of its operands.
template <typename T> __device__ __forceinline__ void scale8_pack(const float (&a)[8], float d, uint32_t (&out)[4]) {
  if constexpr (__is_same(T, f16_t)) {
    asm("v_fma_mixlo_f16 %0, %4, %12, 0\n\t"
        "v_fma_mixlo_f16 %1, %6, %12, 0\n\t"
        "v_fma_mixlo_f16 %2, %8, %12, 0\n\t"
        "v_fma_mixlo_f16 %3, %10, %12, 0\n\t"
        "v_fma_mixhi_f16 %0, %5, %12, 0\n\t"
        "v_fma_mixhi_f16 %1, %7, %12, 0\n\t"
        "v_fma_mixhi_f16 %2, %9, %12, 0\n\t"
        "v_fma_mixhi_f16 %3, %11, %12, 0\n\t"
        "s_nop 1"
        : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3])
        : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]), "v"(d));
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = pack2<T>(__fmul_rn(a[2 * i], d), __fmul_rn(a[2 * i + 1], d));
  }
}

__device__ __forceinline__ half2_t as_half2(uint32_t u) {
  union { uint32_t u; half2_t h; } c;
  c.u = u;
  return c.h;
}
__device__ __forceinline__ uint32_t as_u32(half2_t h) {
  union { uint32_t u; half2_t h; } c;
  c.h = h;
  return c.u;
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  union { uint16_t u; f16_t h; } c;
  c.u = (uint16_t)b;
  return (float)c.h;
}

// ---- Q4_1 helpers ------------------------------------------------------------------------------------
// f16(f16(d*q) + m) for a pair of nibbles given as fp16 numbers 1024 + q (bits 0x6400 | q): the subtraction is exact,
// the product of an fp16 scale and an integer below 16 rounds once like the reference's multiply, then the add.
__device__ __forceinline__ uint32_t q4_pair_dequant(uint32_t pair_bits, uint32_t dbits, uint32_t mbits) {
  const half2_t dd = as_half2(dbits | (dbits << 16)), mm = as_half2(mbits | (mbits << 16));
  const half2_t bias = {(f16_t)1024.0f, (f16_t)1024.0f};
  return as_u32((as_half2(pair_bits) - bias) * dd + mm);
}
// Pair p (elements 2p, 2p+1) of the 8 nibbles of a dword, as two fp16 numbers 1024 + q.
//   linear order (planar planes): element i is nibble i
//   packed order (written by stmoe_prepack): even elements in the low half-word, odd ones in the high half-word
//   (element 2p at bits 4p, element 2p+1 at bits 16 + 4p), so one shift and one and-or extract a pair
__device__ __forceinline__ uint32_t q4_pair_linear(uint32_t w, int p) {
  const uint32_t byte = w >> (8 * p);
  return 0x64006400u | (byte & 0xfu) | ((byte & 0xf0u) << 12);
}
__device__ __forceinline__ uint32_t q4_pair_packed(uint32_t w, int p) { return ((w >> (4 * p)) & 0x000f000fu) | 0x64006400u; }
// The four pairs of a packed dword, dequantised, with fewer operations than four q4_pair_dequant calls.  The nibbles at
// bits 0-3 and 4-7 of each half-word become the fp16 numbers 1024 + q and 64 + q by one and-or each (the nibble lands
// in the mantissa of 0x6400 / 0x5400); the other two pairs come the same way from the dword shifted right by 8.  One
// fused multiply-add per pair removes the bias and applies the scale: (bias + q) * d - bias * d is the exact product
// q * d rounded once, like the reference's multiply (bias * d is exact; it stays finite for |d| < 64, far beyond any
// block scale of fp16-range weights), and one add applies m: the reference's two roundings.
struct Q4Scale {
  half2_t dd, mm, c1024, c64;
};
__device__ __forceinline__ Q4Scale q4_scale(uint32_t dbits, uint32_t mbits) {
  Q4Scale s;
  s.dd = as_half2(dbits | (dbits << 16));
  s.mm = as_half2(mbits | (mbits << 16));
  const half2_t n1024 = {(f16_t)-1024.0f, (f16_t)-1024.0f}, n64 = {(f16_t)-64.0f, (f16_t)-64.0f};
  s.c1024 = s.dd * n1024;
  s.c64 = s.dd * n64;
  return s;
}
// (a & mask) | magic in one instruction; written out because the compiler splits it into an and and an or when both
// constants are literals (a VOP3 instruction of this ISA cannot take two of them; here they sit in registers)
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(mask), "v"(magic));
  return r;
}
__device__ __forceinline__ void q4_dword_dequant_packed(uint32_t w, const Q4Scale& s, uint32_t out[4]) {
  const uint32_t w8 = w >> 8;
  const uint32_t p0 = and_or(w, 0x000f000fu, 0x64006400u), p1 = and_or(w, 0x00f000f0u, 0x54005400u);
  const uint32_t p2 = and_or(w8, 0x000f000fu, 0x64006400u), p3 = and_or(w8, 0x00f000f0u, 0x54005400u);
  out[0] = as_u32(__builtin_elementwise_fma(as_half2(p0), s.dd, s.c1024) + s.mm);
  out[1] = as_u32(__builtin_elementwise_fma(as_half2(p1), s.dd, s.c64) + s.mm);
  out[2] = as_u32(__builtin_elementwise_fma(as_half2(p2), s.dd, s.c1024) + s.mm);
  out[3] = as_u32(__builtin_elementwise_fma(as_half2(p3), s.dd, s.c64) + s.mm);
}
__device__ __forceinline__ uint32_t q4_dword_to_packed(uint32_t w) {
  uint32_t out = 0;
#pragma unroll
  for (int p = 0; p < 4; ++p) out |= (((w >> (8 * p)) & 0xfu) << (4 * p)) | (((w >> (8 * p + 4)) & 0xfu) << (16 + 4 * p));
  return out;
}
__device__ __forceinline__ uint32_t q4_dword_to_linear(uint32_t w) {
  uint32_t out = 0;
#pragma unroll
  for (int p = 0; p < 4; ++p) out |= (((w >> (4 * p)) & 0xfu) << (8 * p)) | (((w >> (16 + 4 * p)) & 0xfu) << (8 * p + 4));
  return out;
}

// Raw bytes of a 16-element chunk and its conversion.  `load` only issues the global loads (so a caller
// can keep a chunk in flight across a compute phase); `to_f32` produces the 16 values as fp32 numbers
// equal to the dequantised weight in the layout dtype (the caller rounds to T).
template <int WF> struct Chunk16;

template <> struct Chunk16<WF_Q8_0> {
  uint4 q;
  uint16_t dbits;
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const int64_t row = e * w.rows + n;
    q = *reinterpret_cast<const uint4*>(w.qs + row * w.cols + k0);
    dbits = reinterpret_cast<const uint16_t*>(w.d)[row * (w.cols >> 5) + (k0 >> 5)];
  }
  __device__ __forceinline__ void zero() { q = make_uint4(0, 0, 0, 0); dbits = 0; }
  // 16 fp16 values as 8 dwords: (q + 1152) built by byte permutation as 0x6400|u8, minus 1152, times d.
  // Products of an fp16 scale and an integer of magnitude <= 128 are exact in the multiplier, so the
  // single rounding of the fp16 multiply equals the reference's f16(d * q).
  __device__ __forceinline__ void to_f16x16(uint32_t out[8]) const {
    const uint32_t r[4] = {q.x, q.y, q.z, q.w};
    const half2_t bias = {(f16_t)1152.0f, (f16_t)1152.0f};
    union { uint16_t u; f16_t h; } dc;
    dc.u = dbits;
    const half2_t dd = {dc.h, dc.h};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = r[i] ^ 0x80808080u;
      const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
      const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
      out[2 * i] = as_u32((as_half2(lo) - bias) * dd);
      out[2 * i + 1] = as_u32((as_half2(hi) - bias) * dd);
    }
  }
  __device__ __forceinline__ void to_f32(float out[16]) const {
    uint32_t h[8];
    to_f16x16(h);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      out[2 * i] = f16_bits_to_f32(h[i] & 0xffffu);
      out[2 * i + 1] = f16_bits_to_f32(h[i] >> 16);
    }
  }
};

template <> struct Chunk16<WF_Q4_1> {
  uint2 q;
  uint16_t dbits, mbits;
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const int64_t row = e * w.rows + n;
    q = *reinterpret_cast<const uint2*>(w.qs + ((row * w.cols + k0) >> 1));
    const int64_t b = row * (w.cols >> 5) + (k0 >> 5);
    dbits = reinterpret_cast<const uint16_t*>(w.d)[b];
    mbits = reinterpret_cast<const uint16_t*>(w.m)[b];
  }
  __device__ __forceinline__ void zero() { q = make_uint2(0, 0); dbits = 0; mbits = 0; }
  // element 2i = low nibble of byte i, element 2i+1 = high nibble.  f16(f16(d*q) + m): two roundings.
  template <bool PACKED = false> __device__ __forceinline__ void decode(uint32_t out[8]) const {
    const uint32_t r[2] = {q.x, q.y};
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        out[4 * i + b] = q4_pair_dequant(PACKED ? q4_pair_packed(r[i], b) : q4_pair_linear(r[i], b), dbits, mbits);
  }
  __device__ __forceinline__ void to_f16x16(uint32_t out[8]) const { decode<false>(out); }
  __device__ __forceinline__ void to_f32(float out[16]) const {
    uint32_t h[8];
    to_f16x16(h);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      out[2 * i] = f16_bits_to_f32(h[i] & 0xffffu);
      out[2 * i + 1] = f16_bits_to_f32(h[i] >> 16);
    }
  }
};

template <bool F16D> struct Chunk16Fp8 {
  uint4 q;
  float dv;
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const int64_t row = e * w.rows + n;
    q = *reinterpret_cast<const uint4*>(w.qs + row * w.cols + k0);
    const int64_t j = w.d_count > 1 ? e : 0;
    dv = F16D ? (float)reinterpret_cast<const f16_t*>(w.d)[j] : reinterpret_cast<const float*>(w.d)[j];
  }
  __device__ __forceinline__ void zero() { q = make_uint4(0, 0, 0, 0); dv = 0.0f; }
  __device__ __forceinline__ void to_f32(float out[16]) const {
    const uint32_t r[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v[4];
      fp8x4_to_f32(r[j], v);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __fmul_rn(v[i], dv);
        out[4 * j + i] = F16D ? round_to<f16_t>(p) : p;
      }
    }
  }
};
template <> struct Chunk16<WF_FP8_F32D> : Chunk16Fp8<false> {};
template <> struct Chunk16<WF_FP8_F16D> : Chunk16Fp8<true> {};

// Packed streaming order (see prepack.hip): only the addresses differ from the planar accessors.
__device__ __forceinline__ int64_t packed_piece(int64_t row, int64_t k0, int64_t cols, int kshift) {
  // byte offset of the 16-byte piece holding (row, k0) when one piece covers 1 << (kshift - 2) reduction elements
  // of one row and one 1 KB block covers 1 << kshift of them: kshift = 6 for 1-byte samples, 7 for nibbles
  const int64_t rt = row >> 4, kb = k0 >> kshift;
  const int g = (int)(k0 >> (kshift - 2)) & 3;
  return ((rt * (cols >> kshift) + kb) * 64 + g * 16 + (row & 15)) << 4;
}
__device__ __forceinline__ int64_t packed_scale(int64_t row, int64_t k0, int64_t cols) {
  return (((row >> 4) * (cols >> 8) + (k0 >> 8)) * 16 + (row & 15)) * 8 + ((k0 >> 5) & 7);
}
template <> struct Chunk16<WF_Q8_0_P> : Chunk16<WF_Q8_0> {
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const int64_t row = e * w.rows + n;
    q = *reinterpret_cast<const uint4*>(w.qs + packed_piece(row, k0, w.cols, 6));
    dbits = reinterpret_cast<const uint16_t*>(w.d)[packed_scale(row, k0, w.cols)];
  }
};
template <> struct Chunk16<WF_Q4_1_P> : Chunk16<WF_Q4_1> {
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const int64_t row = e * w.rows + n;
    q = *reinterpret_cast<const uint2*>(w.qs + packed_piece(row, k0, w.cols, 7) + ((k0 >> 4) & 1) * 8);
    const int64_t b = packed_scale(row, k0, w.cols);
    dbits = reinterpret_cast<const uint16_t*>(w.d)[b];
    mbits = reinterpret_cast<const uint16_t*>(w.m)[b];
  }
  __device__ __forceinline__ void to_f16x16(uint32_t out[8]) const { decode<true>(out); }
  __device__ __forceinline__ void to_f32(float out[16]) const {
    uint32_t h[8];
    decode<true>(h);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      out[2 * i] = f16_bits_to_f32(h[i] & 0xffffu);
      out[2 * i + 1] = f16_bits_to_f32(h[i] >> 16);
    }
  }
};
template <> struct Chunk16<WF_FP8_F32D_P> : Chunk16Fp8<false> {
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const int64_t row = e * w.rows + n;
    q = *reinterpret_cast<const uint4*>(w.qs + packed_piece(row, k0, w.cols, 6));
    dv = reinterpret_cast<const float*>(w.d)[w.d_count > 1 ? e : 0];
  }
};

template <> struct Chunk16<WF_DENSE_F32> {
  float4 v[4];
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(w.qs) + (e * w.rows + n) * w.cols + k0);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = p[i];
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = make_float4(0, 0, 0, 0);
  }
  __device__ __forceinline__ void to_f32(float out[16]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[4 * i] = v[i].x; out[4 * i + 1] = v[i].y; out[4 * i + 2] = v[i].z; out[4 * i + 3] = v[i].w;
    }
  }
};

template <bool BF> struct Chunk16Dense16 {
  uint32_t r[8];
  __device__ __forceinline__ void load(const WeightView& w, int64_t e, int64_t n, int64_t k0) {
    const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(w.qs) + (e * w.rows + n) * w.cols + k0);
    const uint4 a = p[0], b = p[1];
    r[0] = a.x; r[1] = a.y; r[2] = a.z; r[3] = a.w;
    r[4] = b.x; r[5] = b.y; r[6] = b.z; r[7] = b.w;
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = 0;
  }
  __device__ __forceinline__ void to_f32(float out[16]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (BF) {
        out[2 * i] = __uint_as_float(r[i] << 16);
        out[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
      } else {
        out[2 * i] = f16_bits_to_f32(r[i] & 0xffffu);
        out[2 * i + 1] = f16_bits_to_f32(r[i] >> 16);
      }
    }
  }
  __device__ __forceinline__ void raw(uint32_t out[8]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = r[i];
  }
};
template <> struct Chunk16<WF_DENSE_F16> : Chunk16Dense16<false> {};
template <> struct Chunk16<WF_DENSE_BF16> : Chunk16Dense16<true> {};

// 16 values of T as 8 dwords, ready for LDS / MFMA operands.
template <typename T, int WF>
__device__ __forceinline__ void chunk_to_T(const Chunk16<WF>& c, uint32_t out[8]) {
  if constexpr (IsQ8<WF>::value || IsQ4<WF>::value) {
    if constexpr (__is_same(T, f16_t)) {
      c.to_f16x16(out);
      return;
    }
  }
  if constexpr ((WF == WF_DENSE_F16 && __is_same(T, f16_t)) || (WF == WF_DENSE_BF16 && __is_same(T, bf16_t))) {
    c.raw(out);
    return;
  }
  float f[16];
  c.to_f32(f);
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = pack2<T>(f[2 * i], f[2 * i + 1]);
}

// Host-side: compile-time tag of a weight descriptor, or -1.
static inline int weight_tag(const stmoe_weight* w) {
  switch (w->format) {
    case STMOE_W_Q8_0: return WF_Q8_0;
    case STMOE_W_Q4_1: return WF_Q4_1;
    case STMOE_W_FP8: return w->dtype == STMOE_F32 ? WF_FP8_F32D : (w->dtype == STMOE_F16 ? WF_FP8_F16D : -1);
    case STMOE_W_Q8_0_PACKED: return WF_Q8_0_P;
    case STMOE_W_Q4_1_PACKED: return WF_Q4_1_P;
    case STMOE_W_FP8_PACKED: return w->dtype == STMOE_F32 ? WF_FP8_F32D_P : -1;
    case STMOE_W_DENSE:
      return w->dtype == STMOE_F32 ? WF_DENSE_F32 : (w->dtype == STMOE_F16 ? WF_DENSE_F16 : (w->dtype == STMOE_BF16 ? WF_DENSE_BF16 : -1));
    default: return -1;
  }
}

}  // namespace stmoe
