// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/sharktank_moe_hip.h"

namespace stmoe {

// ---- status plumbing --------------------------------------------------------------------------
int set_error(int code, const char* fmt, ...);
int check_launch(const char* what);
int norm_router(const void* h, int dtype, const void* norm_w, int w_dtype, float eps, void* xn, const void* wr,
                int64_t T_tokens, int64_t K, int E, int k, int32_t* idx, void* gate, hipStream_t st,
                int32_t* counts = nullptr, int32_t* offsets = nullptr, int32_t* perm = nullptr, int32_t* inv = nullptr,
                const float* x_fq = nullptr);

// stmoe_dispatch_build that also clears `n_zero` (at most 1024) 32-bit words at `zero_words` (nullable).
int dispatch_build(const int32_t* idx, int64_t n_pairs, int E, int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* inv,
                   int32_t* zero_words, int n_zero, hipStream_t st);

int quantize_fp8_gather(const void* x, int dtype, const float* rscale, const int32_t* perm, int k, int64_t rows, int64_t K, void* out,
                        int64_t block_rows, hipStream_t st);

#define STMOE_REQUIRE(cond, code, ...)            \
  do {                                            \
    if (!(cond)) return ::stmoe::set_error((code), __VA_ARGS__); \
  } while (0)

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline hipStream_t as_stream(stmoe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
static inline int dtype_size(int dt) {
  switch (dt) {
    case STMOE_F32: return 4;
    case STMOE_F16: case STMOE_BF16: return 2;
    case STMOE_F8E4M3FN: case STMOE_I8: case STMOE_U8: return 1;
    default: return 0;
  }
}

// ---- 16-bit float types as raw bits -------------------------------------------------------------
// bf16 is handled as a 16-bit pattern with explicit round-to-nearest-even conversions so that every
// rounding point is spelled out; fp16 uses the native _Float16 type.
typedef _Float16 f16_t;
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  // v_cvt_pk_bf16_f32: round to nearest even, NaN stays a quiet NaN
  bf16_t r;
  r.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
  return r;
}

template <typename T> struct Cvt;
template <> struct Cvt<float> {
  static __device__ __forceinline__ float to_f32(float v) { return v; }
  static __device__ __forceinline__ float from_f32(float v) { return v; }
};
template <> struct Cvt<f16_t> {
  static __device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
  static __device__ __forceinline__ f16_t from_f32(float v) { return (f16_t)v; }
};
template <> struct Cvt<bf16_t> {
  static __device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }
  static __device__ __forceinline__ bf16_t from_f32(float v) { return f32_to_bf16(v); }
};

// Forces an fp32 value into a register as is.  Without it the compiler may fuse an fp32 multiply with the following
// conversion to fp16 into one mixed-precision instruction (v_fma_mix*), which rounds the exact product once; eager
// torch rounds the product to fp32 first and then to fp16, and the two differ about once in 2^13 values.
__device__ __forceinline__ float keep_f32(float v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Round an fp32 value to T and widen it again: the value a tensor of dtype T would hold.
template <typename T> __device__ __forceinline__ float round_to(float v) {
  return Cvt<T>::to_f32(Cvt<T>::from_f32(v));
}

// ---- fp8 e4m3fn (OCP) ---------------------------------------------------------------------------
// gfx950 converts OCP e4m3fn in hardware (v_cvt_f32_fp8 / v_cvt_pk_f32_fp8); every e4m3fn value is exact in fp32.
__device__ __forceinline__ float fp8_e4m3fn_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_f32_fp8((int)b, 0); }
// the four samples of one dword, lowest byte first
__device__ __forceinline__ void fp8x4_to_f32(uint32_t u, float out[4]) {
  typedef float float2_t __attribute__((ext_vector_type(2)));
  const float2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)u, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)u, true);
  out[0] = lo[0]; out[1] = lo[1]; out[2] = hi[0]; out[3] = hi[1];
}

// Round-to-nearest-even fp32 -> e4m3fn; magnitudes above 448 that round past it become NaN (0x7f),
// as torch's cast does; callers that want saturation clamp first.
__device__ __forceinline__ uint8_t f32_to_fp8_e4m3fn(float f) {
  uint32_t u = __float_as_uint(f);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  u &= 0x7fffffffu;
  if (u > 0x7f800000u) return sign | 0x7f;       // NaN
  if (u >= 0x43f00000u) return sign | 0x7f;      // >= 480 rounds beyond 448 -> NaN; (464 handled below)
  if (u < 0x3c800000u) {                         // < 2^-6: subnormal result, step 2^-9
    float a = __uint_as_float(u);
    // a * 512 rounded to nearest even integer in [0, 8]
    float r = rintf(a * 512.0f);
    return sign | (uint8_t)r;                    // r == 8 gives 0x08 = 2^-6, the smallest normal: correct
  }
  // normal: keep 3 mantissa bits
  uint32_t rounded = u + 0x7ffffu + ((u >> 20) & 1u);
  uint32_t e = (rounded >> 23) - 120u;
  uint32_t mnt = (rounded >> 20) & 0x7u;
  uint32_t enc = (e << 3) | mnt;
  if (enc > 0x7eu) return sign | 0x7f;           // rounded above 448
  return sign | (uint8_t)enc;
}

// quantize(x).unpack().dequant() of a static per-tensor e4m3fn quantizer (StaticScaledQuantizer,
// sharktank/sharktank/types/quantizers.py:153-183; applied by LinearLayer, sharktank/sharktank/layers/linear.py:72-78) for
// values of T given widened to fp32: T(f32(e4m3fn(clamp(T(x / rs)))) * rs).  The one definition of that arithmetic: the
// stand-alone pass and the kernels that apply it to a value they have just computed share it.
//   * x / rs, correctly rounded in fp32, comes from the correctly rounded reciprocal of rs (one division per kernel, kept
//     in FakeQuant) and one residual step per value: q0 = x * inv, q = fma(fma(-q0, rs, x), inv, q0);
//   * the e4m3fn rounding and its inverse are the hardware conversions (OCP e4m3fn, round to nearest even; the operand is
//     clamped to +-448 first, NaN stays NaN).
// Both are pinned by a test that runs every fp16 and every bf16 value through the stand-alone pass with many scales and
// compares with eager torch on the host.
struct FakeQuant {
  float rs, inv;  // reciprocal scale of the quantizer (0: no quantizer) and its correctly rounded reciprocal
  __device__ __forceinline__ explicit FakeQuant(const float* rscale) {
    rs = rscale ? *rscale : 0.0f;
    inv = rscale ? __fdiv_rn(1.0f, rs) : 0.0f;
  }
  __device__ __forceinline__ bool on() const { return rs != 0.0f; }
  template <typename T> __device__ __forceinline__ float clamped_quotient(float x) const {
    const float q0 = __fmul_rn(x, inv);
    // (an infinite quotient stays as it is: the residual step would turn it into NaN, where torch clamps it to +-448; so
    // does a zero: the residual step would lose the sign of -0)
    const float q1 = (fabsf(q0) == INFINITY || x == 0.0f) ? q0 : __builtin_fmaf(__builtin_fmaf(-q0, rs, x), inv, q0);
    const float q = round_to<T>(q1);
    // fminf / fmaxf drop a NaN operand; torch.clamp keeps it
    return q != q ? __uint_as_float(0x7fc00000u) : fminf(fmaxf(q, -448.0f), 448.0f);
  }
  // the e4m3fn samples of two values in the two low bytes
  template <typename T> __device__ __forceinline__ uint32_t quantize2(float a, float b) const {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(clamped_quotient<T>(a), clamped_quotient<T>(b), 0, false) & 0xffffu;
  }
  template <typename T> __device__ __forceinline__ void pair(float& a, float& b) const {
    const int bytes = __builtin_amdgcn_cvt_pk_fp8_f32(clamped_quotient<T>(a), clamped_quotient<T>(b), 0, false);
    a = round_to<T>(keep_f32(__fmul_rn(__builtin_amdgcn_cvt_f32_fp8(bytes, 0), rs)));
    b = round_to<T>(keep_f32(__fmul_rn(__builtin_amdgcn_cvt_f32_fp8(bytes, 1), rs)));
  }
  template <typename T> __device__ __forceinline__ float one(float a) const {
    float b = 0.0f;
    pair<T>(a, b);
    return a;
  }
};

// ---- activations ---------------------------------------------------------------------------------
__device__ __forceinline__ float act_silu(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float act_gelu_erf(float v) { return 0.5f * v * (1.0f + erff(v * 0.70710678118654752440f)); }
template <int ACT> __device__ __forceinline__ float apply_act(float v) {
  return ACT == STMOE_ACT_SILU ? act_silu(v) : act_gelu_erf(v);
}

// 1 / sqrt(total / K + eps) with every step (divide, add, square root, divide) correctly rounded in fp32, as IEEE
// host arithmetic gives it.  The fp32 square-root and divide instructions of the GPU are not correctly rounded, so
// the three operations are done in fp64 and rounded once to fp32 (innocuous double rounding: 53 >= 2*24 + 2 bits).
__device__ __forceinline__ float rms_scale(float total, int64_t K, float eps) {
  const float var = (float)((double)total / (double)K);
  const float ve = __fadd_rn(var, eps);
  const float s = (float)sqrt((double)ve);
  return (float)(1.0 / (double)s);
}

// ---- wavefront helpers -----------------------------------------------------------------------------
static constexpr int kWave = 64;

__device__ __forceinline__ float wave_xor_sum(float v) {
  // Fixed butterfly: partner distance 32, 16, 8, 4, 2, 1.  Each step adds a value and its partner's,
  // which is commutative, so every lane ends with the same bits.
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, kWave);
  return v;
}

}  // namespace stmoe
