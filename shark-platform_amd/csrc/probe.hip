// Matrix-core ceiling probe: a launch of nothing but independent MFMA instructions on operands held in registers
// (no memory traffic inside the loop).  A measurement aid for roofline statements: the chip lowers its clock with the
// matrix cores' activity, and how far depends on the operand bits, so the rate a real kernel can reach is the rate of
// this loop on similar data, not the data-sheet figure.
#include "stmoe_common.h"

namespace stmoe {

typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef int probe_int8 __attribute__((ext_vector_type(8)));
typedef float probe_float4 __attribute__((ext_vector_type(4)));
typedef float probe_float16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 15;
  x *= 2246822519u;
  x ^= x >> 13;
  x *= 3266489917u;
  x ^= x >> 16;
  return x;
}

// KIND 0: v_mfma_f32_16x16x32_f16 (8 accumulator tiles per wavefront), KIND 1: v_mfma_scale_f32_32x32x64_f8f6f4 on e4m3
// bytes (4 tiles).  Operands: random_operands == 0: every dword 0x11111111; otherwise hashed bits (fp16: random sign and
// mantissa, exponent of 0.5..1; fp8: random bytes with the top exponent bit cleared, so no NaN).
template <int KIND>
__global__ void __launch_bounds__(512) probe_mfma_kernel(int iters, int random_operands, float* sink) {
  const uint32_t t = blockIdx.x * 512 + threadIdx.x;
  union {
    probe_half8 h;
    probe_int8 i8;
    uint32_t u[8];
  } a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const uint32_t ra = random_operands ? probe_hash(t * 64 + j * 8 + q) : 0x11111111u;
      const uint32_t rb = random_operands ? probe_hash(t * 64 + 32 + j * 8 + q + 7777) : 0x11111111u;
      if (KIND == 0) {
        a[j].u[q] = (ra & 0x83ff83ffu) | 0x38003800u;
        b[j].u[q] = (rb & 0x83ff83ffu) | 0x38003800u;
      } else {
        a[j].u[q] = ra & 0xbfbfbfbfu;
        b[j].u[q] = rb & 0xbfbfbfbfu;
      }
    }
  float r = 0.f;
  if (KIND == 0) {
    probe_float4 c[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = (probe_float4){0.f, 0.f, 0.f, 0.f};
    for (int it0 = 0; it0 < iters; it0 += 4)
#pragma unroll
      for (int it = 0; it < 4; ++it)
#pragma unroll
        for (int j = 0; j < 8; ++j) c[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j & 3].h, b[(j + it) & 3].h, c[j], 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 8; ++j) r += c[j][0] + c[j][3];
  } else {
    probe_float16 c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) c[j][q] = 0.f;
    for (int it0 = 0; it0 < iters; it0 += 4)
#pragma unroll
      for (int it = 0; it < 4; ++it)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          c[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[j & 3].i8, b[(j + it) & 3].i8, c[j], 0, 0, 0, 127, 0, 127);
#pragma unroll
    for (int j = 0; j < 4; ++j) r += c[j][0] + c[j][15];
  }
  if (r == 123.456f) sink[0] = r;  // keeps the loop alive; practically never true
}

}  // namespace stmoe

extern "C" int stmoe_probe_mfma(int kind, int random_operands, int iters, float* sink, double* flop, stmoe_stream_t stream) {
  using namespace stmoe;
  if (!sink) return set_error(STMOE_ERR_NULL, "probe_mfma: sink is NULL");
  if (kind < 0 || kind > 1 || iters <= 0 || iters % 4 != 0)
    return set_error(STMOE_ERR_SHAPE, "probe_mfma: kind 0 (fp16) or 1 (fp8), iters a positive multiple of 4");
  // 256 workgroups of 8 wavefronts: two wavefronts per SIMD on every CU; per wavefront and iteration 8 x 16x16x32 or
  // 4 x 32x32x64 products
  const double per_wave_iter = kind == 0 ? 8.0 * 2 * 16 * 16 * 32 : 4.0 * 2 * 32 * 32 * 64;
  if (flop) *flop = per_wave_iter * iters * 8 * 256;
  hipStream_t st = as_stream(stream);
  if (kind == 0) probe_mfma_kernel<0><<<256, 512, 0, st>>>(iters, random_operands, sink);
  else probe_mfma_kernel<1><<<256, 512, 0, st>>>(iters, random_operands, sink);
  return check_launch("probe_mfma");
}
