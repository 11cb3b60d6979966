// Dequantization and quantization kernels.  Each restates one `dequant()` of the reference layouts
// with every rounding step in the same place, so results are bit-identical to the eager reference:
//   BlockScaledLayout      sharktank/sharktank/types/layouts.py:274-290
//   BlockScaledI4Layout    sharktank/sharktank/types/layouts.py:302-357, layout_utils.py:67-86
//   TensorScaledLayout     sharktank/sharktank/types/layouts.py:163-181
//   StaticScaledQuantizer  sharktank/sharktank/types/quantizers.py:153-183, layout_utils.py:150-176
// All arithmetic is spelled as fp32 operations on values that are exactly representable in the named
// 16-bit type followed by an explicit rounding, which is what eager torch does for half/bfloat16.
#include "stmoe_common.h"

namespace stmoe {

__device__ __forceinline__ float load_as_f32(const void* p, int dt, int64_t i) {
  switch (dt) {
    case STMOE_F32: return reinterpret_cast<const float*>(p)[i];
    case STMOE_F16: return (float)reinterpret_cast<const f16_t*>(p)[i];
    case STMOE_BF16: return bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
    case STMOE_F8E4M3FN: return fp8_e4m3fn_to_f32(reinterpret_cast<const uint8_t*>(p)[i]);
    case STMOE_I8: return (float)reinterpret_cast<const int8_t*>(p)[i];
    default: return (float)reinterpret_cast<const uint8_t*>(p)[i];
  }
}

// out[b*B + i] = D(D(d[b]) * D(q)) (+ D(m[b])), D = OUT.  I4: q is nibble i of the block's packed bytes.
template <typename OUT, bool I4>
__global__ void __launch_bounds__(256)
dequant_block_scaled_kernel(const void* __restrict__ d, const void* __restrict__ m, int dm_dtype,
                            const uint8_t* __restrict__ qs, int64_t n_elems, int block_size, int is_signed,
                            OUT* __restrict__ out) {
  // One thread handles 4 consecutive elements (block_size is a multiple of 4: checked on the host).
  const int64_t i0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i0 >= n_elems) return;
  const int64_t b = i0 / block_size;
  const float dv = round_to<OUT>(load_as_f32(d, dm_dtype, b));
  const float mv = m ? round_to<OUT>(load_as_f32(m, dm_dtype, b)) : 0.0f;
  float q[4];
  if (I4) {
    const uint8_t b0 = qs[i0 / 2], b1 = qs[i0 / 2 + 1];
    int v[4] = {b0 & 0xf, b0 >> 4, b1 & 0xf, b1 >> 4};
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = (float)((is_signed && v[j] >= 8) ? v[j] - 16 : v[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = (float)reinterpret_cast<const int8_t*>(qs)[i0 + j];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float r = round_to<OUT>(__fmul_rn(dv, q[j]));
    if (m) r = round_to<OUT>(__fadd_rn(r, mv));
    out[i0 + j] = Cvt<OUT>::from_f32(r);
  }
}

__global__ void __launch_bounds__(256)
promote_i4_kernel(const uint8_t* __restrict__ packed, int64_t n_bytes, int is_signed, uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_bytes) return;
  const uint8_t b = packed[i];
  int lo = b & 0xf, hi = b >> 4;
  if (is_signed) {
    lo = lo >= 8 ? lo - 16 : lo;
    hi = hi >= 8 ? hi - 16 : hi;
  }
  out[2 * i] = (uint8_t)lo;
  out[2 * i + 1] = (uint8_t)hi;
}

// out = OUT( DD( DD(DD(qs) - DD(m)) * d ) ), DD = dtype of d.
template <typename DD, typename OUT>
__global__ void __launch_bounds__(256)
dequant_tensor_scaled_kernel(const void* __restrict__ qs, int qs_dtype, const DD* __restrict__ d,
                             const DD* __restrict__ m, int64_t per_scale, int64_t d_count, int64_t n, OUT* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t j = (i / per_scale) % d_count;  // scale index along the scaled axis (axes before it repeat the scales)
  float q = round_to<DD>(load_as_f32(qs, qs_dtype, i));
  const float dv = Cvt<DD>::to_f32(d[j]);
  if (m) q = round_to<DD>(__fsub_rn(q, Cvt<DD>::to_f32(m[j])));
  const float r = round_to<DD>(__fmul_rn(q, dv));
  out[i] = Cvt<OUT>::from_f32(r);
}

template <typename T>
__global__ void __launch_bounds__(256)
quantize_fp8_kernel(const T* __restrict__ x, const float* __restrict__ rscale, int64_t n, uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  // eager torch divides in fp32 by the 0-dim fp32 scale and rounds the quotient to x's dtype (FakeQuant::clamped_quotient)
  out[i] = (uint8_t)FakeQuant(rscale).quantize2<T>(Cvt<T>::to_f32(x[i]), 0.0f);
}

// The same samples for rows gathered on the way: out row i = quantised row perm[i] / k of x (rows grouped by expert for the
// fp8 matrix-core kernel, which then reads its token rows without a gather).  One workgroup per row, 8 elements per thread.
template <typename T>
__global__ void __launch_bounds__(256)
quantize_fp8_gather_kernel(const T* __restrict__ x, const float* __restrict__ rscale, const int32_t* __restrict__ perm, int k,
                           int64_t K, uint8_t* __restrict__ out, int64_t block_rows) {
  const int64_t i = blockIdx.x;
  const int64_t src = perm ? perm[i] / k : i;
  const FakeQuant fq(rscale);
  for (int64_t c = (int64_t)threadIdx.x * 8; c < K; c += 256 * 8) {
    float v[8];
    if constexpr (sizeof(T) == 2) {
      const uint4 raw = *reinterpret_cast<const uint4*>(x + src * K + c);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = Cvt<T>::to_f32(__builtin_bit_cast(T, (uint16_t)(w[j] & 0xffffu)));
        v[2 * j + 1] = Cvt<T>::to_f32(__builtin_bit_cast(T, (uint16_t)(w[j] >> 16)));
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = Cvt<T>::to_f32(x[src * K + c + j]);
    }
    uint2 q;
    q.x = fq.quantize2<T>(v[0], v[1]) | (fq.quantize2<T>(v[2], v[3]) << 16);
    q.y = fq.quantize2<T>(v[4], v[5]) | (fq.quantize2<T>(v[6], v[7]) << 16);
    // block_rows > 0: blocks of 64 reduction samples, [K / 64][block_rows][64] (the layout the 256 x 256 fp8 kernel streams)
    const int64_t at = block_rows ? ((c >> 6) * block_rows + i) * 64 + (c & 63) : i * K + c;
    *reinterpret_cast<uint2*>(out + at) = q;
  }
}

// ---- dynamic per-tensor quantisation -------------------------------------------------------------------------
// Pass 1: every workgroup writes the maximum of |x| over its grid-stride share (NaN if it saw one, as torch.max does).
template <typename T>
__global__ void __launch_bounds__(256)
absmax_partial_kernel(const T* __restrict__ x, int64_t n, float* __restrict__ partial) {
  __shared__ float red[4];
  float m = 0.0f;
  bool nan = false;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float v = fabsf(Cvt<T>::to_f32(x[i]));
    nan |= v != v;
    m = fmaxf(m, v);
  }
  if (nan) m = __uint_as_float(0x7fc00000u);
  // max is exact and order-independent, so any reduction tree gives the same bits; NaN is carried by hand
  for (int off = 32; off; off >>= 1) {
    const float o = __shfl_xor(m, off);
    m = (m != m || o != o) ? __uint_as_float(0x7fc00000u) : fmaxf(m, o);
  }
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = red[0];
    for (int w = 1; w < 4; ++w) r = (r != r || red[w] != red[w]) ? __uint_as_float(0x7fc00000u) : fmaxf(r, red[w]);
    partial[blockIdx.x] = r;
  }
}
// Pass 2: every workgroup folds the partial maxima itself (a few KB from L2), derives the scale as eager torch does in
// x's dtype T -- scale = T(T(1 / max(amax, eps)) * 448), rscale = T(1 / scale), eps = finfo(float8_e4m3fn).eps = 0.125 -- and
// quantises its elements: e4m3fn(clamp(T(x * scale))).  (The reference writes `finfo.max / amax.clamp(eps)`, a Python
// number divided by a tensor, which torch evaluates as `tensor.reciprocal() * number`: two roundings in T, not one
// division.  amax = 4.8867 in fp16 gives 91.625 that way and 91.6875 as a quotient.)
template <typename T>
__global__ void __launch_bounds__(256)
dynamic_quantize_fp8_kernel(const T* __restrict__ x, int64_t n, const float* __restrict__ partial, int n_partial,
                            uint8_t* __restrict__ out, float* __restrict__ scale_rscale) {
  __shared__ float red[4];
  float m = 0.0f;
  for (int i = threadIdx.x; i < n_partial; i += 256) {
    const float o = partial[i];
    m = (m != m || o != o) ? __uint_as_float(0x7fc00000u) : fmaxf(m, o);
  }
  for (int off = 32; off; off >>= 1) {
    const float o = __shfl_xor(m, off);
    m = (m != m || o != o) ? __uint_as_float(0x7fc00000u) : fmaxf(m, o);
  }
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  float amax = red[0];
  for (int w = 1; w < 4; ++w) amax = (amax != amax || red[w] != red[w]) ? __uint_as_float(0x7fc00000u) : fmaxf(amax, red[w]);
  const float clamped = amax != amax ? amax : fmaxf(amax, 0.125f);
  const float scale = round_to<T>(keep_f32(__fmul_rn(round_to<T>(__fdiv_rn(1.0f, clamped)), 448.0f)));
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    scale_rscale[0] = scale;
    scale_rscale[1] = round_to<T>(__fdiv_rn(1.0f, scale));
  }
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float q = round_to<T>(__fmul_rn(Cvt<T>::to_f32(x[i]), scale));
  out[i] = f32_to_fp8_e4m3fn(q != q ? __uint_as_float(0x7fc00000u) : fminf(fmaxf(q, -448.0f), 448.0f));
}

// Quantise and dequantise again in one pass: the values a fake-quantised activation tensor holds.
template <typename T>
__global__ void __launch_bounds__(256)
fake_quant_fp8_kernel(const T* __restrict__ x, const float* __restrict__ rscale, int64_t n, T* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  out[i] = Cvt<T>::from_f32(FakeQuant(rscale).one<T>(Cvt<T>::to_f32(x[i])));
}

template <bool I4>
static int launch_block_scaled(const void* d, const void* m, int dm_dtype, const uint8_t* qs, int64_t n_blocks,
                               int block_size, int is_signed, void* out, int out_dtype, hipStream_t st) {
  const int64_t n = n_blocks * block_size;
  if (n == 0) return STMOE_OK;
  const int threads = 256;
  const int64_t blocks = (n / 4 + threads - 1) / threads;
  switch (out_dtype) {
    case STMOE_F32:
      dequant_block_scaled_kernel<float, I4><<<dim3((unsigned)blocks), threads, 0, st>>>(
          d, m, dm_dtype, qs, n, block_size, is_signed, (float*)out);
      break;
    case STMOE_F16:
      dequant_block_scaled_kernel<f16_t, I4><<<dim3((unsigned)blocks), threads, 0, st>>>(
          d, m, dm_dtype, qs, n, block_size, is_signed, (f16_t*)out);
      break;
    case STMOE_BF16:
      dequant_block_scaled_kernel<bf16_t, I4><<<dim3((unsigned)blocks), threads, 0, st>>>(
          d, m, dm_dtype, qs, n, block_size, is_signed, (bf16_t*)out);
      break;
    default:
      return set_error(STMOE_ERR_DTYPE, "dequant_block_scaled: out_dtype %d is not f32/f16/bf16", out_dtype);
  }
  return check_launch("dequant_block_scaled");
}

static int check_block_args(const void* d, const void* qs, void* out, int dm_dtype, int64_t n_blocks,
                            int block_size, const char* who) {
  STMOE_REQUIRE(n_blocks >= 0, STMOE_ERR_SHAPE, "%s: n_blocks %lld < 0", who, (long long)n_blocks);
  if (n_blocks == 0) return STMOE_OK;
  STMOE_REQUIRE(d && qs && out, STMOE_ERR_NULL, "%s: d, qs and out must not be NULL", who);
  STMOE_REQUIRE(dm_dtype == STMOE_F32 || dm_dtype == STMOE_F16 || dm_dtype == STMOE_BF16, STMOE_ERR_DTYPE,
                "%s: scale dtype %d is not f32/f16/bf16", who, dm_dtype);
  STMOE_REQUIRE(block_size > 0 && block_size % 4 == 0, STMOE_ERR_SHAPE,
                "%s: block size %d must be a positive multiple of 4", who, block_size);
  STMOE_REQUIRE(n_blocks * (int64_t)block_size / 4 / 256 < 0x7fffffffLL, STMOE_ERR_SHAPE, "%s: too many elements", who);
  return STMOE_OK;
}

}  // namespace stmoe

using namespace stmoe;

extern "C" int stmoe_dequant_block_scaled(const void* d, const void* m, int dm_dtype, const int8_t* qs,
                                          int64_t n_blocks, int block_size, void* out, int out_dtype,
                                          stmoe_stream_t stream) {
  int rc = check_block_args(d, qs, out, dm_dtype, n_blocks, block_size, "dequant_block_scaled");
  if (rc) return rc;
  return launch_block_scaled<false>(d, m, dm_dtype, (const uint8_t*)qs, n_blocks, block_size, 1, out, out_dtype,
                                    as_stream(stream));
}

extern "C" int stmoe_dequant_block_scaled_i4(const void* d, const void* m, int dm_dtype, const uint8_t* qs_packed,
                                             int64_t n_blocks, int block_size, int is_signed, void* out,
                                             int out_dtype, stmoe_stream_t stream) {
  int rc = check_block_args(d, qs_packed, out, dm_dtype, n_blocks, block_size, "dequant_block_scaled_i4");
  if (rc) return rc;
  return launch_block_scaled<true>(d, m, dm_dtype, qs_packed, n_blocks, block_size, is_signed, out, out_dtype,
                                   as_stream(stream));
}

extern "C" int stmoe_promote_i4(const uint8_t* qs_packed, int64_t n_bytes, int is_signed, void* out,
                                stmoe_stream_t stream) {
  STMOE_REQUIRE(n_bytes >= 0, STMOE_ERR_SHAPE, "promote_i4: n_bytes %lld < 0", (long long)n_bytes);
  if (n_bytes == 0) return STMOE_OK;
  STMOE_REQUIRE(qs_packed && out, STMOE_ERR_NULL, "promote_i4: NULL pointer");
  const int64_t blocks = (n_bytes + 255) / 256;
  promote_i4_kernel<<<dim3((unsigned)blocks), 256, 0, as_stream(stream)>>>(qs_packed, n_bytes, is_signed, (uint8_t*)out);
  return check_launch("promote_i4");
}

template <typename DD>
static int launch_tensor_scaled(const void* qs, int qs_dtype, const void* d, const void* m, int64_t per_scale,
                                int64_t d_count, int64_t n, void* out, int out_dtype, hipStream_t st) {
  const int64_t blocks = (n + 255) / 256;
  dim3 g((unsigned)blocks);
  switch (out_dtype) {
    case STMOE_F32:
      dequant_tensor_scaled_kernel<DD, float><<<g, 256, 0, st>>>(qs, qs_dtype, (const DD*)d, (const DD*)m, per_scale, d_count, n, (float*)out);
      break;
    case STMOE_F16:
      dequant_tensor_scaled_kernel<DD, f16_t><<<g, 256, 0, st>>>(qs, qs_dtype, (const DD*)d, (const DD*)m, per_scale, d_count, n, (f16_t*)out);
      break;
    case STMOE_BF16:
      dequant_tensor_scaled_kernel<DD, bf16_t><<<g, 256, 0, st>>>(qs, qs_dtype, (const DD*)d, (const DD*)m, per_scale, d_count, n, (bf16_t*)out);
      break;
    default:
      return set_error(STMOE_ERR_DTYPE, "dequant_tensor_scaled: out_dtype %d is not f32/f16/bf16", out_dtype);
  }
  return check_launch("dequant_tensor_scaled");
}

extern "C" int stmoe_dequant_tensor_scaled(const void* qs, int qs_dtype, const void* d, const void* m, int d_dtype,
                                           int64_t d_count, int64_t n, void* out, int out_dtype,
                                           stmoe_stream_t stream) {
  STMOE_REQUIRE(n >= 0, STMOE_ERR_SHAPE, "dequant_tensor_scaled: n %lld < 0", (long long)n);
  if (n == 0) return STMOE_OK;
  STMOE_REQUIRE(qs && d && out, STMOE_ERR_NULL, "dequant_tensor_scaled: NULL pointer");
  STMOE_REQUIRE(qs_dtype >= STMOE_F32 && qs_dtype <= STMOE_U8, STMOE_ERR_DTYPE, "dequant_tensor_scaled: qs dtype %d", qs_dtype);
  STMOE_REQUIRE(d_count >= 1 && n % d_count == 0, STMOE_ERR_SHAPE,
                "dequant_tensor_scaled: %lld scales do not divide %lld elements", (long long)d_count, (long long)n);
  const int64_t per_scale = n / d_count;
  switch (d_dtype) {
    case STMOE_F32: return launch_tensor_scaled<float>(qs, qs_dtype, d, m, per_scale, d_count, n, out, out_dtype, as_stream(stream));
    case STMOE_F16: return launch_tensor_scaled<f16_t>(qs, qs_dtype, d, m, per_scale, d_count, n, out, out_dtype, as_stream(stream));
    case STMOE_BF16: return launch_tensor_scaled<bf16_t>(qs, qs_dtype, d, m, per_scale, d_count, n, out, out_dtype, as_stream(stream));
    default: return set_error(STMOE_ERR_DTYPE, "dequant_tensor_scaled: scale dtype %d is not f32/f16/bf16", d_dtype);
  }
}

extern "C" int stmoe_dequant_tensor_scaled_per_axis(const void* qs, int qs_dtype, const void* d, const void* m, int d_dtype,
                                                    int64_t axis_len, int64_t inner, int64_t n, void* out, int out_dtype,
                                                    stmoe_stream_t stream) {
  STMOE_REQUIRE(n >= 0, STMOE_ERR_SHAPE, "dequant_tensor_scaled_per_axis: n %lld < 0", (long long)n);
  if (n == 0) return STMOE_OK;
  STMOE_REQUIRE(qs && d && out, STMOE_ERR_NULL, "dequant_tensor_scaled_per_axis: NULL pointer");
  STMOE_REQUIRE(qs_dtype >= STMOE_F32 && qs_dtype <= STMOE_U8, STMOE_ERR_DTYPE, "dequant_tensor_scaled_per_axis: qs dtype %d", qs_dtype);
  STMOE_REQUIRE(axis_len >= 1 && inner >= 1 && n % (axis_len * inner) == 0, STMOE_ERR_SHAPE,
                "dequant_tensor_scaled_per_axis: an axis of %lld with %lld elements behind it does not divide %lld elements",
                (long long)axis_len, (long long)inner, (long long)n);
  switch (d_dtype) {
    case STMOE_F32: return launch_tensor_scaled<float>(qs, qs_dtype, d, m, inner, axis_len, n, out, out_dtype, as_stream(stream));
    case STMOE_F16: return launch_tensor_scaled<f16_t>(qs, qs_dtype, d, m, inner, axis_len, n, out, out_dtype, as_stream(stream));
    case STMOE_BF16: return launch_tensor_scaled<bf16_t>(qs, qs_dtype, d, m, inner, axis_len, n, out, out_dtype, as_stream(stream));
    default: return set_error(STMOE_ERR_DTYPE, "dequant_tensor_scaled_per_axis: scale dtype %d is not f32/f16/bf16", d_dtype);
  }
}

// Per-axis static quantisation: x * scale[j] with j the index along the scaled axis, in the dtype eager torch gives the
// product of the two tensors (P = T when the scales have x's dtype, fp32 otherwise), clamped and cast.
template <typename T, typename S, typename P>
__global__ void __launch_bounds__(256)
quantize_fp8_per_axis_kernel(const T* __restrict__ x, const S* __restrict__ scale, int64_t axis_len, int64_t inner, int64_t n,
                             uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t j = (i / inner) % axis_len;
  const float q = round_to<P>(__fmul_rn(Cvt<T>::to_f32(x[i]), Cvt<S>::to_f32(scale[j])));
  out[i] = f32_to_fp8_e4m3fn(q != q ? __uint_as_float(0x7fc00000u) : fminf(fmaxf(q, -448.0f), 448.0f));
}

extern "C" int stmoe_quantize_fp8_per_axis(const void* x, int x_dtype, const void* scale, int scale_dtype, int64_t axis_len,
                                           int64_t inner, int64_t n, void* out_fp8, stmoe_stream_t stream) {
  STMOE_REQUIRE(n >= 0, STMOE_ERR_SHAPE, "quantize_fp8_per_axis: n %lld < 0", (long long)n);
  if (n == 0) return STMOE_OK;
  STMOE_REQUIRE(x && scale && out_fp8, STMOE_ERR_NULL, "quantize_fp8_per_axis: NULL pointer");
  STMOE_REQUIRE(axis_len >= 1 && inner >= 1 && n % (axis_len * inner) == 0, STMOE_ERR_SHAPE,
                "quantize_fp8_per_axis: an axis of %lld with %lld elements behind it does not divide %lld elements",
                (long long)axis_len, (long long)inner, (long long)n);
  dim3 g((unsigned)((n + 255) / 256));
  hipStream_t st = as_stream(stream);
#define STMOE_QPA(TT, SS, PP)                                                                                            \
  quantize_fp8_per_axis_kernel<TT, SS, PP><<<g, 256, 0, st>>>((const TT*)x, (const SS*)scale, axis_len, inner, n, (uint8_t*)out_fp8)
  if (x_dtype == STMOE_F32 && scale_dtype == STMOE_F32) STMOE_QPA(float, float, float);
  else if (x_dtype == STMOE_F16 && scale_dtype == STMOE_F32) STMOE_QPA(f16_t, float, float);
  else if (x_dtype == STMOE_BF16 && scale_dtype == STMOE_F32) STMOE_QPA(bf16_t, float, float);
  else if (x_dtype == STMOE_F16 && scale_dtype == STMOE_F16) STMOE_QPA(f16_t, f16_t, f16_t);
  else if (x_dtype == STMOE_BF16 && scale_dtype == STMOE_BF16) STMOE_QPA(bf16_t, bf16_t, bf16_t);
  else return set_error(STMOE_ERR_DTYPE, "quantize_fp8_per_axis: x dtype %d with scale dtype %d not implemented", x_dtype, scale_dtype);
#undef STMOE_QPA
  return check_launch("quantize_fp8_per_axis");
}

extern "C" int stmoe_quantize_fp8(const void* x, int x_dtype, const float* rscale, int64_t n, void* out_fp8,
                                  stmoe_stream_t stream) {
  STMOE_REQUIRE(n >= 0, STMOE_ERR_SHAPE, "quantize_fp8: n %lld < 0", (long long)n);
  if (n == 0) return STMOE_OK;
  STMOE_REQUIRE(x && rscale && out_fp8, STMOE_ERR_NULL, "quantize_fp8: NULL pointer");
  dim3 g((unsigned)((n + 255) / 256));
  hipStream_t st = as_stream(stream);
  switch (x_dtype) {
    case STMOE_F32: quantize_fp8_kernel<float><<<g, 256, 0, st>>>((const float*)x, rscale, n, (uint8_t*)out_fp8); break;
    case STMOE_F16: quantize_fp8_kernel<f16_t><<<g, 256, 0, st>>>((const f16_t*)x, rscale, n, (uint8_t*)out_fp8); break;
    case STMOE_BF16: quantize_fp8_kernel<bf16_t><<<g, 256, 0, st>>>((const bf16_t*)x, rscale, n, (uint8_t*)out_fp8); break;
    default: return set_error(STMOE_ERR_DTYPE, "quantize_fp8: x dtype %d is not f32/f16/bf16", x_dtype);
  }
  return check_launch("quantize_fp8");
}

namespace stmoe {
// rows of x [*, K] (K a multiple of 8, rows 16-byte aligned) quantised into out [rows, K] in the order perm gives
int quantize_fp8_gather(const void* x, int dtype, const float* rscale, const int32_t* perm, int k, int64_t rows, int64_t K, void* out,
                        int64_t block_rows, hipStream_t st) {
  STMOE_REQUIRE(rows >= 0 && rows < 0x7fffffffLL && K > 0 && K % 8 == 0 && k >= 1 && (block_rows == 0 || (block_rows >= rows && K % 64 == 0)),
                STMOE_ERR_SHAPE, "quantize_fp8_gather: rows=%lld K=%lld", (long long)rows, (long long)K);
  if (rows == 0) return STMOE_OK;
  STMOE_REQUIRE(x && rscale && out, STMOE_ERR_NULL, "quantize_fp8_gather: NULL pointer");
  const dim3 g((unsigned)rows);
  switch (dtype) {
    case STMOE_F32: quantize_fp8_gather_kernel<float><<<g, 256, 0, st>>>((const float*)x, rscale, perm, k, K, (uint8_t*)out, block_rows); break;
    case STMOE_F16: quantize_fp8_gather_kernel<f16_t><<<g, 256, 0, st>>>((const f16_t*)x, rscale, perm, k, K, (uint8_t*)out, block_rows); break;
    case STMOE_BF16: quantize_fp8_gather_kernel<bf16_t><<<g, 256, 0, st>>>((const bf16_t*)x, rscale, perm, k, K, (uint8_t*)out, block_rows); break;
    default: return set_error(STMOE_ERR_DTYPE, "quantize_fp8_gather: dtype %d is not f32/f16/bf16", dtype);
  }
  return check_launch("quantize_fp8_gather");
}
}  // namespace stmoe

extern "C" size_t stmoe_dynamic_quantize_fp8_scratch_bytes(void) { return 1024 * sizeof(float); }

extern "C" int stmoe_dynamic_quantize_fp8(const void* x, int dtype, int64_t n, void* out_fp8, float* scale_rscale_out,
                                          void* scratch, size_t scratch_bytes, stmoe_stream_t stream) {
  STMOE_REQUIRE(n >= 0, STMOE_ERR_SHAPE, "dynamic_quantize_fp8: n %lld < 0", (long long)n);
  STMOE_REQUIRE(scale_rscale_out && scratch, STMOE_ERR_NULL, "dynamic_quantize_fp8: NULL pointer");
  STMOE_REQUIRE(scratch_bytes >= stmoe_dynamic_quantize_fp8_scratch_bytes(), STMOE_ERR_WORKSPACE,
                "dynamic_quantize_fp8: scratch %zu < %zu bytes", scratch_bytes, stmoe_dynamic_quantize_fp8_scratch_bytes());
  STMOE_REQUIRE(n == 0 || (x && out_fp8), STMOE_ERR_NULL, "dynamic_quantize_fp8: NULL pointer");
  STMOE_REQUIRE((n + 255) / 256 < ((int64_t)1 << 31), STMOE_ERR_SHAPE, "dynamic_quantize_fp8: n too large");
  hipStream_t st = as_stream(stream);
  float* partial = static_cast<float*>(scratch);
  // an empty tensor has no maximum (torch raises); the scale of amax = 0 is reported and nothing is written
  const int n_partial = (int)(n == 0 ? 1 : ((n + 2047) / 2048 < 1024 ? (n + 2047) / 2048 : 1024));
  const dim3 g2((unsigned)(n == 0 ? 1 : (n + 255) / 256));
#define STMOE_DQ(TT)                                                                                          \
  absmax_partial_kernel<TT><<<dim3((unsigned)n_partial), 256, 0, st>>>((const TT*)x, n, partial);             \
  dynamic_quantize_fp8_kernel<TT><<<g2, 256, 0, st>>>((const TT*)x, n, partial, n_partial, (uint8_t*)out_fp8, scale_rscale_out)
  switch (dtype) {
    case STMOE_F32: STMOE_DQ(float); break;
    case STMOE_F16: STMOE_DQ(f16_t); break;
    case STMOE_BF16: STMOE_DQ(bf16_t); break;
    default: return set_error(STMOE_ERR_DTYPE, "dynamic_quantize_fp8: dtype %d is not f32/f16/bf16", dtype);
  }
#undef STMOE_DQ
  return check_launch("dynamic_quantize_fp8");
}

extern "C" int stmoe_fake_quant_fp8(const void* x, int dtype, const float* rscale, int64_t n, void* out,
                                    stmoe_stream_t stream) {
  STMOE_REQUIRE(n >= 0, STMOE_ERR_SHAPE, "fake_quant_fp8: n %lld < 0", (long long)n);
  if (n == 0) return STMOE_OK;
  STMOE_REQUIRE(x && rscale && out, STMOE_ERR_NULL, "fake_quant_fp8: NULL pointer");
  dim3 g((unsigned)((n + 255) / 256));
  hipStream_t st = as_stream(stream);
  switch (dtype) {
    case STMOE_F32: fake_quant_fp8_kernel<float><<<g, 256, 0, st>>>((const float*)x, rscale, n, (float*)out); break;
    case STMOE_F16: fake_quant_fp8_kernel<f16_t><<<g, 256, 0, st>>>((const f16_t*)x, rscale, n, (f16_t*)out); break;
    case STMOE_BF16: fake_quant_fp8_kernel<bf16_t><<<g, 256, 0, st>>>((const bf16_t*)x, rscale, n, (bf16_t*)out); break;
    default: return set_error(STMOE_ERR_DTYPE, "fake_quant_fp8: dtype %d is not f32/f16/bf16", dtype);
  }
  return check_launch("fake_quant_fp8");
}
