// Generic grouped projection: one wavefront per (sorted row, output feature), fp32 FMA on the vector
// ALU.  It covers every activation dtype x weight format combination, including fp32 activations that
// have no MFMA path here, and serves as a second implementation against which the MFMA kernels are
// cross-checked.
#include "ffn_kernels.h"

namespace stmoe {

template <typename T> __device__ __forceinline__ void load_x16(const T* p, float out[16]);
template <> __device__ __forceinline__ void load_x16<float>(const float* p, float out[16]) {
  const float4* q = reinterpret_cast<const float4*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float4 v = q[i];
    out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
  }
}
template <> __device__ __forceinline__ void load_x16<f16_t>(const f16_t* p, float out[16]) {
  const uint4* q = reinterpret_cast<const uint4*>(p);
  const uint4 a = q[0], b = q[1];
  const uint32_t r[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    out[2 * i] = f16_bits_to_f32(r[i] & 0xffffu);
    out[2 * i + 1] = f16_bits_to_f32(r[i] >> 16);
  }
}
template <> __device__ __forceinline__ void load_x16<bf16_t>(const bf16_t* p, float out[16]) {
  const uint4* q = reinterpret_cast<const uint4*>(p);
  const uint4 a = q[0], b = q[1];
  const uint32_t r[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    out[2 * i] = __uint_as_float(r[i] << 16);
    out[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
  }
}

template <typename T, int WF, int MODE>
__global__ void __launch_bounds__(256)
grouped_generic_kernel(GemmParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int i = blockIdx.y;
  if (n >= p.n_out) return;
  int e = 0, rb, re;
  if (p.offsets) {
    if (i >= p.offsets[p.E]) return;
    while (e + 1 < p.E && i >= p.offsets[e + 1]) ++e;
  } else if (i >= p.fixed_rows) {
    return;
  }
  (void)rb; (void)re;
  const int64_t src = p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i;
  const T* xr = reinterpret_cast<const T*>(p.a) + src * p.lda;

  float acc0 = 0.0f, acc1 = 0.0f;
  for (int64_t k0 = (int64_t)lane * 16; k0 < p.kred; k0 += 64 * 16) {
    float xv[16], wv[16];
    load_x16<T>(xr + k0, xv);
    Chunk16<WF> c;
    c.load(p.w0, e, n, k0);
    c.to_f32(wv);
#pragma unroll
    for (int j = 0; j < 16; ++j) acc0 = fmaf(xv[j], round_to<T>(wv[j]), acc0);
    if (MODE == MODE_GATEUP) {
      c.load(p.w1, e, n, k0);
      c.to_f32(wv);
#pragma unroll
      for (int j = 0; j < 16; ++j) acc1 = fmaf(xv[j], round_to<T>(wv[j]), acc1);
    }
  }
  acc0 = wave_xor_sum(acc0);
  if (MODE == MODE_GATEUP) acc1 = wave_xor_sum(acc1);
  if (lane == 0) {
    const float scale = p.x_scale ? *p.x_scale : 1.0f;
    T* o = reinterpret_cast<T*>(p.out) + out_row(p, i) * p.ldo + n;
    if (MODE == MODE_GATEUP) *o = Cvt<T>::from_f32(gateup_epilogue<T>(p.act, acc0, acc1, scale, fq_scale(p)));
    else *o = Cvt<T>::from_f32(acc0 * scale);
  }
}

template <typename T, int WF>
static int launch_generic_tw(int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0 || p.n_out == 0) return STMOE_OK;
  dim3 grid((unsigned)((p.n_out + 3) / 4), (unsigned)max_rows);
  if (mode == MODE_GATEUP) grouped_generic_kernel<T, WF, MODE_GATEUP><<<grid, 256, 0, st>>>(p);
  else grouped_generic_kernel<T, WF, MODE_DOWN><<<grid, 256, 0, st>>>(p);
  return check_launch("grouped_generic");
}

template <typename T>
static int launch_generic_t(int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  switch (wtag) {
    case WF_Q8_0: return launch_generic_tw<T, WF_Q8_0>(mode, p, max_rows, st);
    case WF_Q4_1: return launch_generic_tw<T, WF_Q4_1>(mode, p, max_rows, st);
    case WF_FP8_F32D: return launch_generic_tw<T, WF_FP8_F32D>(mode, p, max_rows, st);
    case WF_FP8_F16D: return launch_generic_tw<T, WF_FP8_F16D>(mode, p, max_rows, st);
    case WF_DENSE_F32: return launch_generic_tw<T, WF_DENSE_F32>(mode, p, max_rows, st);
    case WF_DENSE_F16: return launch_generic_tw<T, WF_DENSE_F16>(mode, p, max_rows, st);
    case WF_DENSE_BF16: return launch_generic_tw<T, WF_DENSE_BF16>(mode, p, max_rows, st);
    case WF_Q8_0_P: return launch_generic_tw<T, WF_Q8_0_P>(mode, p, max_rows, st);
    case WF_Q4_1_P: return launch_generic_tw<T, WF_Q4_1_P>(mode, p, max_rows, st);
    case WF_FP8_F32D_P: return launch_generic_tw<T, WF_FP8_F32D_P>(mode, p, max_rows, st);
    default: return set_error(STMOE_ERR_UNSUPPORTED, "generic kernel: unknown weight tag %d", wtag);
  }
}

int launch_generic(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows > 65535) return set_error(STMOE_ERR_UNSUPPORTED, "generic kernel: %lld rows exceed its 65535-row grid", (long long)max_rows);
  switch (act_dtype) {
    case STMOE_F32: return launch_generic_t<float>(wtag, mode, p, max_rows, st);
    case STMOE_F16: return launch_generic_t<f16_t>(wtag, mode, p, max_rows, st);
    case STMOE_BF16: return launch_generic_t<bf16_t>(wtag, mode, p, max_rows, st);
    default: return set_error(STMOE_ERR_DTYPE, "generic kernel: activation dtype %d", act_dtype);
  }
}

}  // namespace stmoe
