// Grouped projection with fp8 (e4m3fn) activations and fp8 tensor-scaled weights on the fp8 matrix cores.
//
// Operands stay one byte per element from HBM through LDS into v_mfma_f32_16x16x32_fp8_fp8; products of two e4m3
// values are exact in fp32 and the accumulation is fp32, so the dot product of the quantised samples is formed
// without any intermediate rounding and scaled once by (reciprocal scale of the activations) * (scale of the weights).
// The reference instead dequantises both sides to the activation dtype and multiplies (TensorScaledLayout.dequant,
// sharktank/sharktank/types/layouts.py:163-181, reached through `unbox_tensor`); the two agree to the rounding of the
// dequantised values, well inside the 2e-2 tolerance of the fp8 configuration.
//
// Tile: 128 weight rows x 128 token rows per workgroup (GATEUP: 128 gate + 128 up rows), K step 128, 4 wavefronts of
// 64 x 64, MFMA roles as in the 16-bit kernels (weight rows = "A" rows).  LDS rows are 128 bytes + 16 of padding.
#include "ffn_kernels.h"

namespace stmoe {

typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ floatx4_t mfma_fp8(uint2 a, uint2 b, floatx4_t c) {
  const long la = (long)(((uint64_t)a.y << 32) | a.x), lb = (long)(((uint64_t)b.y << 32) | b.x);
  return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(la, lb, c, 0, 0, 0);
}

// byte address of 16 consecutive samples (row, k0..k0+15) in the planar or the packed streaming order
template <bool PACKED>
__device__ __forceinline__ const uint8_t* fp8_piece(const WeightView& w, int64_t row, int64_t k0) {
  if (PACKED) return w.qs + packed_piece(row, k0, w.cols, 6);
  return w.qs + row * w.cols + k0;
}

template <typename T, int MODE, bool PACKED>
__global__ void __launch_bounds__(256)
grouped_fp8_tile_kernel(GemmParams p) {
  constexpr int BM = 128, BN = 128, BK = 128, LS = BK + 16;
  constexpr int NW = MODE == MODE_GATEUP ? 2 : 1;
  __shared__ __align__(16) uint8_t Xs[BM * LS];
  __shared__ __align__(16) uint8_t Ws[NW][BN * LS];

  int e, row_begin, row_end;
  if (!find_tile(p, blockIdx.x, BM, e, row_begin, row_end)) return;
  const int64_t n0 = (int64_t)blockIdx.y * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave >> 1, wm = wave & 1;
  const int rows_here = row_end - row_begin;

  // producer: tile = 128 rows x 8 pieces of 16 bytes -> 4 pieces per thread per operand
  const uint8_t* xsrc[4];
  int64_t wrow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int id = tid + 256 * j, r = min(id >> 3, rows_here - 1);  // rows past the end re-read the last row; never stored
    const int i = row_begin + r;
    const int64_t src = p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i;
    xsrc[j] = reinterpret_cast<const uint8_t*>(p.a) + src * p.lda + (id & 7) * 16;
    wrow[j] = min(n0 + (id >> 3), p.n_out - 1);
  }

  floatx4_t acc[NW][4][4];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) acc[w][a][b] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  uint4 xreg[4], wreg[NW][4];
  auto load_regs = [&](int64_t k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t kk = k0 + ((tid + 256 * j) & 7) * 16;
      const bool ok = kk < p.kred;
      xreg[j] = ok ? *reinterpret_cast<const uint4*>(xsrc[j] + k0) : make_uint4(0, 0, 0, 0);
      wreg[0][j] = ok ? *reinterpret_cast<const uint4*>(fp8_piece<PACKED>(p.w0, (int64_t)e * p.w0.rows + wrow[j], kk)) : make_uint4(0, 0, 0, 0);
      if (NW == 2)
        wreg[NW - 1][j] = ok ? *reinterpret_cast<const uint4*>(fp8_piece<PACKED>(p.w1, (int64_t)e * p.w1.rows + wrow[j], kk)) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = tid + 256 * j;
      *reinterpret_cast<uint4*>(&Xs[(id >> 3) * LS + (id & 7) * 16]) = xreg[j];
#pragma unroll
      for (int w = 0; w < NW; ++w) *reinterpret_cast<uint4*>(&Ws[w][(id >> 3) * LS + (id & 7) * 16]) = wreg[w][j];
    }
  };

  const int64_t nkt = (p.kred + BK - 1) / BK;
  load_regs(0);
  for (int64_t kt = 0; kt < nkt; ++kt) {
    store_lds();
    __syncthreads();
    if (kt + 1 < nkt) load_regs((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      uint2 bf[4];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj)
        bf[tj] = *reinterpret_cast<const uint2*>(&Xs[(wm * 64 + tj * 16 + (lane & 15)) * LS + ks * 32 + 8 * (lane >> 4)]);
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
          const uint2 af = *reinterpret_cast<const uint2*>(&Ws[w][(wn * 64 + ti * 16 + (lane & 15)) * LS + ks * 32 + 8 * (lane >> 4)]);
#pragma unroll
          for (int tj = 0; tj < 4; ++tj) acc[w][ti][tj] = mfma_fp8(af, bf[tj], acc[w][ti][tj]);
        }
    }
    __syncthreads();
  }

  // scales: activations' reciprocal scale times the weights' scale (per tensor or per expert)
  const float xs = p.x_scale[0];
  const float s0 = xs * reinterpret_cast<const float*>(p.w0.d)[p.w0.d_count > 1 ? e : 0];
  const float s1 = NW == 2 ? xs * reinterpret_cast<const float*>(p.w1.d)[p.w1.d_count > 1 ? e : 0] : 0.0f;
  const float out_rs = p.out_scale ? p.out_scale[0] : 0.0f;
#pragma unroll
  for (int ti = 0; ti < 4; ++ti)
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      const int i = row_begin + wm * 64 + tj * 16 + (lane & 15);
      const int64_t n = n0 + wn * 64 + ti * 16 + 4 * (lane >> 4);
      if (i < row_end && n < p.n_out) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (MODE == MODE_GATEUP) {
            const float gr = round_to<T>(acc[0][ti][tj][r] * s0);
            const float a = round_to<T>(act_rt(p.act, gr));
            const float ur = round_to<T>(acc[NW - 1][ti][tj][r] * s1);
            v[r] = round_to<T>(__fmul_rn(a, ur));
          } else {
            v[r] = acc[0][ti][tj][r] * s0;
          }
        }
        if (p.out_scale) {
          // quantise the intermediate for the next fp8 projection: e4m3fn(clamp(T(v / rscale)))
          uint32_t q = 0;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float t = round_to<T>(__fdiv_rn(v[r], out_rs));
            t = fminf(fmaxf(t, -448.0f), 448.0f);
            q |= (uint32_t)f32_to_fp8_e4m3fn(t) << (8 * r);
          }
          *reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(p.out) + out_row(p, i) * p.ldo + n) = q;
        } else {
          *reinterpret_cast<uint2*>(reinterpret_cast<T*>(p.out) + out_row(p, i) * p.ldo + n) =
              make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
        }
      }
    }
}

template <typename T, bool PACKED>
static int launch_fp8_t(int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  const int64_t experts = p.offsets ? p.E : 1;
  dim3 grid((unsigned)((max_rows + 127) / 128 + experts), (unsigned)((p.n_out + 127) / 128));
  if (mode == MODE_GATEUP) grouped_fp8_tile_kernel<T, MODE_GATEUP, PACKED><<<grid, 256, 0, st>>>(p);
  else grouped_fp8_tile_kernel<T, MODE_DOWN, PACKED><<<grid, 256, 0, st>>>(p);
  return check_launch("grouped_fp8_tile");
}

// act_dtype: dtype of the results (and of the unquantised layer); activations themselves are e4m3fn.
int launch_fp8_tile(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0 || p.n_out == 0) return STMOE_OK;
  if (!p.x_scale) return set_error(STMOE_ERR_NULL, "fp8 kernel: activation scale is NULL");
  if (wtag != WF_FP8_F32D && wtag != WF_FP8_F32D_P)
    return set_error(STMOE_ERR_UNSUPPORTED, "fp8 kernel: weights must be TensorScaledLayout e4m3fn with fp32 scale(s)");
  if (p.kred % 16 != 0 || p.n_out % 4 != 0 || p.ldo % 4 != 0 || p.lda % 16 != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "fp8 kernel: needs K %% 16 == 0 and N %% 4 == 0");
  const bool packed = wtag == WF_FP8_F32D_P;
  if (act_dtype == STMOE_F16) return packed ? launch_fp8_t<f16_t, true>(mode, p, max_rows, st) : launch_fp8_t<f16_t, false>(mode, p, max_rows, st);
  if (act_dtype == STMOE_BF16) return packed ? launch_fp8_t<bf16_t, true>(mode, p, max_rows, st) : launch_fp8_t<bf16_t, false>(mode, p, max_rows, st);
  return set_error(STMOE_ERR_DTYPE, "fp8 kernel: result dtype %d", act_dtype);
}

}  // namespace stmoe
