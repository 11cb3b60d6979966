// Grouped projection on the matrix cores: 128 x 128 output tile per workgroup, K step 64,
// v_mfma_f32_16x16x32_{f16,bf16}, weights dequantised by the producer into LDS.
//
// Operand roles: the weight rows are the MFMA "A" rows and the token rows the "B" columns, so that one
// lane of the 16x16 result holds 4 consecutive output features of one token and stores them as 8 bytes.
//   A fragment (16 weight rows x 32 k):  lane l <- row l%16, k = 8*(l/16) .. +7
//   B fragment (32 k x 16 tokens):       lane l <- token l%16, k = 8*(l/16) .. +7
//   D (16 x 16 fp32):                    lane l -> feature 4*(l/16)+r (r = 0..3), token l%16
#include "ffn_kernels.h"

namespace stmoe {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ floatx4_t mfma16(const uint4& a, const uint4& b, floatx4_t c);
template <> __device__ __forceinline__ floatx4_t mfma16<f16_t>(const uint4& a, const uint4& b, floatx4_t c) {
  union { uint4 u; half8_t h; } ua, ub;
  ua.u = a;
  ub.u = b;
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(ua.h, ub.h, c, 0, 0, 0);
}
template <> __device__ __forceinline__ floatx4_t mfma16<bf16_t>(const uint4& a, const uint4& b, floatx4_t c) {
  union { uint4 u; bf16x8_t h; } ua, ub;
  ua.u = a;
  ub.u = b;
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(ua.h, ub.h, c, 0, 0, 0);
}

template <typename T, int WF, int MODE>
__global__ void __launch_bounds__(256)
grouped_mfma_tile_kernel(GemmParams p) {
  constexpr int BM = 128, BN = 128, BK = 64;
  constexpr int LS = BK + 8;  // LDS row stride in 16-bit elements: 144 B keeps 16-byte row reads conflict free
  constexpr int NW = MODE == MODE_GATEUP ? 2 : 1;
  __shared__ __align__(16) uint16_t Xs[BM * LS];
  __shared__ __align__(16) uint16_t Ws[NW][BN * LS];

  int e, row_begin, row_end;
  if (!find_tile(p, blockIdx.x, BM, e, row_begin, row_end)) return;
  const int64_t n0 = (int64_t)blockIdx.y * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave >> 1, wm = wave & 1;

  // Producer assignment.  X tile: 128 rows x 8 chunks of 8 elements -> 4 chunks per thread.
  const T* xsrc[4];
  bool xok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int id = tid + 256 * j, r = id >> 3;
    const int i = row_begin + r;
    xok[j] = i < row_end;
    const int64_t src = xok[j] ? (p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i) : 0;
    xsrc[j] = reinterpret_cast<const T*>(p.a) + src * p.lda + (id & 7) * 8;
  }
  // W tile: 128 rows x 4 chunks of 16 elements -> 2 chunks per thread per matrix.
  int64_t wrow[2];
  bool wok[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int id = tid + 256 * j;
    wrow[j] = n0 + (id >> 2);
    wok[j] = wrow[j] < p.n_out;
  }

  floatx4_t acc[NW][4][4];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) acc[w][a][b] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  uint4 xreg[4];
  Chunk16<WF> wreg[NW][2];

  auto load_regs = [&](int64_t k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = xok[j] && (k0 + ((tid + 256 * j) & 7) * 8) < p.kred;
      xreg[j] = ok ? *reinterpret_cast<const uint4*>(xsrc[j] + k0) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t kk = k0 + ((tid + 256 * j) & 3) * 16;
      if (wok[j] && kk < p.kred) {
        wreg[0][j].load(p.w0, e, wrow[j], kk);
        if (NW == 2) wreg[NW - 1][j].load(p.w1, e, wrow[j], kk);
      } else {
        wreg[0][j].zero();
        if (NW == 2) wreg[NW - 1][j].zero();
      }
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int id = tid + 256 * j;
      *reinterpret_cast<uint4*>(&Xs[(id >> 3) * LS + (id & 7) * 8]) = xreg[j];
    }
#pragma unroll
    for (int w = 0; w < NW; ++w)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int id = tid + 256 * j;
        uint32_t v[8];
        chunk_to_T<T, WF>(wreg[w][j], v);
        uint4* dst = reinterpret_cast<uint4*>(&Ws[w][(id >> 2) * LS + (id & 3) * 16]);
        dst[0] = make_uint4(v[0], v[1], v[2], v[3]);
        dst[1] = make_uint4(v[4], v[5], v[6], v[7]);
      }
  };

  const int64_t nkt = (p.kred + BK - 1) / BK;
  load_regs(0);
  for (int64_t kt = 0; kt < nkt; ++kt) {
    store_lds();
    __syncthreads();
    if (kt + 1 < nkt) load_regs((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      uint4 bf[4];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj)
        bf[tj] = *reinterpret_cast<const uint4*>(&Xs[(wm * 64 + tj * 16 + (lane & 15)) * LS + ks * 32 + 8 * (lane >> 4)]);
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
          const uint4 af = *reinterpret_cast<const uint4*>(&Ws[w][(wn * 64 + ti * 16 + (lane & 15)) * LS + ks * 32 + 8 * (lane >> 4)]);
#pragma unroll
          for (int tj = 0; tj < 4; ++tj) acc[w][ti][tj] = mfma16<T>(af, bf[tj], acc[w][ti][tj]);
        }
    }
    __syncthreads();
  }

  const float scale = p.x_scale ? *p.x_scale : 1.0f;
  const FakeQuant fq = fq_scale(p);
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
          if (MODE == MODE_GATEUP) v[r] = gateup_epilogue<T>(p.act, acc[0][ti][tj][r], acc[NW - 1][ti][tj][r], scale, fq);
          else v[r] = acc[0][ti][tj][r] * scale;
        }
        uint2 pk = make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
        *reinterpret_cast<uint2*>(reinterpret_cast<T*>(p.out) + out_row(p, i) * p.ldo + n) = pk;
      }
    }
}

template <typename T, int WF>
static int launch_tw(int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0 || p.n_out == 0) return STMOE_OK;
  const int64_t experts = p.offsets ? p.E : 1;
  const int64_t slots = (max_rows + 127) / 128 + experts;
  dim3 grid((unsigned)slots, (unsigned)((p.n_out + 127) / 128));
  if (mode == MODE_GATEUP) grouped_mfma_tile_kernel<T, WF, MODE_GATEUP><<<grid, 256, 0, st>>>(p);
  else grouped_mfma_tile_kernel<T, WF, MODE_DOWN><<<grid, 256, 0, st>>>(p);
  return check_launch("grouped_mfma_tile");
}

int launch_mfma_tile(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (p.kred % 16 != 0 || p.n_out % 4 != 0 || p.ldo % 4 != 0 || p.lda % 8 != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma tile kernel: needs K %% 16 == 0, N %% 4 == 0 and 16-byte aligned rows");
  if (act_dtype == STMOE_F16) {
    switch (wtag) {
      case WF_Q8_0: return launch_tw<f16_t, WF_Q8_0>(mode, p, max_rows, st);
      case WF_Q4_1: return launch_tw<f16_t, WF_Q4_1>(mode, p, max_rows, st);
      case WF_FP8_F32D: return launch_tw<f16_t, WF_FP8_F32D>(mode, p, max_rows, st);
      case WF_DENSE_F16: return launch_tw<f16_t, WF_DENSE_F16>(mode, p, max_rows, st);
      case WF_Q8_0_P: return launch_tw<f16_t, WF_Q8_0_P>(mode, p, max_rows, st);
      case WF_Q4_1_P: return launch_tw<f16_t, WF_Q4_1_P>(mode, p, max_rows, st);
      case WF_FP8_F32D_P: return launch_tw<f16_t, WF_FP8_F32D_P>(mode, p, max_rows, st);
      default: break;
    }
  } else if (act_dtype == STMOE_BF16) {
    switch (wtag) {
      case WF_Q8_0: return launch_tw<bf16_t, WF_Q8_0>(mode, p, max_rows, st);
      case WF_Q4_1: return launch_tw<bf16_t, WF_Q4_1>(mode, p, max_rows, st);
      case WF_FP8_F32D: return launch_tw<bf16_t, WF_FP8_F32D>(mode, p, max_rows, st);
      case WF_DENSE_BF16: return launch_tw<bf16_t, WF_DENSE_BF16>(mode, p, max_rows, st);
      case WF_Q8_0_P: return launch_tw<bf16_t, WF_Q8_0_P>(mode, p, max_rows, st);
      case WF_Q4_1_P: return launch_tw<bf16_t, WF_Q4_1_P>(mode, p, max_rows, st);
      case WF_FP8_F32D_P: return launch_tw<bf16_t, WF_FP8_F32D_P>(mode, p, max_rows, st);
      default: break;
    }
  }
  return set_error(STMOE_ERR_UNSUPPORTED, "mfma tile kernel: no instantiation for activation dtype %d with weight tag %d",
                   act_dtype, wtag);
}

}  // namespace stmoe
