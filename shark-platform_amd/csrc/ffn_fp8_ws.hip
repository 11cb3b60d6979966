// Prefill kernel for fp8 (e4m3fn) activations and packed fp8 tensor-scaled weights on the fp8 matrix cores.
//
// Neither operand needs a conversion on its way to the matrix cores, so no byte passes through a register before the
// MFMA reads it: every wavefront sends its share of the next stage global -> LDS directly (global_load_lds_dwordx4) and
// then only reads LDS operands and issues MFMAs.
//
//   256 x 256 workgroup tile (GATEUP: 128 gate + the same 128 up rows), 8 wavefronts of 128 weight rows x 64 token
//   rows, K stage 64 (one v_mfma_scale_f32_32x32x64_f8f6f4 deep), five stages of 16 KB weights + 16 KB tokens = 160 KB,
//   loads issued four stages ahead, one barrier per stage.
//   weights: a packed 1 KB piece (16 rows x 64 k; lane 16 g + n holds row n, k = 16 g .. + 15) lands in LDS as it is;
//            MFMA lane (r, h) supplies row r, samples 32 h .. 32 h + 31: pieces' units 2 h and 2 h + 1 of row r % 16,
//            16 consecutive lanes read 256 consecutive bytes.
//   tokens:  quantised rows, 64 bytes per stage; lane l of a load fetches the 16 bytes that belong at LDS position l
//            (row l / 4 of the load's 16 rows, the unit that x_unit maps to position l % 4), so that the gather and the
//            bank swizzle cost nothing; rows of a partial token tile are spread over the four token-row groups.
//   results: D[8 (i / 4) + 4 h + i % 4][r] (probed on the hardware: rows are the weight rows, columns the token rows);
//            both token blocks' operands (16 registers) stay resident while the four weight blocks stream through 8
//            registers, so every operand byte is read from LDS once per wavefront.
//   epilogue: the fp32 dot products of the quantised samples are scaled once by scale_x * d_w; the gate/up epilogue can
//            quantise the gated intermediate to e4m3fn for the down projection.
//   What bounds it: at 256 flop per operand byte the tile needs 32 KB per stage from L2 / HBM; with the operand loads
//   alone (no MFMA) the launch takes two thirds of its full time and with the MFMAs alone 60 %, i.e. the two overlap only
//   partly: the bytes in flight are capped by the LDS (4 stages of 32 KB), which covers the load latency under load only
//   just.  Reading the next stage's operands from LDS ahead of the barrier (software pipelining) changed nothing.
#include "ffn_mfma_common.h"

namespace stmoe {

typedef int intx8_t __attribute__((ext_vector_type(8)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));
template <int V> struct F8Int { static constexpr int value = V; };

__device__ __forceinline__ intx8_t join8(const u32x4_t& lo, const u32x4_t& hi) {
  return (intx8_t){(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}

// LDS unit (16 bytes) of a token row's unit u in a 64-byte stage row: rows r and r + 4 share banks, so the unit index
// is flipped with bit 2 of the row; 8 consecutive rows reading the same logical unit then touch 32 distinct banks.
__device__ __forceinline__ int x_unit(int row, int u) { return u ^ ((row >> 2) & 1); }

template <typename T, int MODE>
__global__ void __launch_bounds__(512, 1)
grouped_fp8_ws_kernel(GemmParams p, int n_tiles) {
  constexpr int BN = 256, BM = 256, KS = 64;      // K samples (= bytes per row) per stage
  constexpr int WSTAGE = BN * KS, XSTAGE = BM * KS;  // bytes
  constexpr int STAGE = WSTAGE + XSTAGE, D = 5;   // stages in LDS
  constexpr int LOADS = 4;                        // LDS-direct loads per wavefront and stage: 2 weight pieces + 2 x 16 token rows
  extern __shared__ __align__(16) uint8_t lds8[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  BigTile tile;
  if (!big_tile_id(p, BM, n_tiles, false, tile)) return;
  const int e = tile.e, row_begin = tile.row_begin, row_end = tile.row_end, ntile = tile.ntile;
  const int rows_here = row_end - row_begin;
  const int rpg = min(64, ((rows_here + 3) / 4 + 15) / 16 * 16);  // token rows per group of 64 LDS rows
  const int nst = (int)(p.kred >> 6);

  // ---- what this wavefront loads: weight pieces (row tiles) 2 wave, 2 wave + 1 and LDS token rows 32 wave .. + 31 ----
  const uint8_t* wq[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int rtl = 2 * wave + j;  // row tile of 16 inside the 256 weight rows of the stage
    int64_t row0;
    const WeightView* wv;
    if (MODE == MODE_GATEUP) {
      const bool up = rtl >= BN / 32;
      wv = up ? &p.w1 : &p.w0;
      row0 = (int64_t)e * wv->rows + (int64_t)ntile * (BN / 2) + (rtl % (BN / 32)) * 16;
    } else {
      wv = &p.w0;
      row0 = (int64_t)e * wv->rows + (int64_t)ntile * BN + rtl * 16;
    }
    const uint64_t addr = reinterpret_cast<uint64_t>(wv->qs + (row0 >> 4) * (p.kred >> 6) * 1024);  // K block 0 of the row tile
    // wave-uniform by construction; say so to the compiler (the address goes into scalar registers)
    // (the builtin returns a signed int: go through uint32_t, or the low half sign-extends into the high one)
    const uint32_t addr_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)addr);
    const uint32_t addr_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(addr >> 32));
    wq[j] = reinterpret_cast<const uint8_t*>((uint64_t)addr_lo | ((uint64_t)addr_hi << 32));
  }
  uint32_t xoff[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int lr = 32 * wave + 16 * j + (lane >> 2);  // LDS row this lane fills
    const int r = min((lr >> 6) * rpg + min(lr & 63, rpg - 1), rows_here - 1);
    const int i = row_begin + r;
    const int64_t src = p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i;
    xoff[j] = (uint32_t)(src * p.lda + (x_unit(lr, lane & 3) << 4));  // x_unit is an involution: position -> logical unit
  }
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)lds8);
  const uint32_t w_lds = lds0 + 2 * wave * 1024, x_lds = lds0 + WSTAGE + 32 * wave * KS;
  const uint32_t lane16 = lane * 16;
  auto issue = [&](int st) __attribute__((always_inline)) {  // stage st of the reduction into LDS slot st % D
    const uint32_t slot = (uint32_t)(st % D) * STAGE;
    vm_load16_to_lds(wq[0], lane16 + (uint32_t)st * 1024, w_lds + slot);
    vm_load16_to_lds(wq[1], lane16 + (uint32_t)st * 1024, w_lds + slot + 1024);
    vm_load16_to_lds(p.a, xoff[0] + (uint32_t)st * KS, x_lds + slot);
    vm_load16_to_lds(p.a, xoff[1] + (uint32_t)st * KS, x_lds + slot + 16 * KS);
  };

  // ---- operands: lane (r, h) supplies row r, samples 32 h .. 32 h + 31 ------------------------------------
  const int wn = wave & 1, wm = wave >> 1;
  const int r32 = lane & 31, h32 = lane >> 5;
  // weight row r of a 32-row block: piece r / 16, lane position 16 g + r % 16 for g = 2 h, 2 h + 1
  const uint8_t* const a_rd = lds8 + (MODE == MODE_GATEUP ? wn * 4 : wn * 8) * 1024 + (r32 >> 4) * 1024 + ((32 * h32 + (r32 & 15)) << 4);
  const int xrow = wm * 64 + r32;
  const uint8_t* const b_rd = lds8 + WSTAGE + xrow * KS;
  const int bu0 = x_unit(xrow, 2 * h32) << 4, bu1 = x_unit(xrow, 2 * h32 + 1) << 4;  // rows xrow and xrow + 32 swizzle alike
  floatx16_t acc[4][2];
  const int my_rows = min(rpg, rows_here - wm * rpg);

  auto compute = [&](auto both_tag, int slot) __attribute__((always_inline)) {
    constexpr bool BOTH = decltype(both_tag)::value;  // rows in both 32-row token blocks
    const uint8_t* bp = b_rd + slot * STAGE;
    intx8_t bf[2];
#pragma unroll
    for (int q = 0; q < (BOTH ? 2 : 1); ++q)
      bf[q] = join8(*reinterpret_cast<const u32x4_t*>(bp + q * 32 * KS + bu0), *reinterpret_cast<const u32x4_t*>(bp + q * 32 * KS + bu1));
#pragma unroll
    for (int ti = 0; ti < 4; ++ti) {
      // 32-row block ti of the wavefront: GATEUP blocks 0, 1 are gate rows, 2, 3 the matching up rows (pieces 8 ..)
      const int piece_off = MODE == MODE_GATEUP ? (ti < 2 ? 0 : 8) + (ti & 1) * 2 : ti * 2;
      const uint8_t* ap = a_rd + slot * STAGE + piece_off * 1024;
      const intx8_t af = join8(*reinterpret_cast<const u32x4_t*>(ap), *reinterpret_cast<const u32x4_t*>(ap + 256));
#pragma unroll
      for (int q = 0; q < (BOTH ? 2 : 1); ++q)
        acc[ti][q] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, bf[q], acc[ti][q], 0, 0, 0, 127, 0, 127);
    }
  };
  auto k_loop = [&](auto both_tag) __attribute__((always_inline)) {
    constexpr bool BOTH = decltype(both_tag)::value;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < (BOTH ? 2 : 1); ++b)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[a][b][q] = 0.0f;
    int slot = 0;
    int st = 0;
    // steady part: the loads of stages st + 1 .. st + D - 2 may still be in flight when stage st is needed
    for (; st + D - 1 < nst; ++st) {
      vm_wait<(D - 2) * LOADS>();
      __syncthreads();       // everybody's loads of stage st have landed; everybody is done with stage st - 1
      issue(st + D - 1);     // into the slot of stage st - 1
      compute(both_tag, slot);
      slot = slot == D - 1 ? 0 : slot + 1;
    }
    for (; st < nst; ++st) {
      vm_wait<0>();
      __syncthreads();
      compute(both_tag, slot);
      slot = slot == D - 1 ? 0 : slot + 1;
    }
  };

  // ---- epilogue: scale by the activations' reciprocal scale times the weights' scale ---------------------
  const float xsc = p.x_scale[0];
  const float s0 = xsc * reinterpret_cast<const float*>(p.w0.d)[p.w0.d_count > 1 ? e : 0];
  const float s1 = MODE == MODE_GATEUP ? xsc * reinterpret_cast<const float*>(p.w1.d)[p.w1.d_count > 1 ? e : 0] : 0.0f;
  const float out_rs = p.out_scale ? p.out_scale[0] : 0.0f;
  // 1 / out_rs once; per element q = v * inv refined by one residual step (fma(-q, rs, v) * inv + q), which is the
  // correctly rounded quotient except in rare last-bit cases that the following rounding to T absorbs
  const float out_inv = p.out_scale ? __builtin_amdgcn_rcpf(out_rs) : 0.0f;
  auto epilogue = [&](auto tj_tag, auto act_tag) __attribute__((always_inline)) {
    constexpr int tj = decltype(tj_tag)::value;
    constexpr int ACT = decltype(act_tag)::value;
    if (tj * 32 + r32 < my_rows) {
      const int64_t orow = out_row(p, row_begin + wm * rpg + tj * 32 + r32) * p.ldo;
      if (MODE == MODE_GATEUP) {
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
          for (int b = 0; b < 4; ++b) {  // four consecutive features per 8-row band of the 32 x 32 result
            const int64_t col = (int64_t)ntile * (BN / 2) + wn * 64 + ti * 32 + 8 * b + 4 * h32;
            float gq[4], uq[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              gq[q] = acc[ti][tj][4 * b + q] * s0;
              uq[q] = acc[ti + 2][tj][4 * b + q] * s1;
            }
            if (p.out_scale) {  // e4m3fn(clamp(T(v / rscale))) for the next fp8 projection
              float t[4];
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const float a = round_to<T>(act_fast<ACT>(round_to<T>(gq[q])));
                const float v = round_to<T>(__fmul_rn(a, round_to<T>(uq[q])));
                const float q0 = v * out_inv;
                const float q1 = __builtin_fmaf(__builtin_fmaf(-q0, out_rs, v), out_inv, q0);
                t[q] = fminf(fmaxf(round_to<T>(q1), -448.0f), 448.0f);
              }
              int qv = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], 0, false);  // hardware OCP e4m3fn, round to nearest even
              qv = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], qv, true);
              *reinterpret_cast<int*>(reinterpret_cast<uint8_t*>(p.out) + orow + col) = qv;
            } else {
              *reinterpret_cast<uint2*>(reinterpret_cast<T*>(p.out) + orow + col) = gateup_quad<T, ACT>(gq, uq);
            }
          }
      } else {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const int64_t col = (int64_t)ntile * BN + wn * 128 + ti * 32 + 8 * b + 4 * h32;
            const floatx16_t& c = acc[ti][tj];
            *reinterpret_cast<uint2*>(reinterpret_cast<T*>(p.out) + orow + col) =
                make_uint2(pack2<T>(c[4 * b] * s0, c[4 * b + 1] * s0), pack2<T>(c[4 * b + 2] * s0, c[4 * b + 3] * s0));
          }
      }
    }
  };
  auto epilogues = [&](auto both_tag) __attribute__((always_inline)) {
    constexpr bool BOTH = decltype(both_tag)::value;
    if (MODE == MODE_DOWN || p.act == STMOE_ACT_SILU) {
      epilogue(F8Int<0>{}, EpiAct<STMOE_ACT_SILU>{});
      if constexpr (BOTH) epilogue(F8Int<1>{}, EpiAct<STMOE_ACT_SILU>{});
    } else {
      epilogue(F8Int<0>{}, EpiAct<STMOE_ACT_GELU_ERF>{});
      if constexpr (BOTH) epilogue(F8Int<1>{}, EpiAct<STMOE_ACT_GELU_ERF>{});
    }
  };

  // every wavefront loads its share of every stage and meets every barrier, with or without token rows of its own
#pragma unroll 1
  for (int st = 0; st < min(D - 1, nst); ++st) issue(st);
  if (my_rows <= 0) {
    for (int st = 0; st < nst; ++st) {
      if (st + D - 1 < nst) {
        vm_wait<(D - 2) * LOADS>();
        __syncthreads();
        issue(st + D - 1);
      } else {
        vm_wait<0>();
        __syncthreads();
      }
    }
  } else if (my_rows <= 32) {
    k_loop(F8Int<0>{});
    epilogues(F8Int<0>{});
  } else {
    k_loop(F8Int<1>{});
    epilogues(F8Int<1>{});
  }
}

template <typename T, int MODE>
static int launch_fp8_ws_m(const GemmParams& p, int64_t max_rows, hipStream_t st) {
  constexpr int BN = 256, BM = 256;
  constexpr size_t lds_bytes = (size_t)5 * (BN + BM) * 64;
  static std::atomic<uint64_t> lds_ready{0};
  auto kern = grouped_fp8_ws_kernel<T, MODE>;
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ready, "fp8 ws kernel")) return rc;
  const int n_tiles = (int)(MODE == MODE_GATEUP ? p.n_out / (BN / 2) : p.n_out / BN);
  const int experts = p.offsets ? p.E : 1;
  const int m_slots = (int)((max_rows + BM - 1) / BM) + experts;
  kern<<<dim3((unsigned)big_grid(n_tiles, m_slots, false)), 512, lds_bytes, st>>>(p, n_tiles);
  return check_launch("grouped_fp8_ws");
}

// act_dtype: dtype of the results; activations are e4m3fn bytes (p.a, p.lda in bytes), weights packed fp8.
int launch_fp8_ws(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0) return STMOE_OK;
  if (!p.x_scale) return set_error(STMOE_ERR_NULL, "fp8 ws kernel: activation scale is NULL");
  if (wtag != WF_FP8_F32D_P) return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: needs packed fp8 weights with fp32 scale(s)");
  if (p.offsets && p.E >= 64) return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: at most 63 experts");
  if (p.kred % 256 != 0 || p.lda % 16 != 0 || p.ldo % 4 != 0 || p.n_out % (mode == MODE_GATEUP ? 128 : 256) != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: needs K %% 256 == 0 and output features in whole tiles");
  {
    const int64_t src_rows = p.perm ? (max_rows + p.k_top - 1) / p.k_top : max_rows;
    if (src_rows * p.lda >= (int64_t)1 << 32) return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: activations span 4 GB or more");
  }
  if (act_dtype == STMOE_F16)
    return mode == MODE_GATEUP ? launch_fp8_ws_m<f16_t, MODE_GATEUP>(p, max_rows, st) : launch_fp8_ws_m<f16_t, MODE_DOWN>(p, max_rows, st);
  if (act_dtype == STMOE_BF16)
    return mode == MODE_GATEUP ? launch_fp8_ws_m<bf16_t, MODE_GATEUP>(p, max_rows, st) : launch_fp8_ws_m<bf16_t, MODE_DOWN>(p, max_rows, st);
  return set_error(STMOE_ERR_DTYPE, "fp8 ws kernel: result dtype %d", act_dtype);
}

}  // namespace stmoe
