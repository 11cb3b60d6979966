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

struct F8Args {
  GemmParams p;
  int n_tiles;
  int wgs_per_xcd;  // grid size / 8
};

// One entry of a workgroup's unit table: what lane r of the table holds for the workgroup's r-th unit.
struct F8Unit {
  int e, ntile, row_begin, row_end;
};

// The launch's units in the order of big_unit (ffn_mfma_common.h: an XCD takes an eighth of the main list, expert by
// expert and feature tile by feature tile with an expert's token tiles of one feature tile next to each other, then an
// eighth of the partial token tiles), looked up for a different item in every lane: the loop over the experts is the
// same for all lanes (row counts come from readlane), each lane keeps what matches its own item.  `lane_off`: lane l holds
// the first row of expert l (lane E: the row total).  Returns whether the lane's item exists.
__device__ __forceinline__ bool f8_unit_of_lane(int lane_off, int E, int BM, int n_tiles, int xcd, int item, int balance, F8Unit& out) {
  int F = 0, R = 0;
  for (int e = 0; e < E; ++e) {
    const int rows = __builtin_amdgcn_readlane(lane_off, e + 1) - __builtin_amdgcn_readlane(lane_off, e);
    const BigExpertTiles x = big_expert_tiles(rows, BM, false, balance);
    F += x.main;
    R += x.partial;
  }
  const int UF = F * n_tiles, UR = R * n_tiles;
  const int f0 = (int)((int64_t)UF * xcd / 8), f1 = (int)((int64_t)UF * (xcd + 1) / 8);
  const int r0 = (int)((int64_t)UR * xcd / 8), r1 = (int)((int64_t)UR * (xcd + 1) / 8);
  const bool in_main = item < f1 - f0;
  const bool in_partial = !in_main && item - (f1 - f0) < r1 - r0;
  int u = in_main ? f0 + item : r0 + item - (f1 - f0);
  // partial list: feature tile by feature tile, one unit per expert that has a partial token tile
  const int p_ntile = R > 0 ? u / max(R, 1) : 0;
  int p_s = u - p_ntile * R;
  bool found = false;
  out.e = 0; out.ntile = 0; out.row_begin = 0; out.row_end = 0;
  for (int e = 0; e < E; ++e) {
    const int b = __builtin_amdgcn_readlane(lane_off, e), rows = __builtin_amdgcn_readlane(lane_off, e + 1) - b;
    const BigExpertTiles x = big_expert_tiles(rows, BM, false, balance);
    if (in_main) {
      const int units = x.main * n_tiles;
      if (!found && u < units) {
        const int ntile = u / max(x.main, 1), s = u - ntile * x.main;
        out.e = e;
        out.ntile = ntile;
        if (x.even) {
          out.row_begin = b + (int)((int64_t)rows * s / x.main);
          out.row_end = b + (int)((int64_t)rows * (s + 1) / x.main);
        } else {
          out.row_begin = b + s * BM;
          out.row_end = out.row_begin + BM;
        }
        found = true;
      }
      if (!found) u -= units;
    } else if (in_partial && x.partial) {
      if (!found && p_s == 0) {
        out.e = e;
        out.ntile = p_ntile;
        out.row_begin = b + rows / BM * BM;
        out.row_end = b + rows;
        found = true;
      }
      --p_s;
    }
  }
  return found;
}

// One workgroup per CU walks its XCD's unit list as one uninterrupted stream of K stages: the loads run D - 1 stages
// ahead of the MFMAs across unit boundaries, so a new unit's first operands are already in LDS when the previous unit's
// results are being written, and the pipeline is filled once per launch instead of once per unit (a workgroup per unit
// spent a fifth of its time on its own start: launch, tile lookup, first loads).  Token rows are read in sorted order
// without a gather (p.perm must be NULL: the quantising pass in front of the gate/up launch writes the rows grouped by
// expert), so that a unit's operand addresses are arithmetic on its table entry and nothing has to be fetched to start it.
template <typename T, int MODE>
__global__ void __launch_bounds__(512, 1)
grouped_fp8_ws_kernel(F8Args args) {
  constexpr int BN = 256, BM = 256, KS = 64;      // K samples (= bytes per row) per stage
  constexpr int WSTAGE = BN * KS, XSTAGE = BM * KS;  // bytes
  constexpr int STAGE = WSTAGE + XSTAGE, D = 5;   // stages in LDS
  constexpr int LOADS = 4;                        // LDS-direct loads per wavefront and stage: 2 weight pieces + 2 x 16 token rows
  constexpr int kBalance = 1;
  extern __shared__ __align__(16) uint8_t lds8[];
  const GemmParams& p = args.p;
  const int n_tiles = args.n_tiles;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int xcd = blockIdx.x & 7, wg = blockIdx.x >> 3, wgs = args.wgs_per_xcd;
  const int E = p.offsets ? p.E : 1;
  const int lane_off = p.offsets ? big_lane_offsets(p) : (lane == 1 ? (int)p.fixed_rows : 0);
  const int nst = (int)(p.kred >> 6);
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)lds8);
  const uint32_t w_lds = lds0 + 2 * wave * 1024, x_lds = lds0 + WSTAGE + 32 * wave * KS;
  const uint32_t lane16 = lane * 16;
  // bytes from one K stage of a token row to the next: 64 in a plain row, a whole block of rows in the blocked layout
  const uint32_t x_stage_bytes = p.a_block_rows ? (uint32_t)(p.a_block_rows * KS) : (uint32_t)KS;

  // ---- operands: lane (r, h) supplies row r, samples 32 h .. 32 h + 31 ------------------------------------
  const int wn = wave & 1, wm = wave >> 1;
  const int r32 = lane & 31, h32 = lane >> 5;
  // weight row r of a 32-row block: piece r / 16, lane position 16 g + r % 16 for g = 2 h, 2 h + 1
  const uint8_t* const a_rd = lds8 + (MODE == MODE_GATEUP ? wn * 4 : wn * 8) * 1024 + (r32 >> 4) * 1024 + ((32 * h32 + (r32 & 15)) << 4);
  const int xrow = wm * 64 + r32;
  const uint8_t* const b_rd = lds8 + WSTAGE + xrow * KS;
  const int bu0 = x_unit(xrow, 2 * h32) << 4, bu1 = x_unit(xrow, 2 * h32 + 1) << 4;  // rows xrow and xrow + 32 swizzle alike
  floatx16_t acc[4][2];

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

  // ---- epilogue: scale by the activations' reciprocal scale times the weights' scale ---------------------
  const float xsc = p.x_scale[0];
  const float out_rs = p.out_scale ? p.out_scale[0] : 0.0f;
  // 1 / out_rs once; per element q = v * inv refined by one residual step (fma(-q, rs, v) * inv + q), which is the
  // correctly rounded quotient except in rare last-bit cases that the following rounding to T absorbs
  const float out_inv = p.out_scale ? __builtin_amdgcn_rcpf(out_rs) : 0.0f;
  auto epilogue = [&](auto tj_tag, auto act_tag, const F8Unit& un, int rpg, int my_rows) __attribute__((always_inline)) {
    constexpr int tj = decltype(tj_tag)::value;
    constexpr int ACT = decltype(act_tag)::value;
    const float s0 = xsc * reinterpret_cast<const float*>(p.w0.d)[p.w0.d_count > 1 ? un.e : 0];
    const float s1 = MODE == MODE_GATEUP ? xsc * reinterpret_cast<const float*>(p.w1.d)[p.w1.d_count > 1 ? un.e : 0] : 0.0f;
    if (tj * 32 + r32 < my_rows) {
      const int64_t orow_i = out_row(p, un.row_begin + wm * rpg + tj * 32 + r32);
      const int64_t orow = orow_i * p.ldo;
      if (MODE == MODE_GATEUP) {
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
          for (int b = 0; b < 4; ++b) {  // four consecutive features per 8-row band of the 32 x 32 result
            const int64_t col = (int64_t)un.ntile * (BN / 2) + wn * 64 + ti * 32 + 8 * b + 4 * h32;
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
              const int64_t at = p.out_block_rows ? ((col >> 6) * p.out_block_rows + orow_i) * KS + (col & 63) : orow + col;
              *reinterpret_cast<int*>(reinterpret_cast<uint8_t*>(p.out) + at) = qv;
            } else {
              *reinterpret_cast<uint2*>(reinterpret_cast<T*>(p.out) + orow + col) = gateup_quad<T, ACT>(gq, uq);
            }
          }
      } else {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const int64_t col = (int64_t)un.ntile * BN + wn * 128 + ti * 32 + 8 * b + 4 * h32;
            const floatx16_t& c = acc[ti][tj];
            *reinterpret_cast<uint2*>(reinterpret_cast<T*>(p.out) + orow + col) =
                make_uint2(pack2<T>(c[4 * b] * s0, c[4 * b + 1] * s0), pack2<T>(c[4 * b + 2] * s0, c[4 * b + 3] * s0));
          }
      }
    }
  };
  auto epilogues = [&](auto both_tag, const F8Unit& un, int rpg, int my_rows) __attribute__((always_inline)) {
    constexpr bool BOTH = decltype(both_tag)::value;
    if (MODE == MODE_DOWN || p.act == STMOE_ACT_SILU) {
      epilogue(F8Int<0>{}, EpiAct<STMOE_ACT_SILU>{}, un, rpg, my_rows);
      if constexpr (BOTH) epilogue(F8Int<1>{}, EpiAct<STMOE_ACT_SILU>{}, un, rpg, my_rows);
    } else {
      epilogue(F8Int<0>{}, EpiAct<STMOE_ACT_GELU_ERF>{}, un, rpg, my_rows);
      if constexpr (BOTH) epilogue(F8Int<1>{}, EpiAct<STMOE_ACT_GELU_ERF>{}, un, rpg, my_rows);
    }
  };
  // Rows per token-row group of 64 LDS rows: the rows of a partial tile are spread over the four groups in multiples of 16.
  auto rows_per_group = [](int rows_here) { return min(64, ((rows_here + 3) / 4 + 15) / 16 * 16); };

  // ---- the workgroup's units, up to 64 at a time -----------------------------------------------------------
  // Round r of the walk takes the item of the XCD's list at place (wg + r (wgs / 2 + 1)) mod wgs of that round (see
  // grouped_mfma_ws_kernel: neighbouring items differ systematically in cost and a workgroup that kept its place in every
  // round would collect one kind).  Lane r of the table holds round r's unit.
  for (int round0 = 0;; round0 += 64) {
    F8Unit mine;
    const int round = round0 + lane;
    const int place = (wg + round * ((wgs >> 1) + 1)) % wgs;
    const bool have = f8_unit_of_lane(lane_off, E, BM, n_tiles, xcd, round * wgs + place, kBalance, mine);
    // (the items of later rounds come later in the list: the lanes that hold a unit are lanes 0 .. n_units - 1)
    const int n_units = __builtin_popcountll(__ballot(have));
    if (n_units == 0) return;
    const int t_en = mine.e | (mine.ntile << 8), t_rb = mine.row_begin, t_re = mine.row_end;
    auto unit_at = [&](int i) {
      F8Unit un;
      const int en = __builtin_amdgcn_readlane(t_en, i);
      un.e = en & 0xff;
      un.ntile = en >> 8;
      un.row_begin = __builtin_amdgcn_readlane(t_rb, i);
      un.row_end = __builtin_amdgcn_readlane(t_re, i);
      return un;
    };
    const int total = n_units * nst;  // K stages of this batch of units

    // ---- the load side: stage `gl` of the batch = stage `sl` of unit `ul` ------------------------------------
    const uint8_t* wq[2] = {nullptr, nullptr};
    uint32_t xoff[2] = {0, 0};
    int ul = -1, sl = nst, gl = 0;
    auto issue_next = [&]() __attribute__((always_inline)) {
      if (sl == nst) {  // first stage of the next unit: its operand addresses
        ++ul;
        sl = 0;
        const F8Unit un = unit_at(ul);
        const int rows_here = un.row_end - un.row_begin, rpg = rows_per_group(rows_here);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int rtl = 2 * wave + j;  // row tile of 16 inside the 256 weight rows of the stage
          int64_t row0;
          const WeightView* wv;
          if (MODE == MODE_GATEUP) {
            const bool up = rtl >= BN / 32;
            wv = up ? &p.w1 : &p.w0;
            row0 = (int64_t)un.e * wv->rows + (int64_t)un.ntile * (BN / 2) + (rtl % (BN / 32)) * 16;
          } else {
            wv = &p.w0;
            row0 = (int64_t)un.e * wv->rows + (int64_t)un.ntile * BN + rtl * 16;
          }
          const uint64_t addr = reinterpret_cast<uint64_t>(wv->qs + (row0 >> 4) * (p.kred >> 6) * 1024);  // K block 0 of the row tile
          // wave-uniform by construction; say so to the compiler (the address goes into scalar registers)
          // (the builtin returns a signed int: go through uint32_t, or the low half sign-extends into the high one)
          const uint32_t addr_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)addr);
          const uint32_t addr_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(addr >> 32));
          wq[j] = reinterpret_cast<const uint8_t*>((uint64_t)addr_lo | ((uint64_t)addr_hi << 32));
          // token rows: lane l fills LDS row 32 wave + 16 j + l / 4 with the 16 bytes that belong at position l % 4
          // (x_unit is an involution: position -> logical unit); LDS rows without a tile row re-read a valid one
          const int lr = 32 * wave + 16 * j + (lane >> 2);
          const int r = min((lr >> 6) * rpg + min(lr & 63, rpg - 1), rows_here - 1);
          xoff[j] = (uint32_t)((int64_t)(un.row_begin + r) * (p.a_block_rows ? KS : p.lda) + (x_unit(lr, lane & 3) << 4));
        }
      }
      const uint32_t slot = (uint32_t)(gl % D) * STAGE;
      vm_load16_to_lds(wq[0], lane16 + (uint32_t)sl * 1024, w_lds + slot);
      vm_load16_to_lds(wq[1], lane16 + (uint32_t)sl * 1024, w_lds + slot + 1024);
      vm_load16_to_lds(p.a, xoff[0] + (uint32_t)sl * x_stage_bytes, x_lds + slot);
      vm_load16_to_lds(p.a, xoff[1] + (uint32_t)sl * x_stage_bytes, x_lds + slot + 16 * KS);
      ++sl;
      ++gl;
    };

    // every wavefront loads its share of every stage and meets every barrier, with or without token rows of its own
#pragma unroll 1
    for (int st = 0; st < min(D - 1, total); ++st) issue_next();
    int slot = 0, g = 0;
#pragma unroll 1
    for (int u = 0; u < n_units; ++u) {
      const F8Unit un = unit_at(u);
      const int rows_here = un.row_end - un.row_begin, rpg = rows_per_group(rows_here);
      const int my_rows = min(rpg, rows_here - wm * rpg);
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int q = 0; q < 16; ++q) acc[a][b][q] = 0.0f;
#pragma unroll 1
      for (int st = 0; st < nst; ++st, ++g) {
        // the loads of the D - 2 stages after this one may still be in flight when this stage is needed; the batch's
        // last stages have nothing behind them to issue
        if (g + D - 1 < total) {
          vm_wait<(D - 2) * LOADS>();
          __syncthreads();  // everybody's loads of this stage have landed; everybody is done with the stage before
          issue_next();     // into the slot of the stage before
        } else {
          vm_wait<0>();
          __syncthreads();
        }
        if (my_rows > 32) compute(F8Int<1>{}, slot);
        else if (my_rows > 0) compute(F8Int<0>{}, slot);
        slot = slot == D - 1 ? 0 : slot + 1;
      }
      if (my_rows > 32) epilogues(F8Int<1>{}, un, rpg, my_rows);
      else if (my_rows > 0) epilogues(F8Int<0>{}, un, rpg, my_rows);
    }
    // (a further batch, if the workgroup has more than 64 units, starts with empty LDS stages: every load has landed and
    // the last barrier is passed by all before the next stage 0 is written... after one more barrier)
    __syncthreads();
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
  // one workgroup per CU (it takes all of the CU's LDS), fewer when an XCD's list cannot be longer than that
  const int per_xcd = std::min(kBigCusPerXcd, big_grid(n_tiles, m_slots, false) / 8);
  kern<<<dim3((unsigned)(8 * per_xcd)), 512, lds_bytes, st>>>(F8Args{p, n_tiles, per_xcd});
  return check_launch("grouped_fp8_ws");
}

// act_dtype: dtype of the results; activations are e4m3fn bytes (p.a, p.lda in bytes), weights packed fp8.
int launch_fp8_ws(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0) return STMOE_OK;
  if (!p.x_scale) return set_error(STMOE_ERR_NULL, "fp8 ws kernel: activation scale is NULL");
  if (wtag != WF_FP8_F32D_P) return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: needs packed fp8 weights with fp32 scale(s)");
  if (p.offsets && p.E >= 64) return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: at most 63 experts");
  if (p.perm) return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: token rows must be grouped by expert already (no gather)");
  if (p.kred % 256 != 0 || p.lda % 16 != 0 || p.ldo % 4 != 0 || p.n_out % (mode == MODE_GATEUP ? 128 : 256) != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: needs K %% 256 == 0 and output features in whole tiles");
  if (std::max(max_rows, (int64_t)p.a_block_rows) * p.kred >= (int64_t)1 << 32)
    return set_error(STMOE_ERR_UNSUPPORTED, "fp8 ws kernel: activations span 4 GB or more");
  if (act_dtype == STMOE_F16)
    return mode == MODE_GATEUP ? launch_fp8_ws_m<f16_t, MODE_GATEUP>(p, max_rows, st) : launch_fp8_ws_m<f16_t, MODE_DOWN>(p, max_rows, st);
  if (act_dtype == STMOE_BF16)
    return mode == MODE_GATEUP ? launch_fp8_ws_m<bf16_t, MODE_GATEUP>(p, max_rows, st) : launch_fp8_ws_m<bf16_t, MODE_DOWN>(p, max_rows, st);
  return set_error(STMOE_ERR_DTYPE, "fp8 ws kernel: result dtype %d", act_dtype);
}

}  // namespace stmoe
