// Prefill kernel: grouped projection on the matrix cores with a 256 x 256 workgroup tile.
//
//   workgroup = 8 wavefronts (2 x 4), each owning 128 weight rows x 64 token rows of the tile
//               (GATEUP: 64 gate rows + the same 64 up rows, so the gated product is formed in registers);
//               the 256 x 256 fp32 accumulators are half of the CU's register file, the largest tile that fits
//   K step 64.  LDS (160 KB): two stages of dequantised weights (16-bit, 32 KB each) and three stages of token rows
//               (32 KB each); rows are 128 bytes, XOR-swizzled in 16-byte units, one barrier per K step
//   producer: every wavefront loads whole 1 KB pieces of the packed weight order (prepack.hip) into registers two
//             K steps ahead, dequantises them and writes 16-bit rows into the next weight stage; token rows,
//             gathered through the dispatch permutation, go from global memory straight into LDS
//             (global_load_lds_dwordx4), also two K steps ahead, without passing through registers
//   consumer: v_mfma_f32_16x16x32, weight rows as the "A" rows, token rows as the "B" columns; per K=32 step a
//             wavefront reads 8 + 4 operand fragments from LDS for 32 MFMAs
//   the two wavefronts of a SIMD run producer and consumer halves of a K step in opposite orders, so that one
//             converts and stores while the other feeds the matrix pipe
//   ragged tiles: wavefronts whose 64 token rows are all past the end of the expert's rows skip their MFMAs
//   scheduling: see big_tile_id (equal shares per XCD, partial token tiles last).
//
// The direct loads are written as inline assembly: given the builtin, the compiler waits for every outstanding load
// before each LDS read, which would undo the prefetch.  Their completion is therefore awaited by hand before the
// barrier of the K step that precedes their use (s_waitcnt vmcnt(n): loads return in issue order, and per K step a
// wavefront issues XPIECES token loads followed by WLOADS weight loads, one 16-byte and one 2-byte load per piece).
// The compiler's own waits for the weight registers do not count the hidden token loads and can only be stricter.
#include "ffn_mfma_common.h"

namespace stmoe {

template <int V> struct BigSet { static constexpr int value = V; };
struct BigTagOn { static constexpr bool value = true; };
struct BigTagOff { static constexpr bool value = false; };

// WN x WM wavefronts; each owns 128 weight rows x 64 token rows (32 accumulator tiles = 128 registers, which
// leaves the register allocator room: a 128 x 128 wavefront tile fills all 256 accumulation registers and made
// the compiler shuffle accumulators between register files around every MFMA).
//
// TI: 16-row weight fragments per wavefront (8: the 128 x 64 wavefront tile above).  The narrow form (TI = 2, 2 x 4
// wavefronts: 64 weight rows x 256 token rows per workgroup, 32 x 64 per wavefront) is for a single matrix with a few
// hundred rows: 256 rows of a [14336, 4096] matrix are 56 tiles of 256 x 256 but 224 of 64 x 256, which fill the CUs
// without cutting the reduction (no fp32 partial tiles, no workspace).  A K step then has only four weight pieces: the
// first four wavefronts load and convert one each, the others only send token rows.
template <typename T, int WF, int MODE, int WN, int WM, int STAGES, int TI>
__global__ void __launch_bounds__(64 * WN * WM, 1)
grouped_mfma_big_kernel(GemmParams p, int n_tiles) {
  constexpr int NTHR = 64 * WN * WM;
  constexpr int WROWS = 16 * TI;         // weight rows per wavefront (GATEUP: half gate, half up)
  constexpr int BN = WROWS * WN;         // weight rows per workgroup tile (GATEUP: BN/2 gate + BN/2 up)
  constexpr int BM = 64 * WM;            // token rows per workgroup tile
  static_assert(STAGES == 2, "two weight stages and three token stages");
  static_assert(TI % 2 == 0, "gate and up fragments come in pairs");
  constexpr int WSTAGE = BN * BIG_LS, XSTAGE = BM * BIG_LS;  // elements
  constexpr int NPIECES = BN / 16;                                      // packed weight pieces per K step
  constexpr int WPIECES = NPIECES >= WN * WM ? NPIECES / (WN * WM) : 1;  // per wavefront that loads weights
  constexpr int WLOADERS = NPIECES / WPIECES;                           // wavefronts 0 .. WLOADERS - 1 load weights
  constexpr int XPIECES = BM * 8 / NTHR;          // 16-byte token pieces per thread per K step
  constexpr int XROWS_PER_PASS = NTHR / 8;
  static_assert(WPIECES >= 1 && XPIECES >= 1 && WPIECES * WLOADERS == NPIECES && WLOADERS <= WN * WM, "tile too small for the thread count");
  extern __shared__ __align__(16) uint16_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave / WM, wm = wave % WM;

  BigTile tile;
  if (!big_tile_id(p, BM, n_tiles, false, tile)) return;
  const int e = tile.e, row_begin = tile.row_begin, row_end = tile.row_end, ntile = tile.ntile;
  const int rows_here = row_end - row_begin;

  // ---- producer assignment ---------------------------------------------------------------------------
  const int g = lane >> 4, n_in = lane & 15;
  BigAddr<WF> waddr[WPIECES];
#pragma unroll
  for (int j = 0; j < WPIECES; ++j) {
    const int rtl = (wave < WLOADERS ? wave : 0) * WPIECES + j;  // row tile (16 rows) inside the workgroup tile
    int64_t row0;                         // first global row of the row tile (expert-stacked)
    const WeightView* wv;
    if (MODE == MODE_GATEUP) {
      const bool up = rtl >= BN / 32;
      wv = up ? &p.w1 : &p.w0;
      row0 = (int64_t)e * wv->rows + (int64_t)ntile * (BN / 2) + (rtl % (BN / 32)) * 16;
    } else {
      wv = &p.w0;
      row0 = (int64_t)e * wv->rows + (int64_t)ntile * BN + rtl * 16;
    }
    waddr[j].init(*wv, row0 >> 4, e, lane, p.kred);
  }
  // Token rows past the end of the expert's rows are clamped to its last row: every output row depends on its
  // own token row only and those outputs are never stored, so no zero fill (and no branch) is needed.
  // A direct load puts lane l's 16 bytes at (wave-uniform LDS address) + 16*l, i.e. 8 lanes fill one 128-byte row
  // in order; the XOR swizzle of the row is therefore applied to the source: LDS unit j of row r receives global
  // unit j ^ (r & 7).
  uint32_t xoff[XPIECES];  // byte offsets from p.a (the host checks that the activations span less than 4 GB)
#pragma unroll
  for (int j = 0; j < XPIECES; ++j) {
    const int lr = (tid >> 3) + XROWS_PER_PASS * j;  // LDS row
    const int r = min(lr, rows_here - 1);
    const int i = row_begin + r;
    const int64_t src = p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i;
    xoff[j] = (uint32_t)((src * p.lda + (((tid & 7) ^ (lr & 7)) << 3)) * 2);
  }

  uint16_t* const Wbase = lds;               // [2][BN][64]
  uint16_t* const Xbase = lds + 2 * WSTAGE;  // [3][BM][64]
  const uint32_t lds_addr0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)lds);
  // LDS byte address of the 8 rows this wavefront fills in pass 0 of token stage 0
  const uint32_t x_lds0 = __builtin_amdgcn_readfirstlane(lds_addr0 + (2 * WSTAGE + wave * 8 * BIG_LS) * 2);

  // LDS addressing: rows handled by a lane differ from its base row by multiples of 16, so the swizzle term
  // (unit ^ (row & 7)) depends on the lane (and the K half) only, and everything else is a compile-time offset.
  const int sw = n_in & 7;
  uint16_t* const w_st = Wbase + (wave * WPIECES * 16 + n_in) * BIG_LS;  // producer: first row tile of the wavefront
  const int st_swz0 = ((2 * g) ^ sw) << 3, st_swz1 = ((2 * g + 1) ^ sw) << 3;
  const uint16_t* a_rd[2];  // consumer, K half ks: weight row (wavefront base + n_in), unit ks*4 + g
  const uint16_t* b_rd[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const int u = ((ks * 4 + g) ^ sw) << 3;
    a_rd[ks] = Wbase + ((MODE == MODE_GATEUP ? wn * (WROWS / 2) : wn * WROWS) + n_in) * BIG_LS + u;
    b_rd[ks] = Xbase + (wm * 64 + n_in) * BIG_LS + u;
  }

  BigPiece<WF> wreg[2][WPIECES];
  constexpr int WLOADS = BigPiece<WF>::LOADS * WPIECES;  // vector-memory instructions of one load_w
  auto load_w = [&](auto set_tag, int64_t kt) {
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int j = 0; j < WPIECES; ++j) {
      // plain (cacheable) loads: the token tiles of one (expert, feature tile) run back to back on one XCD and
      // share the weight tile in its L2
      wreg[SET][j].load(waddr[j], kt);
    }
  };
  auto store_w = [&](auto set_tag) {  // registers of set s hold a K step of parity s and go to weight stage s
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int j = 0; j < WPIECES; ++j) {
      uint32_t v[8];
      wreg[SET][j].template convert<T>(waddr[j], v);
      uint16_t* row = w_st + SET * WSTAGE + j * 16 * BIG_LS;  // constants fold into the instruction's offset field
      *reinterpret_cast<u32x4_t*>(row + st_swz0) = (u32x4_t){v[0], v[1], v[2], v[3]};
      *reinterpret_cast<u32x4_t*>(row + st_swz1) = (u32x4_t){v[4], v[5], v[6], v[7]};
    }
  };
  auto load_x = [&](int xstage, int64_t kt) {
#pragma unroll
    for (int j = 0; j < XPIECES; ++j)
      vm_load16_to_lds(p.a, xoff[j] + (uint32_t)kt * (BIG_BK * 2), x_lds0 + (uint32_t)((xstage * XSTAGE + XROWS_PER_PASS * j * BIG_LS) * 2));
  };

  // ---- consumer -----------------------------------------------------------------------------------------
  // wavefront tile: GATEUP gate rows wn*64..+63 (LDS rows wn*64..) and the same up rows (LDS rows BN/2 + wn*64..);
  //                 DOWN rows wn*128..+127.  Token rows wm*64..+63.
  floatx4_t acc[TI][4];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
  const bool active = rows_here > wm * 64;  // wavefronts whose token rows are all past the end skip their MFMAs

  auto compute = [&](auto parity_tag, int xstage, int ks) {
    constexpr int PAR = decltype(parity_tag)::value;
    const uint16_t* bp = b_rd[ks] + xstage * XSTAGE;
    u32x4_t bf[4];
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) bf[tj] = *reinterpret_cast<const u32x4_t*>(bp + tj * 16 * BIG_LS);
#pragma unroll
    for (int ti = 0; ti < TI; ++ti) {
      const int row_off = MODE == MODE_GATEUP ? (ti < TI / 2 ? 0 : BN / 2) + (ti % (TI / 2)) * 16 : ti * 16;
      const u32x4_t af = *reinterpret_cast<const u32x4_t*>(a_rd[ks] + PAR * WSTAGE + row_off * BIG_LS);
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) acc[ti][tj] = mfma16b<T>(af, bf[tj], acc[ti][tj]);
    }
  };

  const int64_t nkt = p.kred >> 6;
  // K step kt reads weight stage kt % 2 and token stage kt % 3.  During step kt a wavefront
  //   converts and stores the weights of step kt + 1 (registers loaded during step kt - 2),
  //   issues the token loads of step kt + 2 (into the stage last read in step kt - 1),
  //   issues the weight loads of step kt + 3 (into the registers just freed),
  // so every global load has about two K steps to arrive.  ACTIVE and LATE are compile-time tags so that a K step is
  // one straight-line block; LATE wavefronts produce before their MFMAs, the others after.
  // STEADY steps (kt + 3 < nkt) contain no branch, so two of them form one basic block and the compiler's waits for
  // the weight registers stay exact; the last steps run the same code with the loads guarded.
  auto k_step = [&](auto active_tag, auto late_tag, auto wload_tag, auto parity_tag, auto steady_tag, int64_t kt, int xs) {
    constexpr bool ACTIVE = decltype(active_tag)::value;
    constexpr bool LATE = decltype(late_tag)::value;
    constexpr bool WLOAD = decltype(wload_tag)::value;  // this wavefront is one of those that load weight pieces
    constexpr int PAR = decltype(parity_tag)::value;  // kt % 2
    constexpr bool STEADY = decltype(steady_tag)::value;
    using Next = BigSet<PAR ^ 1>;
    auto produce = [&]() {
      // the compiler's wait for the registers of step kt + 1 also covers the older token loads of that step
      if (WLOAD && (STEADY || kt + 1 < nkt)) store_w(Next{});
      if (STEADY || kt + 2 < nkt) load_x(xs >= 1 ? xs - 1 : 2, kt + 2);
      if (WLOAD && (STEADY || kt + 3 < nkt)) load_w(Next{}, kt + 3);
    };
    // scheduling fences: without them the compiler hoists the LDS reads of both K halves and the next step's
    // conversions across the whole block and runs out of registers
    // (the narrow form has registers to spare: there the compiler may read the second K half's operands under the first
    // half's MFMAs)
    constexpr bool FENCED = TI >= 8;
    if constexpr (LATE) {
      produce();
      if (FENCED) __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (ACTIVE) {
      compute(parity_tag, xs, 0);
      if (FENCED) __builtin_amdgcn_sched_barrier(0);
      compute(parity_tag, xs, 1);
      if (FENCED) __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!LATE) {
      produce();
      if (FENCED) __builtin_amdgcn_sched_barrier(0);
    }
    // the token loads of step kt + 1 were issued during step kt - 1, before that step's weight loads; in steady state
    // exactly those weight loads and this step's token and weight loads are younger
    // (a wavefront without weight pieces has only this step's token loads behind them)
    if constexpr (STEADY) vm_wait<(WLOAD ? 2 * WLOADS : 0) + XPIECES>();
    else vm_wait<0>();
    __syncthreads();
  };
  auto main_loop = [&](auto active_tag, auto late_tag, auto wload_tag) {
    constexpr bool WLOAD = decltype(wload_tag)::value;
    if (WLOAD) load_w(BigSet<0>{}, 0);
    load_x(0, 0);
    if (nkt > 1) {
      if (WLOAD) load_w(BigSet<1>{}, 1);
      load_x(1, 1);
    }
    vm_wait<0>();
    if (WLOAD) store_w(BigSet<0>{});
    if (WLOAD && nkt > 2) load_w(BigSet<0>{}, 2);
    __syncthreads();  // everything but the last weight loads has arrived
    int xs = 0;       // kt % 3
    int64_t kt = 0;
    for (; kt + 4 < nkt; kt += 2) {
      k_step(active_tag, late_tag, wload_tag, BigSet<0>{}, BigTagOn{}, kt, xs);
      xs = xs == 2 ? 0 : xs + 1;
      k_step(active_tag, late_tag, wload_tag, BigSet<1>{}, BigTagOn{}, kt + 1, xs);
      xs = xs == 2 ? 0 : xs + 1;
    }
    for (; kt < nkt; kt += 2) {
      k_step(active_tag, late_tag, wload_tag, BigSet<0>{}, BigTagOff{}, kt, xs);
      xs = xs == 2 ? 0 : xs + 1;
      if (kt + 1 < nkt) {
        k_step(active_tag, late_tag, wload_tag, BigSet<1>{}, BigTagOff{}, kt + 1, xs);
        xs = xs == 2 ? 0 : xs + 1;
      }
    }
  };
  // The two wavefronts that share a SIMD (w and w + 4) run the K step in opposite orders: one converts and stores
  // the next stage while the other feeds the matrix pipe, then they swap, so the vector-ALU and LDS-write work of
  // the producer overlaps MFMAs instead of leaving the matrix pipe idle between barriers.
  const bool late = (wave & 4) != 0;
  if constexpr (WLOADERS == WN * WM) {
    if (active) {
      if (late) main_loop(BigTagOn{}, BigTagOn{}, BigTagOn{});
      else main_loop(BigTagOn{}, BigTagOff{}, BigTagOn{});
    } else {
      main_loop(BigTagOff{}, BigTagOff{}, BigTagOn{});
    }
  } else {
    // narrow form: the wavefronts that convert weight pieces do so before their MFMAs, the others go straight to theirs
    static_assert(WLOADERS == 4 && WN * WM == 8, "wavefronts 0-3 load weights, one per SIMD");
    if (wave < WLOADERS) {
      if (active) main_loop(BigTagOn{}, BigTagOn{}, BigTagOn{});
      else main_loop(BigTagOff{}, BigTagOff{}, BigTagOn{});
    } else {
      if (active) main_loop(BigTagOn{}, BigTagOff{}, BigTagOff{});
      else main_loop(BigTagOff{}, BigTagOff{}, BigTagOff{});
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------------
  auto store_gateup = [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    const FakeQuant fq = fq_scale(p);
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      const int r = wm * 64 + tj * 16 + n_in;
      if (r < rows_here) {
        T* orow = reinterpret_cast<T*>(p.out) + out_row(p, row_begin + r) * p.ldo + (int64_t)ntile * (BN / 2) + wn * (WROWS / 2) + 4 * g;
#pragma unroll
        for (int ti = 0; ti < TI / 2; ++ti) {
          const float gq[4] = {acc[ti][tj][0], acc[ti][tj][1], acc[ti][tj][2], acc[ti][tj][3]};
          const float uq[4] = {acc[ti + TI / 2][tj][0], acc[ti + TI / 2][tj][1], acc[ti + TI / 2][tj][2], acc[ti + TI / 2][tj][3]};
          *reinterpret_cast<uint2*>(orow + ti * 16) = gateup_quad<T, ACT>(gq, uq, fq);
        }
      }
    }
  };
  if (MODE == MODE_GATEUP) {
    if (p.act == STMOE_ACT_SILU) store_gateup(EpiAct<STMOE_ACT_SILU>{});
    else store_gateup(EpiAct<STMOE_ACT_GELU_ERF>{});
  } else {
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      const int r = wm * 64 + tj * 16 + n_in;
      if (r < rows_here) {
        T* orow = reinterpret_cast<T*>(p.out) + out_row(p, row_begin + r) * p.ldo;
#pragma unroll
        for (int ti = 0; ti < TI; ++ti)
          *reinterpret_cast<uint2*>(orow + (int64_t)ntile * BN + wn * WROWS + ti * 16 + 4 * g) =
              make_uint2(pack2<T>(acc[ti][tj][0], acc[ti][tj][1]), pack2<T>(acc[ti][tj][2], acc[ti][tj][3]));
      }
    }
  }
}

template <typename T, int WF, int MODE, int WN, int WM, int STAGES, int TI = 8>
static int launch_big_m(const GemmParams& p, int64_t max_rows, hipStream_t st) {
  constexpr int BN = 16 * TI * WN, BM = 64 * WM;
  constexpr size_t lds_bytes = (size_t)(2 * BN + 3 * BM) * BIG_LS * 2;
  static std::atomic<uint64_t> lds_ready{0};
  auto kern = grouped_mfma_big_kernel<T, WF, MODE, WN, WM, STAGES, TI>;
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ready, "mfma big kernel")) return rc;
  const int n_tiles = (int)(MODE == MODE_GATEUP ? p.n_out / (BN / 2) : p.n_out / BN);
  const int experts = p.offsets ? p.E : 1;
  const int m_slots = (int)((max_rows + BM - 1) / BM) + experts;
  kern<<<dim3((unsigned)big_grid(n_tiles, m_slots, false)), 64 * WN * WM, lds_bytes, st>>>(p, n_tiles);
  return check_launch("grouped_mfma_big");
}

#ifndef STMOE_BIG_WN
#define STMOE_BIG_WN 2
#endif
#ifndef STMOE_BIG_WM
#define STMOE_BIG_WM 4
#endif
#ifndef STMOE_BIG_STAGES
#define STMOE_BIG_STAGES 2
#endif
template <typename T, int WF>
static int launch_big_t(int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (mode == MODE_GATEUP) return launch_big_m<T, WF, MODE_GATEUP, STMOE_BIG_WN, STMOE_BIG_WM, STMOE_BIG_STAGES>(p, max_rows, st);
  return launch_big_m<T, WF, MODE_DOWN, STMOE_BIG_WN, STMOE_BIG_WM, STMOE_BIG_STAGES>(p, max_rows, st);
}

int launch_mfma_big(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0) return STMOE_OK;
  if (p.offsets && p.E >= 64) return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: at most 63 experts");
  if (wtag != WF_Q8_0_P)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: needs weights in the packed Q8_0 order");
  if (p.kred % 256 != 0 || p.lda % 8 != 0 || p.ldo % 4 != 0 || p.n_out % (mode == MODE_GATEUP ? 64 * STMOE_BIG_WN : 128 * STMOE_BIG_WN) != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: needs K %% 256 == 0 and output features in whole tiles");
  {
    // token rows are addressed with 32-bit byte offsets from the activation base
    const int64_t src_rows = p.perm ? (max_rows + p.k_top - 1) / p.k_top : max_rows;
    if (src_rows * p.lda * 2 >= (int64_t)1 << 32)
      return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: activations span 4 GB or more");
  }
  if (act_dtype == STMOE_F16) return launch_big_t<f16_t, WF_Q8_0_P>(mode, p, max_rows, st);
  if (act_dtype == STMOE_BF16) return launch_big_t<bf16_t, WF_Q8_0_P>(mode, p, max_rows, st);
  return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: activation dtype %d", act_dtype);
}

// The narrow form: 64 weight rows x 256 token rows per workgroup (see the kernel's head).
#ifndef STMOE_NARROW_TI
#define STMOE_NARROW_TI 2
#endif
template <typename T, int WF>
static int launch_narrow_t(int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (mode == MODE_GATEUP) return launch_big_m<T, WF, MODE_GATEUP, 2, 4, 2, STMOE_NARROW_TI>(p, max_rows, st);
  return launch_big_m<T, WF, MODE_DOWN, 2, 4, 2, STMOE_NARROW_TI>(p, max_rows, st);
}

int launch_mfma_narrow(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (max_rows == 0) return STMOE_OK;
  if (p.offsets && p.E >= 64) return set_error(STMOE_ERR_UNSUPPORTED, "mfma narrow kernel: at most 63 experts");
  if (p.kred % 256 != 0 || p.lda % 8 != 0 || p.ldo % 4 != 0 || p.n_out % (mode == MODE_GATEUP ? 16 * STMOE_NARROW_TI : 32 * STMOE_NARROW_TI) != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma narrow kernel: needs K %% 256 == 0 and output features in whole tiles");
  {
    const int64_t src_rows = p.perm ? (max_rows + p.k_top - 1) / p.k_top : max_rows;
    if (src_rows * p.lda * 2 >= (int64_t)1 << 32)
      return set_error(STMOE_ERR_UNSUPPORTED, "mfma narrow kernel: activations span 4 GB or more");
  }
  if (act_dtype == STMOE_F16) {
    if (wtag == WF_Q8_0_P) return launch_narrow_t<f16_t, WF_Q8_0_P>(mode, p, max_rows, st);
    if (wtag == WF_Q4_1_P) return launch_narrow_t<f16_t, WF_Q4_1_P>(mode, p, max_rows, st);
    if (wtag == WF_FP8_F32D_P) return launch_narrow_t<f16_t, WF_FP8_F32D_P>(mode, p, max_rows, st);
  } else if (act_dtype == STMOE_BF16) {
    if (wtag == WF_Q8_0_P) return launch_narrow_t<bf16_t, WF_Q8_0_P>(mode, p, max_rows, st);
    if (wtag == WF_Q4_1_P) return launch_narrow_t<bf16_t, WF_Q4_1_P>(mode, p, max_rows, st);
    if (wtag == WF_FP8_F32D_P) return launch_narrow_t<bf16_t, WF_FP8_F32D_P>(mode, p, max_rows, st);
  }
  return set_error(STMOE_ERR_UNSUPPORTED, "mfma narrow kernel: packed Q8_0, Q4_1 or fp8 weights with fp16 or bf16 activations");
}

}  // namespace stmoe
