// Prefill kernel with specialised wavefronts: 256 weight rows x 256 token rows per unit, one workgroup of 12 wavefronts
// per CU that walks its XCD's list of units.
//
//   units of 129..256 token rows: 8 consumer + 4 loader wavefronts
//   consumers (wavefronts 0-7: 2 weight-row halves x 4 token-row groups): 128 weight rows x 64 token rows each (GATEUP: 64 gate + the same 64 up rows);
//             a K step is nothing but LDS operand reads and 64 MFMAs, so both consumers of a SIMD keep the matrix
//             pipe fed all the time
//   loaders   (wavefronts 8-11, one per SIMD): per K step each loads 4 packed 1 KB weight pieces into registers
//             (four K steps before they are needed), dequantises them and writes 16-bit rows into the next weight
//             stage, and issues 8 direct global->LDS loads of token rows (two K steps ahead)
//   units of at most 128 token rows: 4 consumers (wavefronts 0-3, one per SIMD, the same 128 x 64 each) + 8 loaders
//             (wavefronts 4-11, two weight pieces and two token loads each): such a unit still converts its whole weight slab
//             while its consumers have half the work, and four loaders cannot convert faster than in 2200 cycles per K step
//   LDS (160 KB): 2 weight stages + 3 token stages of 32 KB, rows of 128 bytes XOR-swizzled in 16-byte units;
//             one barrier per K step
//   registers: 12 wavefronts leave 168 per lane; the consumers hold 128 accumulators and 20 operand registers
//
//   tails:    a full token tile may take up to 16 more rows of its expert along (an absorbed tail, see big_tail_absorbed):
//             the four loaders multiply those rows themselves, each against 64 of the tile's 256 weight rows, with the
//             weight operands taken from the registers they have just converted and the token operands straight from
//             global memory (two K steps ahead, two register sets); 8 MFMAs per loader and K step, no LDS traffic
//
// All loads of the loaders are inline assembly with a wave-uniform base in scalar registers and are awaited by hand
// (see ffn_mfma_common.h); per K step a loader issues, piece by piece, WLOADS weight loads and XLOADS token loads, then
// the tail's token loads (if any), always in this order and always all of them.
#include "ffn_mfma_common.h"

namespace stmoe {

template <int V> struct WsInt { static constexpr int value = V; };

// Token of pair id `pair` = pair / k_top; the usual top-k values without the 40 instructions of an integer division.
__device__ __forceinline__ int pair_token(int pair, int k_top) {
  if (k_top == 1) return pair;
  if (k_top == 2) return pair >> 1;
  if (k_top == 4) return pair >> 2;
  if (k_top == 8) return pair >> 3;
  return pair / k_top;
}

// Which experts get equal-sized token tiles (see big_expert_tiles).
constexpr int ws_balance(int wf) { return wf == WF_Q8_0_P ? 2 : 1; }

struct WsArgs {
  GemmParams p;
  int n_tiles;
  int wgs_per_xcd;  // grid size / 8
  float* partial;
  int* tickets;  // one counter per split unit, zero at launch and zero again when the launch is over
};

// A unit that is split along the reduction is finished by whichever of its chunks is done last: every chunk writes its
// fp32 partial tile and draws a ticket (an integer atomic), and the workgroup that draws the last one adds the chunks in
// chunk order, so the sum does not depend on which workgroup that is.  One row of the partial tile (tile rows, then the
// absorbed tail's rows from BM on) per 8 threads.  DOWN: the sums; GATEUP: the gated product of the gate sums (columns
// 0..127 of the partial tile) and the up sums (columns 128..255).
static constexpr size_t kWsSlotFloats = (size_t)256 * (256 + kBigTailRows);
static constexpr int kWsTickets = 8 * kBigChunkSlotsPerXcd;
// The adding workgroup is the tail of its unit and works alone, so its loads must overlap: the chunk count is a template
// argument and a thread first issues the loads of all chunks for 64 of its row's columns (up to 16 loads of 16 bytes in
// flight per thread), then adds them.  (With the chunk count a run-time value every load waited for the one before: the
// sum of one 256-row unit took 45 us, as long as its reduction steps.)
template <typename T, int MODE, int CHUNKS>
__device__ __forceinline__ void ws_reduce_row(const GemmParams& p, const BigTile& t, const float* base, int r, int c8) {
  constexpr int BN = 256, BM = 256;
  const int rows_here = t.row_end - t.row_begin;
  int sorted_row;
  if (r < rows_here) sorted_row = t.row_begin + r;
  else if (r >= BM && r - BM < t.tail_rows) sorted_row = t.tail_begin + (r - BM);
  else return;
  base += (size_t)r * BN;
  // columns of this thread: (c8 + 8 j) * 4 for j = 0..7 (DOWN), or that gate column and its up column for j = 0..3
  auto col_of = [&](int i) { return MODE == MODE_GATEUP ? (i >> 2) * (BN / 2) + (c8 + 8 * (i & 3)) * 4 : (c8 + 8 * i) * 4; };
  T* orow = reinterpret_cast<T*>(p.out) + out_row(p, sorted_row) * p.ldo;
  const FakeQuant fq = fq_scale(p);
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    // GATEUP: j = 2 half, 2 half + 1 (i = j and 4 + j); DOWN: j = 4 half .. 4 half + 3
    floatx4_t v[4][CHUNKS];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i = MODE == MODE_GATEUP ? (q >> 1) * 4 + 2 * half + (q & 1) : 4 * half + q;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) v[q][c] = *reinterpret_cast<const floatx4_t*>(base + (size_t)c * kWsSlotFloats + col_of(i));
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int c = 1; c < CHUNKS; ++c) v[q][0] = v[q][0] + v[q][c];
    if (MODE == MODE_GATEUP) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const floatx4_t gs = v[q][0], us = v[2 + q][0];
        const float gq[4] = {gs[0], gs[1], gs[2], gs[3]}, uq[4] = {us[0], us[1], us[2], us[3]};
        uint2* dst = reinterpret_cast<uint2*>(orow + (int64_t)t.ntile * (BN / 2) + col_of(2 * half + q));
        if (p.act == STMOE_ACT_SILU) *dst = gateup_quad<T, STMOE_ACT_SILU>(gq, uq, fq);
        else *dst = gateup_quad<T, STMOE_ACT_GELU_ERF>(gq, uq, fq);
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const floatx4_t sum = v[q][0];
        *reinterpret_cast<uint2*>(orow + (int64_t)t.ntile * BN + col_of(4 * half + q)) = make_uint2(pack2<T>(sum[0], sum[1]), pack2<T>(sum[2], sum[3]));
      }
    }
  }
}
template <typename T, int MODE>
__device__ __forceinline__ void ws_reduce_unit(const GemmParams& p, const BigTile& t, const float* base, int tid) {
  constexpr int BM = 256;
  for (int r = tid >> 3; r < BM + kBigTailRows; r += 96) {
    if (t.nchunks == 2) ws_reduce_row<T, MODE, 2>(p, t, base, r, tid & 7);
    else if (t.nchunks == 3) ws_reduce_row<T, MODE, 3>(p, t, base, r, tid & 7);
    else ws_reduce_row<T, MODE, 4>(p, t, base, r, tid & 7);
  }
}
__global__ void ws_zero_tickets_kernel(int* tickets) { tickets[threadIdx.x] = 0; }

// ---- the loaders' load queue, checked at compile time --------------------------------------------------------
// A loader's loads are issued by hand and awaited with `s_waitcnt vmcnt(N)`: "at most N of my loads may still be in
// flight", the N youngest.  Each N in the kernel is written as a formula over the loads per step; the model below replays
// the order in which the prologue and the K steps issue their loads (W: the weight pieces of a step, X: its direct token
// loads, T: the operands of the ride-along rows) and derives, for each wait, the largest N that still covers everything
// the code behind the wait reads.  The static_asserts in the kernel compare the two for every unit shape and format.
struct WsLoadQueue {
  static constexpr int kMax = 64;
  int kind[kMax] = {}, step[kMax] = {}, count[kMax] = {}, n = 0;
  constexpr void issue(int k, int s, int c) {
    if (c == 0) return;
    kind[n] = k; step[n] = s; count[n] = c; ++n;
  }
  // loads younger than the youngest entry of (kind k, step s): what may stay in flight when that entry must have landed
  constexpr int younger_than(int k, int s) const {
    int at = -1;
    for (int i = 0; i < n; ++i)
      if (kind[i] == k && step[i] == s) at = i;
    if (at < 0) return -1;  // never issued: a modelling error
    int y = 0;
    for (int i = at + 1; i < n; ++i) y += count[i];
    return y;
  }
};
enum { WS_W = 0, WS_X = 1, WS_T = 2 };
constexpr int ws_min(int a, int b) { return a < b ? a : b; }
// the largest N for the three kinds of wait: 0 = the prologue's first (before the weights of step 0 are converted),
// 1 = its second (before the first barrier), 2 + kt = the wait that ends K step kt
constexpr int ws_model_wait(int which, int W, int X, int T) {
  WsLoadQueue q;
  q.issue(WS_T, 0, T); q.issue(WS_W, 0, W); q.issue(WS_X, 0, X);
  q.issue(WS_T, 1, T); q.issue(WS_W, 1, W); q.issue(WS_X, 1, X);
  q.issue(WS_W, 2, W);
  if (which == 0) return T ? ws_min(q.younger_than(WS_W, 0), q.younger_than(WS_T, 0)) : q.younger_than(WS_W, 0);
  q.issue(WS_T, 2, T); q.issue(WS_W, 3, W);
  // step 0 reads the token rows of step 0 and converts the weights of step 1 (with the ride-along operands of step 1)
  if (which == 1) {
    int need = ws_min(q.younger_than(WS_X, 0), q.younger_than(WS_W, 1));
    return T ? ws_min(need, q.younger_than(WS_T, 1)) : need;
  }
  for (int kt = 0;; ++kt) {
    // K step kt: per piece the reload of the weights of step kt + 4 and its share of the token loads of step kt + 2, then
    // the ride-along operands of step kt + 3 (the interleaving inside a step does not matter to a wait at its end)
    q.issue(WS_W, kt + 4, W); q.issue(WS_X, kt + 2, X); q.issue(WS_T, kt + 3, T);
    if (which == 2 + kt) {
      // behind this wait: the barrier (consumers read the token rows of step kt + 1) and the next step's conversion of the
      // weights of step kt + 2 with the ride-along operands of step kt + 2
      int need = ws_min(q.younger_than(WS_X, kt + 1), q.younger_than(WS_W, kt + 2));
      return T ? ws_min(need, q.younger_than(WS_T, kt + 2)) : need;
    }
  }
}
template <int W, int X, int T> struct WsWaitCheck {
  static_assert(ws_model_wait(0, W, X, T) == 2 * W + 2 * X + T, "prologue: wait before the first conversion");
  static_assert(ws_model_wait(1, W, X, T) == 2 * W + X + T, "prologue: wait before the first barrier");
  // (step 0 could leave the prologue's last weight loads in flight as well; it waits like every other step)
  static_assert(ws_model_wait(2, W, X, T) >= W + X + T && ws_model_wait(3, W, X, T) == W + X + T &&
                ws_model_wait(4, W, X, T) == W + X + T && ws_model_wait(9, W, X, T) == W + X + T, "wait at the end of a K step");
  static constexpr bool ok = true;
};

template <typename T, int WF, int MODE>
__global__ void __launch_bounds__(768, 1)
grouped_mfma_ws_kernel(WsArgs args) {
  constexpr int BN = 256, BM = 256;
  constexpr int kBalance = ws_balance(WF);
  constexpr int WSTAGE = BN * BIG_LS, XSTAGE = BM * BIG_LS;  // elements
  extern __shared__ __align__(16) uint16_t lds[];

  // A workgroup walks its XCD's work list: item `wg`, then every (workgroups per XCD)-th one after it, shifted by half a
  // round in odd rounds (in a block of 32 units the first half belongs to an expert's first token tile, the second half to
  // its second; ride-along rows mostly sit on the first, and a workgroup that always drew the same half would collect
  // them).  The loaders of a unit are done one K step before the consumers and then start the next unit (tile lookup,
  // gather offsets, first loads and conversion) while the consumers still multiply and store: all of LDS is free after the
  // last barrier of a unit.
  // Carried from unit to unit: the round number, this wavefront's index and the experts' row offsets (one per lane).
  // Everything else a unit needs, the plan of the XCD's list included, is derived again inside the loop from values the
  // compiler cannot see through (an opaque zero, the opaque address of the kernel arguments): otherwise it computes the
  // loop-invariant part of every unit's set-up once, in front of the loop, and keeps some hundred values alive through the
  // K loops, whose registers are all taken.
  // Two shapes of unit.  FULL (129..256 token rows): wavefronts 0-7 consume, 8-11 load.  HALF (at most 128 token rows): the
  // consumers' work is halved but a unit still streams and converts its whole 256 x K weight slab, which four loaders
  // cannot do faster than in 2200 cycles per K step; so wavefronts 0-3 consume (one per SIMD, 128 weight rows x 64 token
  // rows each, as in FULL) and wavefronts 4-11 load, two weight pieces each instead of four.  A wavefront's role can
  // change from unit to unit (4-7), which costs nothing: every unit starts from scratch and every wavefront owns the same
  // 168 registers.
  const int wave_id = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int offsets_by_lane = big_lane_offsets(args.p);
  for (int round = 0;; ++round) {
  int zero = 0, wave = wave_id, lane_off = offsets_by_lane;
  asm volatile("" : "+s"(zero), "+s"(wave), "+v"(lane_off));
  const int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, (unsigned)zero));
  const int tid = wave * 64 + lane;
  // A unit's set-up by the loaders (tile lookup, gather offsets, first loads, first conversion) is what its consumers wait
  // for, while the consumers of the previous unit still multiply and store: the loaders go first at the issue stage.
  if (wave >= 8) __builtin_amdgcn_s_setprio(3);
  const int g = lane >> 4, n_in = lane & 15;
  auto kernarg = __builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(kernarg));
  const WsArgs& ka = *reinterpret_cast<const WsArgs*>((const void*)kernarg);
  const GemmParams& p = ka.p;
  const int n_tiles = ka.n_tiles;
  float* const partial = ka.partial;
  const int xcd = blockIdx.x & 7, wg = blockIdx.x >> 3, wgs = ka.wgs_per_xcd;
  const BigPlan pl = big_plan(p, lane_off, BM, n_tiles, xcd, partial != nullptr, true, kBalance);
  // Which item of round `round` (wgs consecutive items of the XCD's list) this workgroup takes: its own index shifted
  // by half a round plus one per round.  Neighbouring items differ systematically in cost (in a block of 32 full units the
  // first half belongs to an expert's first token tile, which carries most ride-along rows; partial units cycle through
  // the experts, some of which have 30 rows and some 250), and a workgroup that drew the same place in every round would
  // collect one kind: the launch ends when the slowest workgroup does.
  const int slot = (wg + round * ((wgs >> 1) + 1)) % wgs;
  BigTile tile;
  if (!big_item(p, lane_off, BM, n_tiles, pl, xcd, round * wgs + slot, tile, true, kBalance)) return;
  const int e = tile.e, row_begin = tile.row_begin, row_end = tile.row_end, ntile = tile.ntile;
  const int rows_here = row_end - row_begin;
  // this workgroup's K steps: all of them, or one chunk of a split unit
  const int kt0 = (int)((p.kred >> 6) * tile.chunk / tile.nchunks);
  const int nkt = (int)((p.kred >> 6) * (tile.chunk + 1) / tile.nchunks) - kt0;

  auto unit = [&](auto loader_tag, auto half_tag) {
  constexpr bool LOADER = decltype(loader_tag)::value != 0;
  constexpr bool HALF = decltype(half_tag)::value != 0;
  constexpr int NLOADERS = HALF ? 8 : 4;
  constexpr int WPIECES = 16 / NLOADERS;                     // packed 16-row weight pieces per loader and K step
  constexpr int XLOADS = (HALF ? 16 : 32) / NLOADERS;        // direct token loads (8 rows each) per loader and K step
  constexpr int XPER = XLOADS / WPIECES;                     // token loads issued after each piece
  constexpr int XROWS = 8 * NLOADERS;                        // LDS rows between a loader's consecutive token loads
  constexpr int GROUPS = HALF ? 2 : 4;                       // token-row groups of 64 LDS rows
  constexpr int WLOADS = BigPiece<WF>::LOADS * WPIECES;
  if constexpr (LOADER) __builtin_amdgcn_s_setprio(3);  // (wavefronts 4-7, which learn their role only here)
  // Rows per token-row group: the rows of a partial tile are spread evenly (in multiples of 16) over the groups, so all
  // consumers share the work and each only multiplies the 16-row column blocks it really has.  Tile row
  // grp * rpg + i (i < rpg) lives in LDS row grp * 64 + i.  Full tiles: rpg = 64, the identity.
  const int rpg = min(64, ((rows_here + GROUPS - 1) / GROUPS + 15) / 16 * 16);

  uint16_t* const Wbase = lds;               // [2][BN][64]
  uint16_t* const Xbase = lds + 2 * WSTAGE;  // [3][BM][64]
  const int sw = n_in & 7;

  if constexpr (LOADER) {
    // =================================== producer ===================================
    const int pw = wave - (HALF ? 4 : 8);
    // This loader's 16-row weight blocks, as rows of the workgroup tile.  GATEUP: WPIECES / 2 gate blocks and the up blocks
    // of the same features (so that an absorbed tail's gate and up sums meet in one lane); DOWN: WPIECES blocks in a row.
    auto piece_block = [&](int j) { return MODE == MODE_GATEUP ? (WPIECES / 2) * pw + j % (WPIECES / 2) : WPIECES * pw + j; };
    auto piece_row = [&](int j) { return (MODE == MODE_GATEUP && j >= WPIECES / 2 ? BN / 2 : 0) + piece_block(j) * 16; };
    BigAddr<WF> waddr[WPIECES];
#pragma unroll
    for (int j = 0; j < WPIECES; ++j) {
      int64_t row0;
      const WeightView* wv;
      if (MODE == MODE_GATEUP) {
        wv = j >= WPIECES / 2 ? &p.w1 : &p.w0;
        row0 = (int64_t)e * wv->rows + (int64_t)ntile * (BN / 2) + piece_block(j) * 16;
      } else {
        wv = &p.w0;
        row0 = (int64_t)e * wv->rows + (int64_t)ntile * BN + piece_row(j);
      }
      waddr[j].init(*wv, row0 >> 4, e, lane, p.kred);
    }
    // token rows: lane l of direct load j fills LDS row pw*8 + XROWS*j + l/8, unit l%8, from global unit (l%8) ^ (row & 7);
    // LDS rows that hold no tile row re-read a valid row (their outputs are never stored)
    uint32_t xoff[XLOADS];
#pragma unroll
    for (int j = 0; j < XLOADS; ++j) {
      const int lr = pw * 8 + XROWS * j + (lane >> 3);
      const int r = min((lr >> 6) * rpg + min(lr & 63, rpg - 1), rows_here - 1);
      const int i = row_begin + r;
      const int64_t src = p.perm ? (int64_t)pair_token(p.perm[i], p.k_top) : (int64_t)i;
      xoff[j] = (uint32_t)((src * p.lda + (((lane & 7) ^ (lr & 7)) << 3)) * 2);
    }
    const uint32_t lds_addr0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)lds);
    const uint32_t x_lds0 = __builtin_amdgcn_readfirstlane(lds_addr0 + (2 * WSTAGE + pw * 8 * BIG_LS) * 2);
    uint16_t* const w_st = Wbase + n_in * BIG_LS;
    const int st_swz0 = ((2 * g) ^ sw) << 3, st_swz1 = ((2 * g + 1) ^ sw) << 3;

    // Absorbed tail.  A converted piece sits in the lane's registers as row n_in of the block, reduction elements
    // 16 g .. 16 g + 15 of the K step: exactly a weight operand of two MFMAs whose K index is permuted (lane group g
    // supplies elements 16 g .. 16 g + 7 to the first and 16 g + 8 .. 16 g + 15 to the second).  A dot product does not care
    // about the order of its terms as long as both operands agree, so lane (n_in, g) fetches the same 16 elements of token row
    // tail_begin + n_in (rows past the end re-read the last one; never stored) straight from global memory and the tail
    // costs neither LDS traffic nor extra operand registers: 8 MFMAs per producer and K step.
    uint32_t toff = 0;
    if (tile.tail_rows > 0) {
      const int i = tile.tail_begin + min(n_in, tile.tail_rows - 1);
      const int64_t src = p.perm ? (int64_t)pair_token(p.perm[i], p.k_top) : (int64_t)i;
      toff = (uint32_t)((src * p.lda + g * 16) * 2);
    }
    u32x4_t tx[2][2];  // [register set = K step % 2][half of the lane's 16 elements]
    floatx4_t tacc[WPIECES];
#pragma unroll
    for (int j = 0; j < WPIECES; ++j) tacc[j] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

    BigPiece<WF> wreg[3][WPIECES];  // three register sets: weights are loaded three K steps before their conversion
    auto load_w = [&](auto set_tag, int kt) {
      constexpr int SET = decltype(set_tag)::value;
#pragma unroll
      for (int j = 0; j < WPIECES; ++j) wreg[SET][j].load_async(waddr[j], kt0 + kt);
    };
    // Converts register set SET (the weights of a K step s) into weight stage STAGE; with TAIL the tail's MFMAs of step s
    // follow each piece's conversion (token operands: register set s % 2 = TXSET).
    auto store_piece = [&](auto set_tag, auto stage_tag, auto tail_tag, auto txset_tag, int j) {
      constexpr int SET = decltype(set_tag)::value, STAGE = decltype(stage_tag)::value, TXSET = decltype(txset_tag)::value;
      constexpr bool TAIL = decltype(tail_tag)::value != 0;
      uint32_t v[8];
      wreg[SET][j].landed();  // awaited by the previous step's vm_wait (or the prologue's)
      wreg[SET][j].template convert<T>(waddr[j], v);
      uint16_t* row = w_st + STAGE * WSTAGE + piece_row(j) * BIG_LS;
      const u32x4_t lo = (u32x4_t){v[0], v[1], v[2], v[3]}, hi = (u32x4_t){v[4], v[5], v[6], v[7]};
      *reinterpret_cast<u32x4_t*>(row + st_swz0) = lo;
      *reinterpret_cast<u32x4_t*>(row + st_swz1) = hi;
      if constexpr (TAIL) {
        tacc[j] = mfma16b<T>(lo, tx[TXSET][0], tacc[j]);
        tacc[j] = mfma16b<T>(hi, tx[TXSET][1], tacc[j]);
      }
    };
    auto store_w = [&](auto set_tag, auto stage_tag, auto tail_tag, auto txset_tag) {
      constexpr int SET = decltype(set_tag)::value, STAGE = decltype(stage_tag)::value, TXSET = decltype(txset_tag)::value;
      constexpr bool TAIL = decltype(tail_tag)::value != 0;
      if constexpr (TAIL) {
        vm_landed(tx[TXSET][0]);
        vm_landed(tx[TXSET][1]);
      }
#pragma unroll
      for (int j = 0; j < WPIECES; ++j) store_piece(set_tag, stage_tag, tail_tag, txset_tag, j);
    };
    auto load_x = [&](auto xstage_tag, int kt) {
      constexpr int XS = decltype(xstage_tag)::value;
      const char* xsrc = reinterpret_cast<const char*>(p.a) + (kt0 + kt) * (BIG_BK * 2);  // the step's columns: a scalar add
#pragma unroll
      for (int j = 0; j < XLOADS; ++j)
        vm_load16_to_lds(xsrc, xoff[j], x_lds0 + (uint32_t)((XS * XSTAGE + XROWS * j * BIG_LS) * 2));
    };
    auto load_tx = [&](auto set_tag, int kt) {
      constexpr int SET = decltype(set_tag)::value;
      const char* src = reinterpret_cast<const char*>(p.a) + (kt0 + kt) * (BIG_BK * 2);
      vm_load16_to_regs(tx[SET][0], src, toff);
      vm_load16_to_regs(tx[SET][1], src + 16, toff);
    };
    // K step kt (R = kt % 6 fixes every stage and register set at compile time): convert the weights of step kt + 1
    // (register set (kt+1) % 3, loaded during step kt - 3) into weight stage (kt+1) % 2 (TAIL: and multiply them with the
    // tail's token operands of step kt + 1, then request those of step kt + 3 into the set just freed), issue the token
    // loads of step kt + 2 into token stage (kt+2) % 3 and the weight loads of step kt + 4 into the register set just
    // freed.  Before the barrier the token loads of step kt + 1 must have landed, and before the next step's conversion the
    // weights of step kt + 2 and the tail operands of step kt + 2: all were issued before the 2 WLOADS + XLOADS (+ TLOADS)
    // youngest loads (the weight loads of steps kt + 3 and kt + 4, the token loads of step kt + 2, the tail operands of
    // step kt + 3).
    // Every step issues every load: requests past the last step read the last step again (cache hits, results unused), so
    // the number of loads in flight is the same at every wait and the steps of a unit are one straight sequence without
    // joins.  That matters because the loads into registers are invisible to the compiler: a register copy or a spill that
    // it placed where two paths with different register assignments meet would move a register whose load has not landed.
    const int last = nkt - 1;
    // The loads of a step are spread between the conversions of its four weight pieces instead of following them in one
    // burst: the compute unit's one vector-memory path takes a wavefront's 1 KB request about every 13 cycles, and the 64
    // requests of a step (4 producers x 16) queue up behind each other; a producer that issues them back to back sits in
    // that queue for 800 cycles after its 1200 cycles of conversion, one that feeds them in between does both at once.
    // Piece j's registers are free once it is converted, so its reload (step kt + 4) follows directly, then two of the
    // step's eight token loads.  All loads of a step are therefore younger than all loads of the step before, and the
    // wait at the end of a step lets exactly this step's loads stay in flight.
    auto k_step = [&](auto r_tag, auto tail_tag, int kt) {
      constexpr int R = decltype(r_tag)::value;
      constexpr bool TAIL = decltype(tail_tag)::value != 0;
      constexpr int TLOADS = TAIL ? 2 : 0;
      constexpr int XS = (R + 2) % 3;
      using Set = WsInt<(R + 1) % 3>;
      using TxSet = WsInt<(R + 1) % 2>;
      using Stage = WsInt<(R + 1) % 2>;
      const char* xsrc = reinterpret_cast<const char*>(p.a) + (kt0 + min(kt + 2, last)) * (BIG_BK * 2);
      const int ktw = kt0 + min(kt + 4, last);
      const bool conv = kt < last;
      if constexpr (TAIL) {
        vm_landed(tx[TxSet::value][0]);
        vm_landed(tx[TxSet::value][1]);
      }
#pragma unroll
      for (int j = 0; j < WPIECES; ++j) {
        if (conv) store_piece(Set{}, Stage{}, tail_tag, TxSet{}, j);
        __builtin_amdgcn_sched_barrier(0);
        wreg[Set::value][j].load_async(waddr[j], ktw);
#pragma unroll
        for (int i = XPER * j; i < XPER * j + XPER; ++i)
          vm_load16_to_lds(xsrc, xoff[i], x_lds0 + (uint32_t)((XS * XSTAGE + XROWS * i * BIG_LS) * 2));
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (TAIL) load_tx(TxSet{}, min(kt + 3, last));
      vm_wait<WLOADS + XLOADS + TLOADS>();
      __syncthreads();
    };
    auto run = [&](auto tail_tag) {
      constexpr bool TAIL = decltype(tail_tag)::value != 0;
      constexpr int TLOADS = TAIL ? 2 : 0;
      static_assert(WsWaitCheck<WLOADS, XLOADS, TLOADS>::ok, "the hand-counted waits no longer match the order of the loads");
      // what step 0 waits for goes first: a unit's first requests queue behind each other for the CU's one vector-memory path
      if constexpr (TAIL) load_tx(WsInt<0>{}, 0);
      load_w(WsInt<0>{}, 0);
      load_x(WsInt<0>{}, 0);
      if constexpr (TAIL) load_tx(WsInt<1>{}, min(1, last));
      load_w(WsInt<1>{}, min(1, last));
      load_x(WsInt<1>{}, min(1, last));
      load_w(WsInt<2>{}, min(2, last));
      // the weights of step 0 (and the tail operands of step 0) are older than everything else issued so far
      vm_wait<2 * WLOADS + 2 * XLOADS + TLOADS>();
      store_w(WsInt<0>{}, WsInt<0>{}, tail_tag, WsInt<0>{});
      if constexpr (TAIL) load_tx(WsInt<0>{}, min(2, last));
      load_w(WsInt<0>{}, min(3, last));
      // step 0 reads the weights stored above and the token rows of step 0, and converts the weights of step 1 (TAIL: with
      // the tail operands of step 1): younger than all of these are the weight loads of steps 2 and 3, the token loads of
      // step 1 and the tail operands of step 2
      vm_wait<2 * WLOADS + XLOADS + TLOADS>();
      __syncthreads();
      // With a tail the loaders carry 8 MFMAs per K step on top of their conversions and are the wavefronts every step
      // waits for; served first at the issue stage they lose less time to the consumers' instructions (measured:
      // tail-carrying tiles 4 % faster; without a tail a raised priority made the consumers 2-4 % slower).
      __builtin_amdgcn_s_setprio(TAIL ? 2 : 0);
      for (int kt = 0;; kt += 6) {
        k_step(WsInt<0>{}, tail_tag, kt);
        if (kt + 1 >= nkt) break;
        k_step(WsInt<1>{}, tail_tag, kt + 1);
        if (kt + 2 >= nkt) break;
        k_step(WsInt<2>{}, tail_tag, kt + 2);
        if (kt + 3 >= nkt) break;
        k_step(WsInt<3>{}, tail_tag, kt + 3);
        if (kt + 4 >= nkt) break;
        k_step(WsInt<4>{}, tail_tag, kt + 4);
        if (kt + 5 >= nkt) break;
        k_step(WsInt<5>{}, tail_tag, kt + 5);
        if (kt + 6 >= nkt) break;
      }
      vm_wait<0>();  // the requests past the last step: nothing may land in registers or LDS after this wavefront is done
    };
    if (HALF || tile.tail_rows == 0) {
      run(WsInt<0>{});
      return;
    }
    if constexpr (!HALF) {
    run(WsInt<1>{});
    // ---- the tail's results: lane (n_in, g) holds, for token row tail_begin + n_in, features 4 g .. 4 g + 3 of each block
    if (n_in < tile.tail_rows) {
      if (tile.nchunks > 1) {
        float* pt = partial + (size_t)tile.chunk_slot * (BN * (BM + kBigTailRows)) + (BM + n_in) * BN;
#pragma unroll
        for (int bi = 0; bi < 4; ++bi) *reinterpret_cast<floatx4_t*>(pt + piece_row(bi) + 4 * g) = tacc[bi];
      } else if (MODE == MODE_GATEUP) {
        T* orow = reinterpret_cast<T*>(p.out) + out_row(p, tile.tail_begin + n_in) * p.ldo + (int64_t)ntile * (BN / 2) + 4 * g;
        const FakeQuant fq = fq_scale(p);
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
          const float gq[4] = {tacc[bi][0], tacc[bi][1], tacc[bi][2], tacc[bi][3]};
          const float uq[4] = {tacc[bi + 2][0], tacc[bi + 2][1], tacc[bi + 2][2], tacc[bi + 2][3]};
          uint2* dst = reinterpret_cast<uint2*>(orow + (2 * pw + bi) * 16);
          if (p.act == STMOE_ACT_SILU) *dst = gateup_quad<T, STMOE_ACT_SILU>(gq, uq, fq);
          else *dst = gateup_quad<T, STMOE_ACT_GELU_ERF>(gq, uq, fq);
        }
      } else {
        T* orow = reinterpret_cast<T*>(p.out) + out_row(p, tile.tail_begin + n_in) * p.ldo + (int64_t)ntile * BN + 4 * g;
#pragma unroll
        for (int bi = 0; bi < 4; ++bi)
          *reinterpret_cast<uint2*>(orow + (4 * pw + bi) * 16) =
              make_uint2(pack2<T>(tacc[bi][0], tacc[bi][1]), pack2<T>(tacc[bi][2], tacc[bi][3]));
      }
    }
    __builtin_amdgcn_s_setprio(0);
    }  // !HALF
  } else {
  // =================================== consumer ===================================
  // Wavefront w runs on SIMD w % 4.  Token-row groups (wm) are spread so that a partial tile, where only the first
  // groups have rows, still uses several SIMDs: wm 0 -> SIMDs 0,1; wm 1 -> SIMDs 2,3; wm 2 -> 0,1; wm 3 -> 2,3 (HALF: two
  // groups, wm 0 -> SIMDs 0,1; wm 1 -> 2,3).
  const int wn = wave & 1, wm = wave >> 1;
  const uint16_t* a_rd[2];  // K half ks: weight row (wavefront base + n_in), unit ks*4 + g
  const uint16_t* b_rd[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const int u = ((ks * 4 + g) ^ sw) << 3;
    a_rd[ks] = Wbase + ((MODE == MODE_GATEUP ? wn * 64 : wn * 128) + n_in) * BIG_LS + u;
    b_rd[ks] = Xbase + (wm * 64 + n_in) * BIG_LS + u;
  }
  floatx4_t acc[8][4];
#pragma unroll
  for (int a = 0; a < 8; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
  const int my_rows = min(rpg, rows_here - wm * rpg);  // tile rows of this wavefront's group (<= 0: none)
  const bool active = my_rows > 0;                     // wavefronts without rows skip their MFMAs
  const int ntj = (my_rows + 15) >> 4;                 // 16-row column blocks that hold rows

  auto compute = [&](auto parity_tag, auto ntj_tag, int xstage, int ks) {
    constexpr int PAR = decltype(parity_tag)::value;
    constexpr int NTJ = decltype(ntj_tag)::value;
    const uint16_t* bp = b_rd[ks] + xstage * XSTAGE;
    u32x4_t bf[NTJ];
#pragma unroll
    for (int tj = 0; tj < NTJ; ++tj) bf[tj] = *reinterpret_cast<const u32x4_t*>(bp + tj * 16 * BIG_LS);
#pragma unroll
    for (int ti = 0; ti < 8; ++ti) {
      const int row_off = MODE == MODE_GATEUP ? (ti < 4 ? 0 : BN / 2) + (ti & 3) * 16 : ti * 16;
      const u32x4_t af = *reinterpret_cast<const u32x4_t*>(a_rd[ks] + PAR * WSTAGE + row_off * BIG_LS);
      // Token fragments in alternating direction: from one instruction to the next only one of the two operands changes
      // (a loop that starts again at fragment 0 changes both at once).  On a launch of nothing but these MFMAs with random
      // operand bits the alternating order runs 5 % faster: the chip is at its power limit there, as it is here.
#pragma unroll
      for (int tj = 0; tj < NTJ; ++tj) {
        const int tjj = (ti & 1) ? NTJ - 1 - tj : tj;
        acc[ti][tjj] = mfma16b<T>(af, bf[tjj], acc[ti][tjj]);
      }
    }
    // Issue order of the block above: the token fragments and two weight fragments first, then one weight fragment
    // read after every fragment's MFMAs, so that each read has the next fragment's MFMAs to land in.  Left alone the
    // compiler reads the fragments in pairs and waits for each pair right away (same registers either way).
    __builtin_amdgcn_sched_group_barrier(0x100, NTJ + 2, 0);
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, NTJ, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2 * NTJ, 0);
  };
  __syncthreads();  // first stage filled
  // The two consumers of a SIMD share its matrix pipe, and the SIMD issues the older wavefront's instruction whenever both
  // have one ready: left alone, wavefronts 0-3 run at the pace their own operand reads allow (about 1500 cycles for the
  // 1024 cycles of MFMAs of a K step), wavefronts 4-7 only fill the gaps and then run the rest of their step alone, where
  // nobody covers their waits for LDS (2500 cycles; every barrier waits for them).  Issue priorities hand the pipe over in
  // the middle of the step instead: the first group runs its first K half above the second group and its second K half
  // below it, so each group has one half in which it is served first and one in which it fills the other's gaps, and both
  // reach the barrier within a few hundred cycles of each other (2575 instead of 2680 cycles per step).  The priority
  // changes sit between the two halves, outside the pinned MFMA / LDS-read sequences; a change inside one (after 40-48 of
  // the 64 MFMAs, nearer the balance point) disturbs that order and gains nothing.
  auto k_loop = [&](auto ntj_tag, auto group_tag) {
    constexpr bool FIRST = decltype(group_tag)::value == 0;
    if (!FIRST) __builtin_amdgcn_s_setprio(1);
    int xs = 0;
    for (int kt = 0; kt < nkt; kt += 2) {
      if (FIRST) __builtin_amdgcn_s_setprio(2);
      compute(WsInt<0>{}, ntj_tag, xs, 0);
      if (FIRST) __builtin_amdgcn_s_setprio(0);
      compute(WsInt<0>{}, ntj_tag, xs, 1);
      __syncthreads();
      xs = xs == 2 ? 0 : xs + 1;
      if (kt + 1 < nkt) {
        if (FIRST) __builtin_amdgcn_s_setprio(2);
        compute(WsInt<1>{}, ntj_tag, xs, 0);
        if (FIRST) __builtin_amdgcn_s_setprio(0);
        compute(WsInt<1>{}, ntj_tag, xs, 1);
        __syncthreads();
        xs = xs == 2 ? 0 : xs + 1;
      }
    }
    __builtin_amdgcn_s_setprio(0);
  };
  // HALF: one consumer per SIMD, nothing to hand over; it stays above the two loaders it shares the SIMD with.
  auto k_loop_of_group = [&](auto ntj_tag) {
    if constexpr (HALF) k_loop(ntj_tag, WsInt<1>{});
    else if (wave < 4) k_loop(ntj_tag, WsInt<0>{});
    else k_loop(ntj_tag, WsInt<1>{});
  };
  if (!active) {
    for (int kt = 0; kt < nkt; ++kt) __syncthreads();
  } else if (ntj == 1) {
    k_loop_of_group(WsInt<1>{});
  } else if (ntj == 2) {
    k_loop_of_group(WsInt<2>{});
  } else {
    k_loop_of_group(WsInt<4>{});
  }

  // ---- epilogue ---------------------------------------------------------------------------------------
  // Rows are written in whole 128-byte lines (see lane_group_transpose4; the launcher checks their alignment).
  auto store_gateup = [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    const FakeQuant fq = fq_scale(p);  // (a quantizer of the intermediate is applied here, where the intermediate is made)
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      const int r = wm * rpg + tj * 16 + n_in;
      const bool mine = tj * 16 + n_in < my_rows;
      if constexpr (ACT == STMOE_ACT_SILU) {
        uint2 q[4];
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
          const float gq[4] = {acc[ti][tj][0], acc[ti][tj][1], acc[ti][tj][2], acc[ti][tj][3]};
          const float uq[4] = {acc[ti + 4][tj][0], acc[ti + 4][tj][1], acc[ti + 4][tj][2], acc[ti + 4][tj][3]};
          q[ti] = gateup_quad<T, ACT>(gq, uq, fq);
        }
        lane_group_transpose4(q);
        if (mine)
          store_16_features(reinterpret_cast<T*>(p.out) + out_row(p, row_begin + r) * p.ldo + (int64_t)ntile * (BN / 2) + wn * 64 + 16 * g, q);
        __builtin_amdgcn_sched_barrier(0);  // one column block at a time: the accumulators leave no room for more
      } else if (mine) {
        // (erf-GELU: its branches keep too much alive next to four finished blocks; every block is stored as it is done)
        T* orow = reinterpret_cast<T*>(p.out) + out_row(p, row_begin + r) * p.ldo + (int64_t)ntile * (BN / 2) + wn * 64 + 4 * g;
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
          const float gq[4] = {acc[ti][tj][0], acc[ti][tj][1], acc[ti][tj][2], acc[ti][tj][3]};
          const float uq[4] = {acc[ti + 4][tj][0], acc[ti + 4][tj][1], acc[ti + 4][tj][2], acc[ti + 4][tj][3]};
          *reinterpret_cast<uint2*>(orow + ti * 16) = gateup_quad<T, ACT>(gq, uq, fq);
        }
      }
    }
  };
  if (tile.nchunks > 1) {
    // chunk of a split unit: fp32 partial tile [BM][BN], added to the other chunks by the workgroup that finishes last (below)
    float* pt = partial + (size_t)tile.chunk_slot * (BN * (BM + kBigTailRows));
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      const int r = wm * rpg + tj * 16 + n_in;
      if (tj * 16 + n_in < my_rows) {
#pragma unroll
        for (int ti = 0; ti < 8; ++ti) {
          const int col = (MODE == MODE_GATEUP ? (ti < 4 ? 0 : BN / 2) + wn * 64 + (ti & 3) * 16 : wn * 128 + ti * 16) + 4 * g;
          *reinterpret_cast<floatx4_t*>(pt + r * BN + col) = acc[ti][tj];
        }
      }
    }
  } else if (MODE == MODE_GATEUP) {
    if (p.act == STMOE_ACT_SILU) store_gateup(EpiAct<STMOE_ACT_SILU>{});
    else store_gateup(EpiAct<STMOE_ACT_GELU_ERF>{});
  } else {
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) {
      const int r = wm * rpg + tj * 16 + n_in;
      const bool mine = tj * 16 + n_in < my_rows;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint2 q[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const floatx4_t v = acc[4 * half + i][tj];
          q[i] = make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
        }
        lane_group_transpose4(q);
        if (mine)
          store_16_features(reinterpret_cast<T*>(p.out) + out_row(p, row_begin + r) * p.ldo + (int64_t)ntile * BN + wn * 128 + half * 64 + 16 * g, q);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  }  // consumer
  };  // unit
  if (rows_here <= BM / 2) {
    if (wave < 4) unit(WsInt<0>{}, WsInt<1>{});
    else unit(WsInt<1>{}, WsInt<1>{});
  } else {
    if (wave < 8) unit(WsInt<0>{}, WsInt<0>{});
    else unit(WsInt<1>{}, WsInt<0>{});
  }
  if (tile.nchunks > 1) {
    // chunk of a split unit (every wavefront of the workgroup gets here): the workgroup that draws the unit's last ticket
    // adds the chunks.  One thread speaks for the workgroup: the barrier orders every thread's partial sums before its
    // draw, whose release makes them visible device-wide (a write-back of the XCD's L2, which all of the workgroup's stores
    // have reached by then) and whose acquire drops what this CU's caches hold of the other chunks before anyone here
    // reads them.  A fence per thread would do the same write-back and invalidation twelve times per workgroup: with a few
    // hundred split units in a launch those took longer than the units themselves.  LDS is free after the unit's last
    // K step; the next unit's loaders start only after the last barrier below.
    __syncthreads();
    int* const drawn_s = reinterpret_cast<int*>(lds);
    int* const ticket = ka.tickets + (tile.chunk_slot - tile.chunk);
    if (tid == 0) *drawn_s = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int drawn = *drawn_s;
    __syncthreads();
    if (drawn == tile.nchunks - 1) {
      const float* base = partial + (size_t)(tile.chunk_slot - tile.chunk) * kWsSlotFloats;
      ws_reduce_unit<T, MODE>(p, tile, base, tid);
      if (tid == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // as the launch found it
    }
  }
  }  // next item
}

template <typename T, int WF, int MODE>
static int launch_ws_m(const GemmParams& p, int64_t max_rows, float* partial, hipStream_t st) {
  constexpr int BN = 256, BM = 256;
  constexpr size_t lds_bytes = (size_t)(2 * BN + 3 * BM) * BIG_LS * 2;
  static std::atomic<uint64_t> lds_ready{0};
  auto kern = grouped_mfma_ws_kernel<T, WF, MODE>;
  if (int rc = reserve_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ready, "mfma ws kernel")) return rc;
  const int n_tiles = (int)(MODE == MODE_GATEUP ? p.n_out / (BN / 2) : p.n_out / BN);
  const int experts = p.offsets ? p.E : 1;
  const int m_slots = (int)((max_rows + BM - 1) / BM) + experts;
  // one workgroup per CU (it takes all of the CU's LDS), fewer when an XCD's list cannot be longer than that
  const int per_xcd = std::min(kBigCusPerXcd, big_grid(n_tiles, m_slots, partial != nullptr) / 8);
  // the tickets of the split units follow the partial tiles; a launch leaves them at zero, so only a caller that cannot
  // vouch for the scratch's history has them cleared first
  int* tickets = partial ? reinterpret_cast<int*>(partial + (size_t)kWsTickets * kWsSlotFloats) : nullptr;
  if (tickets && !p.split_tickets_zeroed) {
    ws_zero_tickets_kernel<<<1, kWsTickets, 0, st>>>(tickets);
    if (int rc = check_launch("ws_zero_tickets")) return rc;
  }
  kern<<<dim3((unsigned)(8 * per_xcd)), 768, lds_bytes, st>>>(WsArgs{p, n_tiles, per_xcd, partial, tickets});
  return check_launch("grouped_mfma_ws");
}

template <typename T, int WF>
static int launch_ws_t(int mode, const GemmParams& p, int64_t max_rows, float* partial, hipStream_t st) {
  return mode == MODE_GATEUP ? launch_ws_m<T, WF, MODE_GATEUP>(p, max_rows, partial, st)
                             : launch_ws_m<T, WF, MODE_DOWN>(p, max_rows, partial, st);
}

size_t mfma_ws_partial_bytes() { return big_partial_bytes(256, 256) + kWsTickets * sizeof(int); }
size_t mfma_ws_tickets_offset() { return big_partial_bytes(256, 256); }
int mfma_ws_ticket_count() { return kWsTickets; }

// `partial`: optional fp32 scratch of mfma_ws_partial_bytes() bytes; with it the last units of a launch, which would
// run on a few CUs only, are split along the reduction.
int launch_mfma_ws(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, float* partial, hipStream_t st) {
  if (max_rows == 0) return STMOE_OK;
  if (p.offsets && p.E >= 64) return set_error(STMOE_ERR_UNSUPPORTED, "mfma ws kernel: at most 63 experts");
  if (wtag != WF_Q8_0_P && wtag != WF_Q4_1_P && wtag != WF_FP8_F32D_P)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma ws kernel: needs weights in a packed streaming order");
  if (p.kred % 256 != 0 || p.lda % 8 != 0 || p.ldo % 8 != 0 || !aligned16(p.out) || p.n_out % (mode == MODE_GATEUP ? 128 : 256) != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma ws kernel: needs K %% 256 == 0, output features in whole tiles and 16-byte aligned output rows");
  {
    // token rows are addressed with 32-bit byte offsets from the activation base
    const int64_t src_rows = p.perm ? (max_rows + p.k_top - 1) / p.k_top : max_rows;
    if (src_rows * p.lda * 2 >= (int64_t)1 << 32)
      return set_error(STMOE_ERR_UNSUPPORTED, "mfma ws kernel: activations span 4 GB or more");
  }
  if (act_dtype == STMOE_F16) {
    if (wtag == WF_Q8_0_P) return launch_ws_t<f16_t, WF_Q8_0_P>(mode, p, max_rows, partial, st);
    if (wtag == WF_Q4_1_P) return launch_ws_t<f16_t, WF_Q4_1_P>(mode, p, max_rows, partial, st);
    return launch_ws_t<f16_t, WF_FP8_F32D_P>(mode, p, max_rows, partial, st);
  }
  if (act_dtype == STMOE_BF16) {
    if (wtag == WF_Q8_0_P) return launch_ws_t<bf16_t, WF_Q8_0_P>(mode, p, max_rows, partial, st);
    if (wtag == WF_Q4_1_P) return launch_ws_t<bf16_t, WF_Q4_1_P>(mode, p, max_rows, partial, st);
    return launch_ws_t<bf16_t, WF_FP8_F32D_P>(mode, p, max_rows, partial, st);
  }
  return set_error(STMOE_ERR_UNSUPPORTED, "mfma ws kernel: activation dtype %d", act_dtype);
}

}  // namespace stmoe
