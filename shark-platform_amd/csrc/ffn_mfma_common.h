// Pieces shared by the prefill kernels: MFMA wrappers, the swizzled LDS row layout, the hand-issued direct
// global->LDS load and the register form of one packed weight piece.
#pragma once
#include <atomic>
#include "ffn_kernels.h"

namespace stmoe {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ floatx4_t mfma16b(const u32x4_t& a, const u32x4_t& b, floatx4_t c);
template <> __device__ __forceinline__ floatx4_t mfma16b<f16_t>(const u32x4_t& a, const u32x4_t& b, floatx4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ floatx4_t mfma16b<bf16_t>(const u32x4_t& a, const u32x4_t& b, floatx4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

static constexpr int BIG_BK = 64;
static constexpr int BIG_LS = BIG_BK;  // LDS row stride (elements): 128 bytes = 8 units of 16 bytes, no padding

// LDS rows are XOR-swizzled: the 16-byte unit u of row r lives at unit u ^ (r & 7).  ds_read_b128 serves lanes
// in groups {0-3, 20-23}, {32-35, 52-55}, ... (4 rows of one K group and the next 4 rows of the neighbouring
// K group) and ds_write_b128 in groups of 8 consecutive lanes; with the swizzle every such group touches 8
// distinct 16-byte bank groups for the operand reads, the weight-row writes and the token-row writes alike.
__device__ __forceinline__ int lds_off(int row, int unit) { return row * BIG_LS + ((unit ^ (row & 7)) << 3); }

template <int A> struct EpiAct { static constexpr int value = A; };

// ---- work distribution ---------------------------------------------------------------------------------
// Token tiles are the full ones (BM rows) and the partial ones (the last rows of an expert).  A unit is one token
// tile times one feature tile.  Workgroup ids are dealt round-robin to the 8 XCDs; XCD i takes the i-th eighth of
// the full units and then the i-th eighth of the partial units, so every XCD gets the same amount of work (within
// one unit) and the short partial units run last, where they fill the end of the launch instead of delaying full
// units.  The order inside each class (big_unit) keeps workgroups that share operands together on an XCD.
struct BigTile {
  int e, row_begin, row_end, ntile;
  int chunk, nchunks;  // this workgroup's part of the reduction (0 of 1 unless the unit is split)
  int chunk_slot;      // index of the fp32 partial tile of a split unit's chunk
  int tail_begin, tail_rows;  // rows of the expert's absorbed tail that ride along with this full tile (tail_rows 0: none)
};
// Absorbed tails.  An expert whose row count is a few rows above a multiple of BM would need a whole partial token tile
// (its own pass over the weight slab of every feature tile) for those few rows.  A kernel that asks for it (`absorb`)
// instead lets every full token tile of such an expert take up to kBigTailRows of the tail rows along: full tile s of
// the expert's c full tiles takes tail rows [16 s, 16 s + 16).  A tail is absorbed when it fits: 0 < tail <= 16 c.
static constexpr int kBigTailRows = 16;
__device__ __forceinline__ bool big_tail_absorbed(int rows, int BM, bool absorb) {
  const int c = rows / BM, t = rows - c * BM;
  return absorb && t > 0 && t <= kBigTailRows * c;
}
// Token tiles of an expert with `rows` rows.  Usually rows / BM full tiles and, if rows remain that no full tile takes
// along, one partial tile, which is listed with the other experts' partial tiles at the end of the launch.  With `balance`
// an expert whose remainder is more than half a tile gets rows / BM + 1 tiles of equal size instead (470 rows: 235 + 235
// instead of 256 + 214), all of them listed like full tiles: the same work, but the workgroups that take the same feature
// tile of the two token tiles then run side by side at the same pace and the second one finds the weight tile in L2 (a
// full tile and its expert's partial tile, half a launch apart, both fetch it from memory).  balance = 1 does that for
// experts with one full tile, balance = 2 for any number of full tiles (650 rows: 3 x 217 instead of 256 + 256 + 138),
// which pays where a tile with fewer rows is a faster unit (Q8_0: Mixtral layer at 4096 tokens 2 % faster) and costs
// where the loaders set the pace of a unit whatever its rows (Q4_1: Grok-shape skewed prefill 2.4 % slower).
struct BigExpertTiles {
  int main;     // tiles in the main list (full tiles, or the equal-sized ones)
  int partial;  // 1: a partial tile in the list of partial tiles
  bool even;    // main tiles are the equal-sized ones: tile s = rows [s rows / main, (s + 1) rows / main)
};
__device__ __forceinline__ BigExpertTiles big_expert_tiles(int rows, int BM, bool absorb, int balance) {
  const int c = rows / BM, t = rows - c * BM;
  BigExpertTiles x;
  x.main = c;
  x.partial = 0;
  x.even = false;
  if (t == 0 || big_tail_absorbed(rows, BM, absorb)) return x;
  if (2 * t > BM && (balance == 2 ? c > 0 : balance == 1 && c == 1)) {
    x.main = c + 1;
    x.even = true;
  } else {
    x.partial = 1;
  }
  return x;
}
// A launch whose units do not fill a whole number of rounds over the 32 CUs of an XCD leaves most CUs idle while the
// last few units run.  With `allow_split` those last units (the partial token tiles come last) are cut along the
// reduction into up to 4 chunks (as many as keep units x chunks within the 32 CUs) that run on separate CUs and write
// fp32 partial tiles; big_reduce_kernel adds the chunks in order.  Everything is a pure function of the offsets, so the result is
// the same on every run.
static constexpr int kBigCusPerXcd = 32;
static constexpr int kBigChunkSlotsPerXcd = 32;  // rest * chunks <= 32
struct BigPlan {
  int F, R, f0, f1, r0, r1, whole, rest, chunks;
};
// The offsets are fetched with one vector load (lane l holds offsets[l]) and read back with readlane: walking them with
// scalar loads costs one memory latency per expert, twice per workgroup.  Needs E < 64 (checked by the launchers).
__device__ __forceinline__ int big_lane_offsets(const GemmParams& p) {
  const int lane = threadIdx.x & 63;
  return (p.offsets && lane <= p.E) ? p.offsets[lane] : 0;
}
__device__ __forceinline__ BigPlan big_plan(const GemmParams& p, int lane_off, int BM, int n_tiles, int xcd, bool allow_split,
                                            bool absorb = false, int balance = 0) {
  BigPlan pl;
  pl.F = 0;
  pl.R = 0;
  if (p.offsets) {
    for (int e = 0; e < p.E; ++e) {
      const int rows = __builtin_amdgcn_readlane(lane_off, e + 1) - __builtin_amdgcn_readlane(lane_off, e);
      const BigExpertTiles x = big_expert_tiles(rows, BM, absorb, balance);
      pl.F += x.main;
      pl.R += x.partial;
    }
  } else {
    const BigExpertTiles x = big_expert_tiles((int)p.fixed_rows, BM, absorb, balance);
    pl.F = x.main;
    pl.R = x.partial;
  }
  const int UF = pl.F * n_tiles, UR = pl.R * n_tiles;
  pl.f0 = (int)((int64_t)UF * xcd / 8);
  pl.f1 = (int)((int64_t)UF * (xcd + 1) / 8);
  pl.r0 = (int)((int64_t)UR * xcd / 8);
  pl.r1 = (int)((int64_t)UR * (xcd + 1) / 8);
  const int n = (pl.f1 - pl.f0) + (pl.r1 - pl.r0);
  pl.whole = n;
  pl.rest = 0;
  pl.chunks = 1;
  if (allow_split) {
    const int rest = n % kBigCusPerXcd;
    const int chunks = rest == 0 ? 1 : (kBigCusPerXcd / rest > 4 ? 4 : kBigCusPerXcd / rest);
    if (chunks > 1) {
      pl.whole = n - rest;
      pl.rest = rest;
      pl.chunks = chunks;
    }
  }
  return pl;
}
// Unit number `unit` of the XCD's list: full units, then partial ones.
// Full units are listed expert by expert, and inside an expert feature tile by feature tile with the expert's token
// tiles of one feature tile next to each other: the 32 workgroups of an XCD that run consecutive units then share a few
// token tiles and a few weight tiles through its L2 instead of each fetching its own (with 4 token tiles per expert:
// 4 + 8 operand streams for 32 workgroups), and the workgroups that need the same weight tile start together whatever
// the number of token tiles (blocks of all token tiles x 32 / tiles feature tiles, listed token tile by token tile, gave
// the same sets only when the tile count divides 32: with 3 token tiles the partners drifted into different rounds).
// Partial units: feature tile by feature tile, one unit per expert that has a partial token tile.
__device__ __forceinline__ void big_full_unit(int u, int c, int n_tiles, int& token_tile, int& ntile) {
  ntile = u / c;
  token_tile = u - ntile * c;
}
// Tail rows that full token tile s of an expert (first row b, `rows` rows) takes along.
__device__ __forceinline__ void big_set_tail(int b, int rows, int BM, int s, bool absorb, BigTile& t) {
  t.tail_begin = 0;
  t.tail_rows = 0;
  if (!big_tail_absorbed(rows, BM, absorb)) return;
  const int c = rows / BM, first = c * BM + kBigTailRows * s;
  if (first >= rows) return;
  t.tail_begin = b + first;
  t.tail_rows = min(kBigTailRows, rows - first);
}
// Rows of main tile s of an expert (first row b, `rows` rows) and the tail rows it takes along.
__device__ __forceinline__ void big_main_tile(int b, int rows, int BM, int s, const BigExpertTiles& x, bool absorb, BigTile& t) {
  if (x.even) {
    t.row_begin = b + (int)((int64_t)rows * s / x.main);
    t.row_end = b + (int)((int64_t)rows * (s + 1) / x.main);
    t.tail_begin = 0;
    t.tail_rows = 0;
  } else {
    t.row_begin = b + s * BM;
    t.row_end = t.row_begin + BM;
    big_set_tail(b, rows, BM, s, absorb, t);
  }
}
__device__ __forceinline__ bool big_unit(const GemmParams& p, int lane_off, int BM, int n_tiles, const BigPlan& pl, int unit, BigTile& t,
                                         bool absorb = false, int balance = 0) {
  int u;
  bool partial;
  t.tail_begin = 0;
  t.tail_rows = 0;
  if (unit < pl.f1 - pl.f0) {
    u = pl.f0 + unit;
    partial = false;
  } else if (unit - (pl.f1 - pl.f0) < pl.r1 - pl.r0) {
    u = pl.r0 + unit - (pl.f1 - pl.f0);
    partial = true;
  } else {
    return false;
  }
  if (!p.offsets) {
    t.e = 0;
    if (partial) {
      t.ntile = u;
      t.row_begin = (int)(p.fixed_rows / BM) * BM;
      t.row_end = (int)p.fixed_rows;
    } else {
      int s;
      big_full_unit(u, pl.F, n_tiles, s, t.ntile);
      big_main_tile(0, (int)p.fixed_rows, BM, s, big_expert_tiles((int)p.fixed_rows, BM, absorb, balance), absorb, t);
    }
    return true;
  }
  if (!partial) {
    for (int e = 0; e < p.E; ++e) {
      const int b = __builtin_amdgcn_readlane(lane_off, e), rows = __builtin_amdgcn_readlane(lane_off, e + 1) - b;
      const BigExpertTiles x = big_expert_tiles(rows, BM, absorb, balance);
      const int units = x.main * n_tiles;
      if (u < units) {
        int s;
        big_full_unit(u, x.main, n_tiles, s, t.ntile);
        t.e = e;
        big_main_tile(b, rows, BM, s, x, absorb, t);
        return true;
      }
      u -= units;
    }
    return false;
  }
  t.ntile = u / pl.R;
  int s = u - t.ntile * pl.R;
  for (int e = 0; e < p.E; ++e) {
    const int b = __builtin_amdgcn_readlane(lane_off, e), rows = __builtin_amdgcn_readlane(lane_off, e + 1) - b;
    if (big_expert_tiles(rows, BM, absorb, balance).partial) {
      if (s == 0) {
        t.e = e;
        t.row_begin = b + rows / BM * BM;
        t.row_end = b + rows;
        return true;
      }
      --s;
    }
  }
  return false;
}
__device__ __forceinline__ bool big_tile_id(const GemmParams& p, int BM, int n_tiles, bool allow_split, BigTile& t, bool absorb = false) {
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int lane_off = big_lane_offsets(p);
  const BigPlan pl = big_plan(p, lane_off, BM, n_tiles, xcd, allow_split, absorb);
  int unit;
  if (j < pl.whole) {
    unit = j;
    t.chunk = 0;
    t.nchunks = 1;
    t.chunk_slot = 0;
  } else {
    const int c = j - pl.whole;
    if (c >= pl.rest * pl.chunks) return false;
    unit = pl.whole + c / pl.chunks;
    t.chunk = c % pl.chunks;
    t.nchunks = pl.chunks;
    t.chunk_slot = xcd * kBigChunkSlotsPerXcd + c;
  }
  return big_unit(p, lane_off, BM, n_tiles, pl, unit, t, absorb);
}
// Item j of an XCD's work list: the whole units first, then the chunks of the split ones (the same numbering as the
// workgroup index j of big_tile_id), from a plan and offsets fetched once: for workgroups that walk several items.
__device__ __forceinline__ bool big_item(const GemmParams& p, int lane_off, int BM, int n_tiles, const BigPlan& pl, int xcd, int j, BigTile& t,
                                         bool absorb = false, int balance = 0) {
  int unit;
  if (j < pl.whole) {
    unit = j;
    t.chunk = 0;
    t.nchunks = 1;
    t.chunk_slot = 0;
  } else {
    const int c = j - pl.whole;
    if (c >= pl.rest * pl.chunks) return false;
    unit = pl.whole + c / pl.chunks;
    t.chunk = c % pl.chunks;
    t.nchunks = pl.chunks;
    t.chunk_slot = xcd * kBigChunkSlotsPerXcd + c;
  }
  return big_unit(p, lane_off, BM, n_tiles, pl, unit, t, absorb, balance);
}
// Grid size that covers every XCD's share for at most `slots_bound` token tiles (a split adds up to 24 workgroups).
static inline int big_grid(int n_tiles, int slots_bound, bool allow_split) {
  return 8 * ((n_tiles * slots_bound + 7) / 8 + 2 + (allow_split ? 24 : 0));
}
// fp32 partial tiles of the split units: BM rows plus the rows of an absorbed tail
static inline size_t big_partial_bytes(int BN, int BM) { return (size_t)8 * kBigChunkSlotsPerXcd * BN * (BM + kBigTailRows) * sizeof(float); }

// ---- LDS reservation --------------------------------------------------------------------------------------
// Kernels that use more than 64 KB of dynamic LDS must be told so once per device.  `done` is a per-kernel bit mask of
// the devices already set up (a process that uses several GPUs launches the same kernel on each of them).
static inline int reserve_lds(const void* kernel, size_t bytes, std::atomic<uint64_t>& done, const char* what) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return set_error(STMOE_ERR_LAUNCH, "%s: no current device", what);
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return STMOE_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
    return set_error(STMOE_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", what, bytes);
  done.fetch_or(bit, std::memory_order_release);
  return STMOE_OK;
}

// ---- hand-issued vector-memory operations ------------------------------------------------------------
// Lane l's 16 bytes at base + byte_off land at LDS byte address lds_addr + 16*l (base and lds_addr wave-uniform).
__device__ __forceinline__ void vm_load16_to_lds(const void* base, uint32_t byte_off, uint32_t lds_addr) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);  // the compiler cannot always prove it uniform
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(byte_off), "s"(base), "s"(lds_addr)
               : "memory", "m0");
}
template <int N> __device__ __forceinline__ void vm_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// Loads into registers from a wave-uniform base (scalar registers) plus a 32-bit lane offset, issued by hand: the compiler
// places no wait for the result, so nothing may read it before a vm_wait that covers the load, followed by vm_landed on
// the same variable (an empty statement that makes every later use of the variable come after it in program order).
__device__ __forceinline__ void vm_load16_to_regs(u32x4_t& dst, const void* base, uint32_t byte_off) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(dst) : "v"(byte_off), "s"(base) : "memory");
}
__device__ __forceinline__ void vm_load8_to_regs(uint2& dst, const void* base, uint32_t byte_off) {
  asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(dst) : "v"(byte_off), "s"(base) : "memory");
}
__device__ __forceinline__ void vm_load_u16_to_reg(uint32_t& dst, const void* base, uint32_t byte_off) {
  asm volatile("global_load_ushort %0, %1, %2" : "=&v"(dst) : "v"(byte_off), "s"(base) : "memory");
}
template <typename V> __device__ __forceinline__ void vm_landed(V& v) { asm volatile("" : "+v"(v)::"memory"); }

// ---- packed weight pieces -----------------------------------------------------------------------------
// Per K step (64 reduction elements) and row tile (16 rows), lane (n = lane % 16, g = lane / 16) fetches the samples
// of row n, k = 16*g .. 16*g + 15 and their block scale, and later converts them to 16 values of T (8 dwords) that
// go to LDS units 2g and 2g + 1 of row n.  BigAddr holds what does not change along K, BigPiece what is in flight.
template <int WF> struct BigAddr;
template <int WF> struct BigPiece;

// (q + 1152) built by byte permutation as 0x6400 | u8, minus 1152, times d: f16(d * q) with one rounding
__device__ __forceinline__ void q8x16_to_f16(const u32x4_t& q, uint32_t dbits, uint32_t out[8]) {
  const half2_t dd = as_half2(dbits | (dbits << 16));
  const half2_t bias = {(f16_t)1152.0f, (f16_t)1152.0f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t u = q[i] ^ 0x80808080u;
    const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
    const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
    out[2 * i] = as_u32((as_half2(lo) - bias) * dd);
    out[2 * i + 1] = as_u32((as_half2(hi) - bias) * dd);
  }
}
template <typename T> __device__ __forceinline__ void f16x16_to_T(uint32_t v[8]) {
  if constexpr (!__is_same(T, f16_t)) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = pack2<T>(f16_bits_to_f32(v[i] & 0xffffu), f16_bits_to_f32(v[i] >> 16));
  }
}

// Q8_0: 1 KB piece = 16 rows x 64 k; scales d_p[rt][K/256][16][8]
template <> struct BigAddr<WF_Q8_0_P> {
  const uint8_t* q;  // the row tile's pieces (the same for every lane, so it lives in scalar registers)
  const uint8_t* d;
  uint32_t lq, ld;   // the lane's byte offsets inside a piece / inside the scales of 256 reduction elements
  __device__ __forceinline__ void init(const WeightView& w, int64_t rt, int64_t, int lane, int64_t kred) {
    q = w.qs + rt * (kred >> 6) * 1024;
    d = w.d + rt * (kred >> 8) * 256;
    lq = (uint32_t)lane * 16;
    ld = (uint32_t)(((lane & 15) * 8 + (lane >> 5)) * 2);
  }
};
template <> struct BigPiece<WF_Q8_0_P> {
  static constexpr int LOADS = 2;
  u32x4_t q;
  uint32_t d;  // fp16 bits, zero-extended
  __device__ __forceinline__ void load(const BigAddr<WF_Q8_0_P>& a, int64_t kt) {
    q = *reinterpret_cast<const u32x4_t*>(a.q + kt * 1024 + a.lq);
    d = *reinterpret_cast<const uint16_t*>(a.d + ((kt >> 2) * 256 + (kt & 3) * 4) + a.ld);
  }
  __device__ __forceinline__ void load_async(const BigAddr<WF_Q8_0_P>& a, int64_t kt) {
    vm_load16_to_regs(q, a.q + kt * 1024, a.lq);
    vm_load_u16_to_reg(d, a.d + ((kt >> 2) * 256 + (kt & 3) * 4), a.ld);
  }
  __device__ __forceinline__ void landed() {
    vm_landed(q);
    vm_landed(d);
  }
  template <typename T> __device__ __forceinline__ void convert(const BigAddr<WF_Q8_0_P>&, uint32_t out[8]) const {
    q8x16_to_f16(q, d, out);
    f16x16_to_T<T>(out);
  }
};

// fp8 e4m3fn with one fp32 scale per tensor or per expert: pieces as Q8_0, T(f32(q) * d)
template <> struct BigAddr<WF_FP8_F32D_P> {
  const uint8_t* q;
  uint32_t lq;
  float dv;
  __device__ __forceinline__ void init(const WeightView& w, int64_t rt, int64_t e, int lane, int64_t kred) {
    q = w.qs + rt * (kred >> 6) * 1024;
    lq = (uint32_t)lane * 16;
    dv = reinterpret_cast<const float*>(w.d)[w.d_count > 1 ? e : 0];
  }
};
template <> struct BigPiece<WF_FP8_F32D_P> {
  static constexpr int LOADS = 1;
  u32x4_t q;
  __device__ __forceinline__ void load(const BigAddr<WF_FP8_F32D_P>& a, int64_t kt) {
    q = *reinterpret_cast<const u32x4_t*>(a.q + kt * 1024 + a.lq);
  }
  __device__ __forceinline__ void load_async(const BigAddr<WF_FP8_F32D_P>& a, int64_t kt) { vm_load16_to_regs(q, a.q + kt * 1024, a.lq); }
  __device__ __forceinline__ void landed() { vm_landed(q); }
  template <typename T> __device__ __forceinline__ void convert(const BigAddr<WF_FP8_F32D_P>& a, uint32_t out[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float f[4];
      fp8x4_to_f32(q[i], f);
      out[2 * i] = pack2<T>(__fmul_rn(f[0], a.dv), __fmul_rn(f[1], a.dv));
      out[2 * i + 1] = pack2<T>(__fmul_rn(f[2], a.dv), __fmul_rn(f[3], a.dv));
    }
  }
};

// Q4_1: 1 KB piece = 16 rows x 128 k (lane (n, g') holds block g' of row n, nibbles in the packed order); a K step
// takes half of it: the lane's 16 samples are 8 bytes of block 2*(kt % 2) + g/2, half g % 2
template <> struct BigAddr<WF_Q4_1_P> {
  const uint8_t* q;
  const uint8_t* d;
  const uint8_t* m;
  uint32_t lq, ld;
  __device__ __forceinline__ void init(const WeightView& w, int64_t rt, int64_t, int lane, int64_t kred) {
    const int n = lane & 15, g = lane >> 4;
    q = w.qs + rt * (kred >> 7) * 1024;
    lq = (uint32_t)((((g >> 1) * 16 + n) * 16 + (g & 1) * 8));
    d = w.d + rt * (kred >> 8) * 256;
    m = w.m + rt * (kred >> 8) * 256;
    ld = (uint32_t)((n * 8 + (g >> 1)) * 2);
  }
};
template <> struct BigPiece<WF_Q4_1_P> {
  static constexpr int LOADS = 3;
  uint2 q;
  uint32_t d, m;
  __device__ __forceinline__ void load(const BigAddr<WF_Q4_1_P>& a, int64_t kt) {
    q = *reinterpret_cast<const uint2*>(a.q + ((kt >> 1) * 1024 + (kt & 1) * 512) + a.lq);
    const int64_t s = (kt >> 2) * 256 + (kt & 3) * 4;
    d = *reinterpret_cast<const uint16_t*>(a.d + s + a.ld);
    m = *reinterpret_cast<const uint16_t*>(a.m + s + a.ld);
  }
  __device__ __forceinline__ void load_async(const BigAddr<WF_Q4_1_P>& a, int64_t kt) {
    vm_load8_to_regs(q, a.q + ((kt >> 1) * 1024 + (kt & 1) * 512), a.lq);
    const int64_t s = (kt >> 2) * 256 + (kt & 3) * 4;
    vm_load_u16_to_reg(d, a.d + s, a.ld);
    vm_load_u16_to_reg(m, a.m + s, a.ld);
  }
  __device__ __forceinline__ void landed() {
    vm_landed(q);
    vm_landed(d);
    vm_landed(m);
  }
  template <typename T> __device__ __forceinline__ void convert(const BigAddr<WF_Q4_1_P>&, uint32_t out[8]) const {
    const Q4Scale sc = q4_scale(d, m);
    q4_dword_dequant_packed(q.x, sc, out);
    q4_dword_dequant_packed(q.y, sc, out + 4);
    f16x16_to_T<T>(out);
  }
};

// ---- output rows in whole cache lines ---------------------------------------------------------------------
// An MFMA result leaves lane (n, g) with 4 consecutive features of token row n per 16-feature block: features
// 16 i + 4 g .. + 3 of block i.  Stored as they are, a wavefront instruction writes 32 bytes to each of 16 rows and a
// 128-byte line of the output is touched by four instructions.  A 4 x 4 transpose over the lane groups (register i of group g
// <-> register g of group i; two v_permlane32_swap and two v_permlane16_swap per dword) gives lane (n, g) the 16 consecutive
// features 16 g .. 16 g + 15 of the four blocks' 64: 32 bytes per lane, a whole line per row and instruction pair.
// Every lane of the wavefront must take part.
__device__ __forceinline__ void lane_group_transpose4(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
  typedef uint32_t pair_t __attribute__((ext_vector_type(2)));
  const pair_t a = __builtin_amdgcn_permlane32_swap(r0, r2, false, false);
  const pair_t b = __builtin_amdgcn_permlane32_swap(r1, r3, false, false);
  const pair_t c = __builtin_amdgcn_permlane16_swap(a.x, b.x, false, false);
  const pair_t d = __builtin_amdgcn_permlane16_swap(a.y, b.y, false, false);
  r0 = c.x; r1 = c.y; r2 = d.x; r3 = d.y;
}
// q[i] = this lane's 4 features (two packed 16-bit pairs) of block i; afterwards q[0..3] are 16 consecutive features.
__device__ __forceinline__ void lane_group_transpose4(uint2 (&q)[4]) {
  lane_group_transpose4(q[0].x, q[1].x, q[2].x, q[3].x);
  lane_group_transpose4(q[0].y, q[1].y, q[2].y, q[3].y);
}
__device__ __forceinline__ void store_16_features(void* dst, const uint2 (&q)[4]) {
  uint4* d = reinterpret_cast<uint4*>(dst);
  d[0] = make_uint4(q[0].x, q[0].y, q[1].x, q[1].y);
  d[1] = make_uint4(q[2].x, q[2].y, q[3].x, q[3].y);
}

}  // namespace stmoe
