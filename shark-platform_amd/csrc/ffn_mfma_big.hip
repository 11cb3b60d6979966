// Prefill kernel: grouped projection on the matrix cores with a 256 x 256 workgroup tile.
//
//   workgroup = 4 wavefronts (2 x 2), each owning 128 weight rows x 128 token rows of the tile
//               (GATEUP: 64 gate rows + the same 64 up rows, so the gated product is formed in registers)
//   K step 64, two LDS stages (weights and tokens as 16-bit values, row stride 72 elements so that the
//   16-byte operand reads of 16 consecutive rows fall into distinct banks), one barrier per K step
//   producer: every wavefront loads whole 1 KB pieces of the packed weight order (prepack.hip), dequantises
//             them in registers and writes 16-bit rows into the next LDS stage; token rows are gathered
//             through the dispatch permutation with 128-byte row segments per 8 lanes
//   consumer: v_mfma_f32_16x16x32, weight rows as the "A" rows, token rows as the "B" columns; per K=32 step a
//             wavefront reads 8 + 8 operand fragments from LDS for 64 MFMAs, i.e. half the LDS bytes per flop
//             of a 64 x 64 wavefront tile
//   ragged tiles: MFMAs of 16-token groups past the end of the expert's rows are skipped
//   scheduling: workgroup ids are remapped so that consecutive logical tiles run on the same XCD (one L2),
//               with the token tiles of one (expert, feature tile) adjacent so they share its weights in L2.
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

// One packed 1 KB piece (16 rows x 64 k of 1-byte samples, or 16 rows x 128 k of nibbles) as held by one lane.
template <int WF> struct BigPiece;
template <> struct BigPiece<WF_Q8_0_P> {
  u32x4_t q;
  uint32_t dsel;  // the lane's block scale, duplicated into both halves
  // 16 values of T: row n = lane%16, k = 16*g .. 16*g+15 of the 64-wide K step
  template <typename T> __device__ __forceinline__ void convert(uint32_t out[8]) const {
    const half2_t dd = as_half2(dsel);
    const half2_t bias = {(f16_t)1152.0f, (f16_t)1152.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = q[i] ^ 0x80808080u;
      const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
      const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
      const uint32_t a = as_u32((as_half2(lo) - bias) * dd), b = as_u32((as_half2(hi) - bias) * dd);
      if constexpr (__is_same(T, f16_t)) {
        out[2 * i] = a;
        out[2 * i + 1] = b;
      } else {
        out[2 * i] = pack2<bf16_t>(f16_bits_to_f32(a & 0xffffu), f16_bits_to_f32(a >> 16));
        out[2 * i + 1] = pack2<bf16_t>(f16_bits_to_f32(b & 0xffffu), f16_bits_to_f32(b >> 16));
      }
    }
  }
};

struct BigTagOn { static constexpr bool value = true; };
struct BigTagOff { static constexpr bool value = false; };

// WN x WM wavefronts; each owns 128 weight rows x 64 token rows (32 accumulator tiles = 128 registers, which
// leaves the register allocator room: a 128 x 128 wavefront tile fills all 256 accumulation registers and made
// the compiler shuffle accumulators between register files around every MFMA).
template <typename T, int WF, int MODE, int WN, int WM, int STAGES>
__global__ void __launch_bounds__(64 * WN * WM, STAGES == 1 ? 2 : 1)
grouped_mfma_big_kernel(GemmParams p, int n_tiles, int m_slots) {
  constexpr int NTHR = 64 * WN * WM;
  constexpr int BN = 128 * WN;           // weight rows per workgroup tile (GATEUP: BN/2 gate + BN/2 up)
  constexpr int BM = 64 * WM;            // token rows per workgroup tile
  constexpr int STAGE = (BN + BM) * BIG_LS;
  constexpr int WPIECES = (BN / 16) / (WN * WM);  // packed weight pieces per wavefront per K step
  constexpr int XPIECES = BM * 8 / NTHR;          // 16-byte token pieces per thread per K step
  constexpr int XROWS_PER_PASS = NTHR / 8;
  static_assert(WPIECES >= 1 && XPIECES >= 1, "tile too small for the thread count");
  extern __shared__ __align__(16) uint16_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave / WM, wm = wave % WM;

  // ---- tile id: XCD-aware remap, token tile fastest -------------------------------------------------
  int pid = blockIdx.x;
  {
    const int per_xcd = gridDim.x >> 3;  // the host rounds the grid up to a multiple of 8
    pid = (pid & 7) * per_xcd + (pid >> 3);
  }
  const int slot = pid % m_slots, ntile = pid / m_slots;
  if (ntile >= n_tiles) return;
  int e, row_begin, row_end;
  if (!find_tile(p, slot, BM, e, row_begin, row_end)) return;
  const int rows_here = row_end - row_begin;

  // ---- producer assignment ---------------------------------------------------------------------------
  const int g = lane >> 4, n_in = lane & 15;
  const uint8_t* wq[WPIECES];
  const uint16_t* wd[WPIECES];
  const int64_t kblocks = p.kred >> 6;
#pragma unroll
  for (int j = 0; j < WPIECES; ++j) {
    const int rtl = wave * WPIECES + j;  // row tile (16 rows) inside the workgroup tile
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
    const int64_t rt = row0 >> 4;
    wq[j] = wv->qs + (rt * kblocks * 64 + lane) * 16;
    wd[j] = reinterpret_cast<const uint16_t*>(wv->d) + (rt * (p.kred >> 8) * 16 + n_in) * 8 + (g >> 1);
  }
  // Token rows past the end of the expert's rows are clamped to its last row: every output row depends on its
  // own token row only and those outputs are never stored, so no zero fill (and no branch) is needed.
  const uint16_t* xp[XPIECES];
#pragma unroll
  for (int j = 0; j < XPIECES; ++j) {
    const int r = min((tid >> 3) + XROWS_PER_PASS * j, rows_here - 1);
    const int i = row_begin + r;
    const int64_t src = p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i;
    xp[j] = reinterpret_cast<const uint16_t*>(p.a) + src * p.lda + (tid & 7) * 8;
  }

  BigPiece<WF> wreg[WPIECES];
  u32x4_t xreg[XPIECES];
  auto load_global = [&](int64_t kt) {
#pragma unroll
    for (int j = 0; j < WPIECES; ++j) {
      // plain (cacheable) loads: the token tiles of one (expert, feature tile) run back to back on one XCD and
      // share the weight tile in its L2
      wreg[j].q = *reinterpret_cast<const u32x4_t*>(wq[j] + kt * 1024);
      const uint32_t d = wd[j][(kt >> 2) * 128 + (kt & 3) * 2];
      wreg[j].dsel = d | (d << 16);
    }
#pragma unroll
    for (int j = 0; j < XPIECES; ++j) xreg[j] = *reinterpret_cast<const u32x4_t*>(xp[j] + kt * BIG_BK);
  };
  auto store_lds = [&](int stage) {
    uint16_t* Ws = lds + stage * STAGE;
    uint16_t* Xs = Ws + BN * BIG_LS;
#pragma unroll
    for (int j = 0; j < WPIECES; ++j) {
      uint32_t v[8];
      wreg[j].template convert<T>(v);
      const int row = (wave * WPIECES + j) * 16 + n_in;
      *reinterpret_cast<u32x4_t*>(&Ws[lds_off(row, 2 * g)]) = (u32x4_t){v[0], v[1], v[2], v[3]};
      *reinterpret_cast<u32x4_t*>(&Ws[lds_off(row, 2 * g + 1)]) = (u32x4_t){v[4], v[5], v[6], v[7]};
    }
#pragma unroll
    for (int j = 0; j < XPIECES; ++j)
      *reinterpret_cast<u32x4_t*>(&Xs[lds_off((tid >> 3) + XROWS_PER_PASS * j, tid & 7)]) = xreg[j];
  };

  // ---- consumer -----------------------------------------------------------------------------------------
  // wavefront tile: GATEUP gate rows wn*64..+63 (LDS rows wn*64..) and the same up rows (LDS rows BN/2 + wn*64..);
  //                 DOWN rows wn*128..+127.  Token rows wm*64..+63.
  floatx4_t acc[8][4];
#pragma unroll
  for (int a = 0; a < 8; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
  const bool active = rows_here > wm * 64;  // wavefronts whose token rows are all past the end skip their MFMAs

  auto w_lds_row = [&](int ti) -> int {
    if (MODE == MODE_GATEUP) return (ti < 4 ? 0 : BN / 2) + wn * 64 + (ti & 3) * 16;
    return wn * 128 + ti * 16;
  };
  auto compute = [&](int stage, int ks) {
    const uint16_t* Ws = lds + stage * STAGE;
    const uint16_t* Xs = Ws + BN * BIG_LS;
    u32x4_t bf[4];
#pragma unroll
    for (int tj = 0; tj < 4; ++tj)
      bf[tj] = *reinterpret_cast<const u32x4_t*>(&Xs[lds_off(wm * 64 + tj * 16 + n_in, ks * 4 + g)]);
#pragma unroll
    for (int ti = 0; ti < 8; ++ti) {
      const u32x4_t af = *reinterpret_cast<const u32x4_t*>(&Ws[lds_off(w_lds_row(ti) + n_in, ks * 4 + g)]);
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) acc[ti][tj] = mfma16b<T>(af, bf[tj], acc[ti][tj]);
    }
  };

  const int64_t nkt = p.kred >> 6;
  // ACTIVE is a compile-time tag so that the steady-state loop is one straight-line block (producer and MFMA
  // instructions can be interleaved by the scheduler); wavefronts whose token rows are all past the end run the
  // producer-only copy of the loop.
  auto main_loop = [&](auto active_tag) {
    constexpr bool ACTIVE = decltype(active_tag)::value;
    if constexpr (STAGES == 2) {
      load_global(0);
      store_lds(0);
      __syncthreads();
      if (nkt > 1) load_global(1);
      for (int64_t kt = 0; kt < nkt; ++kt) {
        const int stage = (int)(kt & 1);
        if constexpr (ACTIVE) compute(stage, 0);
        if (kt + 1 < nkt) {
          store_lds(stage ^ 1);
          if (kt + 2 < nkt) load_global(kt + 2);
        }
        if constexpr (ACTIVE) compute(stage, 1);
        __syncthreads();
      }
    } else {
      // one LDS stage, next K step prefetched into registers; two workgroups share a CU and fill each other's
      // barrier and load bubbles
      load_global(0);
      for (int64_t kt = 0; kt < nkt; ++kt) {
        store_lds(0);
        __syncthreads();
        load_global(kt + 1 < nkt ? kt + 1 : kt);
        if constexpr (ACTIVE) {
          compute(0, 0);
          compute(0, 1);
        }
        __syncthreads();
      }
    }
  };
  if (active) main_loop(BigTagOn{});
  else main_loop(BigTagOff{});

  // ---- epilogue -------------------------------------------------------------------------------------------
#pragma unroll
  for (int tj = 0; tj < 4; ++tj) {
    const int r = wm * 64 + tj * 16 + n_in;
    if (r < rows_here) {
      T* orow = reinterpret_cast<T*>(p.out) + out_row(p, row_begin + r) * p.ldo;
      if (MODE == MODE_GATEUP) {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
          float v[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = gateup_epilogue<T>(p.act, acc[ti][tj][q], acc[ti + 4][tj][q], 1.0f);
          *reinterpret_cast<uint2*>(orow + (int64_t)ntile * (BN / 2) + wn * 64 + ti * 16 + 4 * g) =
              make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
        }
      } else {
#pragma unroll
        for (int ti = 0; ti < 8; ++ti)
          *reinterpret_cast<uint2*>(orow + (int64_t)ntile * BN + wn * 128 + ti * 16 + 4 * g) =
              make_uint2(pack2<T>(acc[ti][tj][0], acc[ti][tj][1]), pack2<T>(acc[ti][tj][2], acc[ti][tj][3]));
      }
    }
  }
}

template <typename T, int WF, int MODE, int WN, int WM, int STAGES>
static int launch_big_m(const GemmParams& p, int64_t max_rows, hipStream_t st) {
  constexpr int BN = 128 * WN, BM = 64 * WM;
  constexpr size_t lds_bytes = (size_t)STAGES * (BN + BM) * BIG_LS * 2;
  static bool attr_set = false;
  auto kern = grouped_mfma_big_kernel<T, WF, MODE, WN, WM, STAGES>;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
      return set_error(STMOE_ERR_LAUNCH, "mfma big kernel: cannot reserve %zu bytes of LDS", lds_bytes);
    attr_set = true;
  }
  const int n_tiles = (int)(MODE == MODE_GATEUP ? p.n_out / (BN / 2) : p.n_out / BN);
  const int experts = p.offsets ? p.E : 1;
  const int m_slots = (int)((max_rows + BM - 1) / BM) + experts;
  const int total = (n_tiles * m_slots + 7) / 8 * 8;
  kern<<<dim3((unsigned)total), 64 * WN * WM, lds_bytes, st>>>(p, n_tiles, m_slots);
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
  if (wtag != WF_Q8_0_P)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: needs weights in the packed Q8_0 order");
  if (p.kred % 256 != 0 || p.lda % 8 != 0 || p.ldo % 4 != 0 || p.n_out % (mode == MODE_GATEUP ? 64 * STMOE_BIG_WN : 128 * STMOE_BIG_WN) != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: needs K %% 256 == 0 and output features in whole tiles");
  if (act_dtype == STMOE_F16) return launch_big_t<f16_t, WF_Q8_0_P>(mode, p, max_rows, st);
  if (act_dtype == STMOE_BF16) return launch_big_t<bf16_t, WF_Q8_0_P>(mode, p, max_rows, st);
  return set_error(STMOE_ERR_UNSUPPORTED, "mfma big kernel: activation dtype %d", act_dtype);
}

}  // namespace stmoe
