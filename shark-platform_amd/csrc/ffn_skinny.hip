// Grouped projection for few rows per expert (decode): bandwidth-bound streaming of the expert weights.
//
// Every wavefront works alone (no LDS, no barriers).  A work item is one expert and 16 output features of
// NT weight tiles (gate + up of the same features, or two adjacent 16-row tiles of the down matrix); the
// wavefront walks the reduction dimension in chunks of 256, keeping one chunk of weights (and of the <= 16*MT
// token rows, read through L2) in flight in registers while the matrix cores consume the previous one.
// Weights are loaded with non-temporal 16-byte loads straight into the MFMA operand layout and dequantised
// in registers.  Wavefronts are persistent: item ids are strided by the number of launched wavefronts, which
// the host picks so that every wavefront gets the same number of items.
//
// MFMA roles as in the tile kernel: weight rows are the "A" rows, token rows the "B" columns.  Because the
// operands of one MFMA only have to agree on which 32 reduction indices they cover, each format picks the
// lane <-> k assignment that makes its own loads 16 bytes wide and row-contiguous:
//   1 byte / element (Q8_0, fp8): lane (n, g) load i covers k = 64*i + 16*g .. +15; MFMA steps 2i, 2i+1 take its
//                          low / high 8 bytes.  The token operand of lane (m, g) is x[m][64*i + 16*g .. +15].
//   Q4_1 (1/2 byte):       lane (n, g) load i covers block 4*i + g (32 k); steps 4i .. 4i+3 take 4 bytes each.
//                          Token operand: x[m][128*i + 32*g .. +31].
//   16-bit dense:          as the 1-byte case with 32-byte loads.
#include "ffn_mfma_common.h"

namespace stmoe {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

template <typename T> __device__ __forceinline__ floatx4_t mfma16s(const u32x4_t& a, const u32x4_t& b, floatx4_t c);
template <> __device__ __forceinline__ floatx4_t mfma16s<f16_t>(const u32x4_t& a, const u32x4_t& b, floatx4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ floatx4_t mfma16s<bf16_t>(const u32x4_t& a, const u32x4_t& b, floatx4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ u32x4_t ld_stream16(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
}
__device__ __forceinline__ u32x2_t ld_stream8(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
}
__device__ __forceinline__ u32x4_t ld16(const void* p) { return *reinterpret_cast<const u32x4_t*>(p); }

// fp16 pair -> T pair (identity for fp16; fp16 -> fp32 -> bf16 with round-to-nearest-even for bf16)
template <typename T> __device__ __forceinline__ uint32_t h2_to_T(uint32_t h2) {
  if constexpr (__is_same(T, f16_t)) return h2;
  else return pack2<bf16_t>(f16_bits_to_f32(h2 & 0xffffu), f16_bits_to_f32(h2 >> 16));
}

// ---- per-format weight chunk: 256 reduction elements of one row, as seen by lane (n = lane%16, g = lane/16) ----
template <int WF> struct SkinnyW;

// Which 16 token elements lane group g needs for MFMA steps: returns element offset of the j-th 8-element
// piece of step s inside the chunk.  Q4_1 differs from the others.
template <int WF> __device__ __forceinline__ int x_offset(int s, int g) {
  if constexpr (IsQ4<WF>::value) return 128 * (s >> 2) + 32 * g + 8 * (s & 3);
  else return 64 * (s >> 1) + 16 * g + 8 * (s & 1);
}

template <> struct SkinnyW<WF_Q8_0> {
  u32x4_t q[4];
  u32x4_t d;  // the chunk's 8 block scales
  __device__ __forceinline__ void init(const WeightView&, int64_t) {}
  __device__ __forceinline__ void touch() { asm volatile("" : "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]), "+v"(d)); }
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const uint8_t* base = w.qs + row * w.cols + c * 256 + 16 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = ld_stream16(base + 64 * i);
    d = ld_stream16(w.d + (row * (w.cols >> 5) + c * 8) * 2);
  }
  template <typename T> __device__ __forceinline__ u32x4_t frag(int s, int g) const {
    const int i = s >> 1, h = s & 1;
    const uint32_t dw = d[i];
    const uint32_t dsel = (g & 2) ? (dw >> 16) : (dw & 0xffffu);
    const half2_t dd = as_half2(dsel | (dsel << 16));
    const half2_t bias = {(f16_t)1152.0f, (f16_t)1152.0f};
    u32x4_t out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t u = q[i][2 * h + j] ^ 0x80808080u;
      const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
      const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
      out[2 * j] = h2_to_T<T>(as_u32((as_half2(lo) - bias) * dd));
      out[2 * j + 1] = h2_to_T<T>(as_u32((as_half2(hi) - bias) * dd));
    }
    return out;
  }
};

template <> struct SkinnyW<WF_Q4_1> {
  u32x4_t q[2];
  // fp16 bits of the scale / offset of the lane's own two blocks (4*i + g, i = 0, 1).  Kept as 32-bit values: a 16-bit
  // field is zero-extended again where a register of it is named, and the compiler placed that instruction, with a
  // wait for the prefetch just issued, in the middle of the running chunk, which serialised load and compute.
  uint32_t d[2], m[2];
  __device__ __forceinline__ void init(const WeightView&, int64_t) {}
  __device__ __forceinline__ void touch() { asm volatile("" : "+v"(q[0]), "+v"(q[1]), "+v"(d[0]), "+v"(d[1]), "+v"(m[0]), "+v"(m[1])); }
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const uint8_t* base = w.qs + ((row * w.cols + c * 256) >> 1) + 16 * g;
#pragma unroll
    for (int i = 0; i < 2; ++i) q[i] = ld_stream16(base + 64 * i);
    const int64_t b = row * (w.cols >> 5) + c * 8 + g;
    load_dm(reinterpret_cast<const uint16_t*>(w.d) + b, reinterpret_cast<const uint16_t*>(w.m) + b);
  }
  __device__ __forceinline__ void load_dm(const uint16_t* dp, const uint16_t* mp) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      d[i] = __builtin_nontemporal_load(dp + 4 * i);
      m[i] = __builtin_nontemporal_load(mp + 4 * i);
    }
  }
  template <typename T, bool PACKED = false> __device__ __forceinline__ u32x4_t frag(int s, int g) const {
    const int i = s >> 2, j = s & 3;
    const uint32_t w4 = q[i][j];  // 8 nibbles of block 4*i + g
    u32x4_t out;
    if constexpr (PACKED) {
      uint32_t h[4];
      q4_dword_dequant_packed(w4, q4_scale(d[i], m[i]), h);
#pragma unroll
      for (int b = 0; b < 4; ++b) out[b] = h2_to_T<T>(h[b]);
    } else {
#pragma unroll
      for (int b = 0; b < 4; ++b) out[b] = h2_to_T<T>(q4_pair_dequant(q4_pair_linear(w4, b), d[i], m[i]));
    }
    return out;
  }
};

template <> struct SkinnyW<WF_FP8_F32D> {
  u32x4_t q[4];
  float dv;
  __device__ __forceinline__ void touch() { asm volatile("" : "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]), "+v"(dv)); }
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const uint8_t* base = w.qs + row * w.cols + c * 256 + 16 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = ld_stream16(base + 64 * i);
  }
  // the scale depends on the item only (one per tensor or per expert): fetched once, not with every chunk
  __device__ __forceinline__ void init(const WeightView& w, int64_t row) {
    dv = reinterpret_cast<const float*>(w.d)[w.d_count > 1 ? row / w.rows : 0];
  }
  template <typename T> __device__ __forceinline__ u32x4_t frag(int s, int g) const {
    const int i = s >> 1, h = s & 1;
    float f[8];
    fp8x4_to_f32(q[i][2 * h], f);
    float f2[4];
    fp8x4_to_f32(q[i][2 * h + 1], f2);
#pragma unroll
    for (int b = 0; b < 4; ++b) f[4 + b] = f2[b];
    uint32_t o[4];
    scale8_pack<T>(f, dv, o);
    return (u32x4_t){o[0], o[1], o[2], o[3]};
  }
};

// Packed streaming order: the 16 lanes x 4 groups of one load instruction read one contiguous kilobyte.
template <> struct SkinnyW<WF_Q8_0_P> : SkinnyW<WF_Q8_0> {
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const int64_t rt = row >> 4;
    const int r = (int)(row & 15);
    const uint8_t* base = w.qs + (rt * (w.cols >> 6) + c * 4) * 1024 + (g * 16 + r) * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = ld_stream16(base + 1024 * i);
    d = ld_stream16(w.d + (rt * (w.cols >> 8) + c) * 256 + r * 16);
  }
};
template <> struct SkinnyW<WF_Q4_1_P> : SkinnyW<WF_Q4_1> {
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const int64_t rt = row >> 4;
    const int r = (int)(row & 15);
    const uint8_t* base = w.qs + (rt * (w.cols >> 7) + c * 2) * 1024 + (g * 16 + r) * 16;
#pragma unroll
    for (int i = 0; i < 2; ++i) q[i] = ld_stream16(base + 1024 * i);
    const int64_t b = (rt * (w.cols >> 8) + c) * 128 + r * 8 + g;
    load_dm(reinterpret_cast<const uint16_t*>(w.d) + b, reinterpret_cast<const uint16_t*>(w.m) + b);
  }
  template <typename T> __device__ __forceinline__ u32x4_t frag(int s, int g) const {
    return SkinnyW<WF_Q4_1>::template frag<T, true>(s, g);
  }
};
template <> struct SkinnyW<WF_FP8_F32D_P> : SkinnyW<WF_FP8_F32D> {
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const int64_t rt = row >> 4;
    const uint8_t* base = w.qs + (rt * (w.cols >> 6) + c * 4) * 1024 + (g * 16 + (int)(row & 15)) * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = ld_stream16(base + 1024 * i);
  }
};

template <bool BF> struct SkinnyWDense16 {
  u32x4_t q[8];
  __device__ __forceinline__ void touch() {}
  __device__ __forceinline__ void init(const WeightView&, int64_t) {}
  __device__ __forceinline__ void load(const WeightView& w, int64_t row, int64_t c, int g) {
    const uint8_t* base = w.qs + (row * w.cols + c * 256 + 16 * g) * 2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q[2 * i] = ld_stream16(base + 128 * i);
      q[2 * i + 1] = ld_stream16(base + 128 * i + 16);
    }
  }
  template <typename T> __device__ __forceinline__ u32x4_t frag(int s, int g) const { return q[s]; }
};
template <> struct SkinnyW<WF_DENSE_F16> : SkinnyWDense16<false> {};
template <> struct SkinnyW<WF_DENSE_BF16> : SkinnyWDense16<true> {};

// Token operand of one chunk for one 16-row M tile: 8 MFMA steps x 16 bytes.
template <int WF> struct SkinnyX {
  u32x4_t v[8];
  __device__ __forceinline__ void load(const uint16_t* row_ptr, bool valid, int64_t c, int g) {
    if (!valid) {
#pragma unroll
      for (int s = 0; s < 8; ++s) v[s] = (u32x4_t){0u, 0u, 0u, 0u};
      return;
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) v[s] = ld16(row_ptr + c * 256 + x_offset<WF>(s, g));
  }
};

// The experts' row ranges, fetched once per wavefront with two vector loads (lane l holds expert l's first and end
// row) instead of a scalar load per expert and step of the search: walking the offsets with dependent scalar loads cost a
// workgroup of a one-token launch about 2 us of its 13.  At most 64 experts (checked by the launcher).
// With p.choices (GATEUP launches of at most 64 pairs) the wavefront builds the dispatch from the router's choices instead:
// lane i owns pair i; per expert that occurs a ballot gives its count (kept by lane `expert`) and the rank of each of its
// pairs, a scan over the lanes gives the experts' first rows, and a lane-to-lane scatter leaves the pair id of sorted
// position l in lane l.  The result is the stable counting sort the dispatch launch computes.
struct SkinnyExperts {
  int begin, end;    // of expert `lane`
  uint64_t active;   // experts that received rows
  int n_active;
  int pair_at_lane;  // with p.choices: the pair at sorted position `lane`
  template <int MODE> __device__ __forceinline__ void init(const GemmParams& p, int lane, bool write_out) {
    begin = 0;
    end = 0;
    pair_at_lane = 0;
    if (MODE == MODE_GATEUP && p.choices) {
      const int n = p.n_choices;
      int e = -1;
      if (lane < n) {
        e = p.choices[lane];
        e = e < 0 ? 0 : (e >= p.E ? p.E - 1 : e);  // (out-of-range ids are a caller error; clamped to stay in bounds)
      }
      int rank = 0, count = 0;  // of pair `lane` inside its expert; of expert `lane`
      uint64_t todo = __ballot(lane < n);
      while (todo) {
        const int ee = __builtin_amdgcn_readlane(e, (int)__builtin_ctzll(todo));
        const uint64_t m = __ballot(e == ee);
        if (e == ee) rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        if (lane == ee) count = __builtin_popcountll(m);
        todo &= ~m;
      }
      int run = 0;
      for (int ee = 0; ee < p.E; ++ee) {
        if (lane == ee) begin = run;
        run += __builtin_amdgcn_readlane(count, ee);
      }
      end = begin + count;
      const int first_of_mine = __builtin_amdgcn_ds_bpermute((e < 0 ? 0 : e) << 2, begin);
      const int pos = lane < n ? first_of_mine + rank : lane;  // (lanes without a pair send to themselves)
      pair_at_lane = __builtin_amdgcn_ds_permute(pos << 2, lane);
      if (write_out) {
        if (lane < p.E) {
          p.dispatch_counts[lane] = count;
          const_cast<int32_t*>(p.offsets)[lane] = begin;
        }
        if (lane == 0) const_cast<int32_t*>(p.offsets)[p.E] = n;
        if (lane < n) {
          const_cast<int32_t*>(p.perm)[lane] = pair_at_lane;
          p.dispatch_inv[lane] = pos;
        }
      }
    } else if (p.offsets) {
      if (lane < p.E) {
        begin = p.offsets[lane];
        end = p.offsets[lane + 1];
      }
    } else if (lane == 0) {
      end = (int)p.fixed_rows;
    }
    active = __ballot(end > begin);
    n_active = __builtin_popcountll(active);
  }
  // the a-th expert with rows (a < n_active, the same for every lane of the wavefront)
  __device__ __forceinline__ void find(int a, int& e, int& rb, int& re) const {
    uint64_t m = active;
    for (int i = 0; i < a; ++i) m &= m - 1;
    e = __builtin_ctzll(m);
    rb = __builtin_amdgcn_readlane(begin, e);
    re = __builtin_amdgcn_readlane(end, e);
  }
  // Source row of sorted position i (every lane of the wavefront calls this together).
  template <int MODE> __device__ __forceinline__ int64_t source_row(const GemmParams& p, int i) const {
    if (MODE == MODE_GATEUP && p.choices) return (int64_t)(__builtin_amdgcn_ds_bpermute(i << 2, pair_at_lane) / p.k_top);
    return p.perm ? (int64_t)(p.perm[i] / p.k_top) : (int64_t)i;
  }
};

// One pass of one work item: rows [r0, min(r0 + 16*MT, re)) of expert rows against the item's two weight tiles.
// KS > 1: the KS wavefronts of a workgroup share the item, each takes a contiguous 1/KS of the chunks, and the partial
// sums are added through LDS in a fixed order ((w0 + w1) + (w2 + w3)) by wavefront 0, which then writes the result.
template <typename T, int WF, int MODE, int MT, int KS>
__device__ __forceinline__ void skinny_pass(const GemmParams& p, const SkinnyExperts& experts, const int64_t (&wrow)[2], int tile,
                                            int r0, int re, int64_t nch_total, int lane, bool pin_prefetch) {
  constexpr int NT = 2;
  const int kw = KS > 1 ? (int)(threadIdx.x >> 6) : 0;
  const int64_t c_begin = KS > 1 ? nch_total * kw / KS : 0;
  const int64_t nch = KS > 1 ? nch_total * (kw + 1) / KS : nch_total;  // end of this wavefront's chunk range
  const int g = lane >> 4, n_in = lane & 15;
  // Lanes whose row is past the end of the expert's rows: with one token tile they read the tile's last row instead,
  // so that the loads stay unconditional (see below; the results are never stored); with two tiles they load nothing
  // and multiply zeros, which spares the cache the second tile's reads when it is mostly empty.
  const uint16_t* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int i = r0 + mt * 16 + n_in;
    xok[mt] = MT == 1 || i < re;
    i = min(i, re - 1);
    xrow[mt] = reinterpret_cast<const uint16_t*>(p.a) + experts.template source_row<MODE>(p, i) * p.lda;
  }
  floatx4_t acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = (floatx4_t){0.f, 0.f, 0.f, 0.f};

  // MT == 1: weights and token rows of the next chunk are both in flight during a chunk's MFMAs.
  // MT == 2: only the weights are double-buffered (the two token tiles of both buffers do not fit the
  // 256-register budget of two wavefronts per SIMD); token rows come from L2 and are requested just
  // before the next weight chunk so that weight requests stay in flight while they arrive.
  constexpr bool XDB = MT == 1;
  SkinnyW<WF> w0[NT], w1[NT];
  w0[0].init(p.w0, wrow[0]);
  w1[0].init(p.w0, wrow[0]);
  w0[1].init(MODE == MODE_GATEUP ? p.w1 : p.w0, wrow[1]);
  w1[1].init(MODE == MODE_GATEUP ? p.w1 : p.w0, wrow[1]);
  SkinnyX<WF> x0[MT], x1[XDB ? MT : 1];
  auto load_w = [&](SkinnyW<WF>* w, int64_t c) {
    w[0].load(p.w0, wrow[0], c, g);
    w[1].load(MODE == MODE_GATEUP ? p.w1 : p.w0, wrow[1], c, g);
  };
  auto load_x = [&](SkinnyX<WF>* x, int64_t c) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) x[mt].load(xrow[mt], xok[mt], c, g);
  };
  auto compute = [&](const SkinnyW<WF>* w, const SkinnyX<WF>* x) {
#pragma unroll
    for (int s = 0; s < 8; ++s) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const u32x4_t wf = w[t].template frag<T>(s, g);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt][t] = mfma16s<T>(wf, x[mt].v[s], acc[mt][t]);
      }
    }
  };

  // Every load of the loop is issued unconditionally (past the end the last chunk is simply read again, and rows past
  // the end re-read a valid row): a load that is issued on one path only makes the compiler's wait counters assume,
  // where the paths join, that nothing younger is in flight, and it then waits for the whole prefetch
  // (s_waitcnt vmcnt(0)) in front of the chunk's first MFMA.  The scheduling barriers keep the prefetch in front of
  // the arithmetic it is meant to overlap; without them the loads sink below it to save registers.
  const int64_t last = nch - 1;
  if constexpr (XDB) {
    if (!pin_prefetch) {
      // launches with more rows (8 experts x 8 rows measured 1-3 % faster this way): prefetch under a condition
      if (c_begin < nch) {
        load_w(w0, c_begin);
        load_x(x0, c_begin);
      }
      for (int64_t c = c_begin; c < nch; c += 2) {
        if (c + 1 < nch) { load_w(w1, c + 1); load_x(x1, c + 1); }
        compute(w0, x0);
        if (c + 2 < nch) { load_w(w0, c + 2); load_x(x0, c + 2); }
        if (c + 1 < nch) compute(w1, x1);
      }
    } else if (c_begin < nch) {
      load_w(w0, c_begin);
      load_x(x0, c_begin);
      for (int64_t c = c_begin; c < nch; c += 2) {
        const int64_t c1 = c + 1 < nch ? c + 1 : last, c2 = c + 2 < nch ? c + 2 : last;
        load_w(w1, c1);
        load_x(x1, c1);
        __builtin_amdgcn_sched_barrier(0);
        compute(w0, x0);
        __builtin_amdgcn_sched_barrier(0);
        load_w(w0, c2);
        load_x(x0, c2);
        __builtin_amdgcn_sched_barrier(0);
        if (c + 1 < nch) compute(w1, x1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
    // Two token tiles: here the same treatment measured 2-5 % slower at 32 rows per expert than leaving the weight
    // prefetch conditional (the chunk then starts once its token rows and the prefetch have both landed).
    if (c_begin < nch) load_w(w0, c_begin);
    for (int64_t c = c_begin; c < nch; c += 2) {
      load_x(x0, c);
      if (c + 1 < nch) load_w(w1, c + 1);
      compute(w0, x0);
      if (c + 1 < nch) {
        load_x(x0, c + 1);
        if (c + 2 < nch) load_w(w0, c + 2);
        compute(w1, x0);
      }
    }
  }

  if constexpr (KS > 1) {
    __shared__ floatx4_t red[KS][MT * NT][64];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < NT; ++t) red[kw][mt * NT + t][lane] = acc[mt][t];
    __syncthreads();
    if (kw == 0) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          floatx4_t sum = red[0][mt * NT + t][lane] + red[1][mt * NT + t][lane];
#pragma unroll
          for (int w = 2; w < KS; w += 2) sum = sum + (red[w][mt * NT + t][lane] + red[w + 1][mt * NT + t][lane]);
          acc[mt][t] = sum;
        }
    }
    __syncthreads();  // the buffer is reused by the next pass
    if (kw != 0) return;
  }

  const FakeQuant fq = fq_scale(p);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int i = r0 + mt * 16 + n_in;
    if (i < re) {
      T* orow = reinterpret_cast<T*>(p.out) + out_row(p, i) * p.ldo;
      if (MODE == MODE_GATEUP) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = gateup_epilogue<T>(p.act, acc[mt][0][r], acc[mt][1][r], 1.0f, fq);
        *reinterpret_cast<uint2*>(orow + tile * 16 + 4 * g) = make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
      } else {
#pragma unroll
        for (int t = 0; t < NT; ++t)
          *reinterpret_cast<uint2*>(orow + tile * 32 + t * 16 + 4 * g) =
              make_uint2(pack2<T>(acc[mt][t][0], acc[mt][t][1]), pack2<T>(acc[mt][t][2], acc[mt][t][3]));
      }
    }
  }
}

// The packed formats use the LDS-shared variant.
template <int WF> struct SkinnyUsesLds { static constexpr bool value = WF == WF_Q8_0_P || WF == WF_Q4_1_P || WF == WF_FP8_F32D_P; };

// Workgroups resident per CU (two wavefronts per SIMD: the double-buffered chunks need about 200 registers).
template <int WF> struct SkinnyOcc { static constexpr int value = 2; };

// KS == 1: `total_workers` wavefronts, one item each at a time.  KS == 4: `total_workers` workgroups, the four
// wavefronts of a workgroup split the reduction of one item (for launches with too few items to fill the chip).
template <typename T, int WF, int MODE, int KS>
__global__ void __launch_bounds__(256, SkinnyOcc<WF>::value)
grouped_skinny_kernel(GemmParams p, int tiles_per_expert, int total_waves, bool pin_prefetch) {
  const int lane = threadIdx.x & 63;
  const int n_in = lane & 15;
  const int wave_global = KS > 1 ? (int)blockIdx.x : (int)(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int64_t nch = p.kred >> 8;

  // experts that received rows, in increasing id
  SkinnyExperts experts;
  experts.template init<MODE>(p, lane, blockIdx.x == 0 && threadIdx.x < 64);
  const int n_items = experts.n_active * tiles_per_expert;

  for (int item = wave_global; item < n_items; item += total_waves) {
    const int a_idx = item / tiles_per_expert, tile = item - a_idx * tiles_per_expert;
    int e, rb, re;
    experts.find(__builtin_amdgcn_readfirstlane(a_idx), e, rb, re);

    // the two weight tiles of this item
    int64_t wrow[2];
    if (MODE == MODE_GATEUP) {
      wrow[0] = (int64_t)e * p.w0.rows + tile * 16 + n_in;
      wrow[1] = (int64_t)e * p.w1.rows + tile * 16 + n_in;
    } else {
      wrow[0] = (int64_t)e * p.w0.rows + tile * 32 + n_in;
      wrow[1] = wrow[0] + 16;
    }
    // up to 16 rows: one 16-row token tile; otherwise passes of two tiles (one pass up to 32 rows)
    if (re - rb <= 16) {
      skinny_pass<T, WF, MODE, 1, KS>(p, experts, wrow, tile, rb, re, nch, lane, pin_prefetch);
    } else {
      for (int r0 = rb; r0 < re; r0 += 32) skinny_pass<T, WF, MODE, 2, KS>(p, experts, wrow, tile, r0, re, nch, lane, false);
    }
  }
}

// ---- variant with the token rows shared through LDS ------------------------------------------------------
// Feeding the token operand straight from global memory costs one cache-line access per token row and MFMA step pair
// in every wavefront, and those accesses, not HBM, bound the kernel above.  Here the four wavefronts of a workgroup
// take four neighbouring items of one expert (the same token rows): per chunk of 256 reduction elements the rows
// go global -> LDS once per workgroup with fully coalesced direct loads (global_load_lds_dwordx4, one chunk ahead,
// two LDS stages, one barrier per chunk) and every wavefront reads its MFMA operands from LDS.  LDS rows are 512 bytes;
// the 16-byte unit u of row r lives at unit u ^ (r & 15), which makes the operand reads of 16 rows conflict-free and
// is applied on the source side of the direct loads.  Weights are handled as above (registers, one chunk ahead).
template <typename T, int WF, int MODE, int MT, int G>
__device__ __forceinline__ void skinny_lds_pass(const GemmParams& p, const SkinnyExperts& experts, const int64_t (&wrow)[2], int tile,
                                                int r0, int re, int64_t nch, int lane, int wave, uint16_t* xs, uint32_t xs_addr) {
  // G chunks of 256 reduction elements form one pipeline step (G = 2 for the 4-bit format, whose chunks are half
  // as many bytes, so that as many bytes are in flight per wavefront as for the 8-bit formats)
  constexpr int NT = 2;
  constexpr int XROWS = 16 * MT, XCHUNK = XROWS * 256, XSTAGE = G * XCHUNK;  // elements
  constexpr int XL = XROWS / 8;                                             // direct loads (2 rows each) per wavefront per chunk
  const int g = lane >> 4, n_in = lane & 15;
  // The pass's first weight chunk is requested before anything else: the look-ups of the token rows' addresses (the
  // dispatch permutation) and the token loads that depend on them then run while it is on its way from memory.
  SkinnyW<WF> w0[G][NT], w1[G][NT];
#pragma unroll
  for (int q = 0; q < G; ++q) {
    w0[q][0].init(p.w0, wrow[0]);
    w1[q][0].init(p.w0, wrow[0]);
    w0[q][1].init(MODE == MODE_GATEUP ? p.w1 : p.w0, wrow[1]);
    w1[q][1].init(MODE == MODE_GATEUP ? p.w1 : p.w0, wrow[1]);
  }
  auto load_w = [&](SkinnyW<WF> (*w)[NT], int64_t c) {
#pragma unroll
    for (int q = 0; q < G; ++q) {
      w[q][0].load(p.w0, wrow[0], c + q, g);
      w[q][1].load(MODE == MODE_GATEUP ? p.w1 : p.w0, wrow[1], c + q, g);
    }
  };
  load_w(w0, 0);
  __builtin_amdgcn_sched_barrier(0);  // (left alone the compiler sinks the requests below the look-ups to save registers)
  uint32_t xoff[XL];  // byte offsets from p.a (the host checks that the activations span less than 4 GB)
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    const int lr = 2 * (wave * XL + j) + (lane >> 5);  // LDS row; rows past the end re-read the last row (never stored)
    const int i = min(r0 + lr, re - 1);
    const int64_t src = experts.template source_row<MODE>(p, i);
    xoff[j] = (uint32_t)((src * p.lda + (((lane & 31) ^ (lr & 15)) << 3)) * 2);
  }
  auto load_x = [&](int stage, int64_t c) {  // chunks c .. c + G - 1
#pragma unroll
    for (int q = 0; q < G; ++q)
#pragma unroll
      for (int j = 0; j < XL; ++j)
        vm_load16_to_lds(p.a, xoff[j] + (uint32_t)(c + q) * 512u,
                         xs_addr + (uint32_t)((stage * XSTAGE + q * XCHUNK + 2 * (wave * XL + j) * 256) * 2));
  };
  floatx4_t acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = (floatx4_t){0.f, 0.f, 0.f, 0.f};
  auto compute = [&](const SkinnyW<WF> (*w)[NT], int stage) {
#pragma unroll
    for (int q = 0; q < G; ++q) {
      const uint16_t* xb = xs + stage * XSTAGE + q * XCHUNK + n_in * 256;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        u32x4_t xf[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          xf[mt] = *reinterpret_cast<const u32x4_t*>(xb + mt * 16 * 256 + (((x_offset<WF>(s, g) >> 3) ^ n_in) << 3));
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const u32x4_t wf = w[q][t].template frag<T>(s, g);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt][t] = mfma16s<T>(wf, xf[mt], acc[mt][t]);
        }
      }
    }
  };
  // After the hand-written wait every load has landed; naming the weight registers as operands of an empty statement
  // makes the compiler place its own waits for them here, where they cost nothing, instead of in front of the next
  // step's MFMAs, where they would also wait for the token loads issued in between.
  auto arrived = [&](SkinnyW<WF> (*w)[NT]) {
    vm_wait<0>();
#pragma unroll
    for (int q = 0; q < G; ++q)
#pragma unroll
      for (int t = 0; t < NT; ++t) w[q][t].touch();
    __syncthreads();
  };
  load_x(0, 0);
  arrived(w0);
  for (int64_t c = 0; c < nch; c += 2 * G) {
    if (c + G < nch) {
      load_x(1, c + G);
      load_w(w1, c + G);
    }
    compute(w0, 0);
    arrived(w1);
    if (c + G < nch) {
      if (c + 2 * G < nch) {
        load_x(0, c + 2 * G);
        load_w(w0, c + 2 * G);
      }
      compute(w1, 1);
      arrived(w0);
    }
  }
  const FakeQuant fq = fq_scale(p);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int i = r0 + mt * 16 + n_in;
    if (i < re) {
      T* orow = reinterpret_cast<T*>(p.out) + out_row(p, i) * p.ldo;
      if (MODE == MODE_GATEUP) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = gateup_epilogue<T>(p.act, acc[mt][0][r], acc[mt][1][r], 1.0f, fq);
        *reinterpret_cast<uint2*>(orow + tile * 16 + 4 * g) = make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
      } else {
#pragma unroll
        for (int t = 0; t < NT; ++t)
          *reinterpret_cast<uint2*>(orow + tile * 32 + t * 16 + 4 * g) =
              make_uint2(pack2<T>(acc[mt][t][0], acc[mt][t][1]), pack2<T>(acc[mt][t][2], acc[mt][t][3]));
      }
    }
  }
}

// Workgroups per CU (three for the 4-bit format, which then has to fit 168 registers, measured 4-10 % slower).
template <int WF> struct SkinnyLdsOcc { static constexpr int value = 2; };

// A workgroup takes groups of four neighbouring items (tiles 4q .. 4q+3 of one expert), strided by the grid size.
// MAXMT: the most 16-row token tiles a pass takes (2 or 4).  Launches in which no expert can have more than 32 rows get the
// instance without four-tile passes: its registers and LDS are what the one- and two-tile passes need, and it is the
// kernel of a 32-token decode step (the instance with four-tile passes runs those 0.4 % slower).
template <typename T, int WF, int MODE, int MAXMT>
__global__ void __launch_bounds__(256, SkinnyLdsOcc<WF>::value)
grouped_skinny_lds_kernel(GemmParams p, int tiles_per_expert) {
  constexpr int G = 1;                                     // chunks per pipeline step (the host checks K % (256 G) == 0)
  __shared__ __align__(16) uint16_t xs[2 * G * 16 * MAXMT * 256];  // two stages of up to 16 MAXMT token rows x 256 G reduction elements
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n_in = lane & 15;
  const int64_t nch = p.kred >> 8;
  const uint32_t xs_addr = __builtin_amdgcn_readfirstlane(
      (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)xs));
  SkinnyExperts experts;
  experts.template init<MODE>(p, lane, blockIdx.x == 0 && wave == 0);
  const int groups_per_expert = tiles_per_expert >> 2;
  const int n_groups = experts.n_active * groups_per_expert;
  for (int grp = blockIdx.x; grp < n_groups; grp += gridDim.x) {
    const int a_idx = grp / groups_per_expert, tile = (grp - a_idx * groups_per_expert) * 4 + wave;
    int e, rb, re;
    experts.find(a_idx, e, rb, re);
    int64_t wrow[2];
    if (MODE == MODE_GATEUP) {
      wrow[0] = (int64_t)e * p.w0.rows + tile * 16 + n_in;
      wrow[1] = (int64_t)e * p.w1.rows + tile * 16 + n_in;
    } else {
      wrow[0] = (int64_t)e * p.w0.rows + tile * 32 + n_in;
      wrow[1] = wrow[0] + 16;
    }
    // Passes of up to 64 rows (four 16-row token tiles against the same weight registers): every pass streams the item's
    // weights once, so an expert with 33..64 rows costs one pass, not two.  The token tiles only cost MFMAs, of which the
    // kernel has plenty to spare (the matrix cores are busy in 0.07 of the cycles with one or two tiles).
    for (int r0 = rb; r0 < re; r0 += 16 * MAXMT) {
      const int left = re - r0;
      if (left <= 16) skinny_lds_pass<T, WF, MODE, 1, G>(p, experts, wrow, tile, r0, re, nch, lane, wave, xs, xs_addr);
      else if (MAXMT == 2 || left <= 32) skinny_lds_pass<T, WF, MODE, 2, G>(p, experts, wrow, tile, r0, re, nch, lane, wave, xs, xs_addr);
      else skinny_lds_pass<T, WF, MODE, MAXMT, G>(p, experts, wrow, tile, r0, re, nch, lane, wave, xs, xs_addr);
    }
  }
}

static int pick_waves(int64_t items, int wg_per_cu) {
  // 256 CUs x resident workgroups x 4 wavefronts; give every wavefront the same number of items
  const int64_t capacity = 1024 * wg_per_cu;
  if (items <= capacity) return (int)((items + 3) / 4 * 4);
  const int64_t per_wave = (items + capacity - 1) / capacity;
  const int64_t waves = (items + per_wave - 1) / per_wave;
  return (int)((waves + 3) / 4 * 4);
}

template <typename T, int WF>
static int launch_skinny_t(int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  const int tiles = (int)(mode == MODE_GATEUP ? p.n_out / 16 : p.n_out / 32);
  // at most min(E, rows) experts receive rows; with so few items that four wavefronts per item still fit the chip,
  // a workgroup shares each item and splits its reduction
  const int64_t active_bound = max_rows < p.E ? max_rows : p.E;
  const bool pin = max_rows <= 16;  // a handful of rows in the whole launch: the pinned, unconditional prefetch pays
  const int64_t items_bound = active_bound * tiles;
  if (items_bound * 4 <= 2 * 1024 * SkinnyOcc<WF>::value && (p.kred >> 8) >= 4) {
    dim3 grid((unsigned)items_bound);
    if (mode == MODE_GATEUP) grouped_skinny_kernel<T, WF, MODE_GATEUP, 4><<<grid, 256, 0, st>>>(p, tiles, (int)items_bound, pin);
    else grouped_skinny_kernel<T, WF, MODE_DOWN, 4><<<grid, 256, 0, st>>>(p, tiles, (int)items_bound, pin);
    return check_launch("grouped_skinny(split)");
  }
  {
    // token rows shared through LDS: needs whole groups of four tiles and 32-bit token offsets.  The down projection
    // has four times fewer groups than the gate/up projection; with few rows per expert (one token tile, few loads to
    // share) it is better off with independent wavefronts.
    const int64_t src_rows = p.perm ? (max_rows + p.k_top - 1) / p.k_top : max_rows;
    const bool worth = (mode == MODE_GATEUP || max_rows > 12 * (int64_t)p.E) ;
    if constexpr (SkinnyUsesLds<WF>::value) if (worth && tiles % 4 == 0 && src_rows * p.lda * 2 < ((int64_t)1 << 32)) {
      const int64_t groups = (int64_t)(tiles / 4) * p.E, capacity = 256 * SkinnyLdsOcc<WF>::value;
      const int64_t per_wg = (groups + capacity - 1) / capacity;
      dim3 grid((unsigned)((groups + per_wg - 1) / per_wg));
      // the most rows one expert can have: one per token (when the caller says how many tokens there are), else all of them
      const int64_t rows_bound = p.expert_rows_bound > 0 && p.expert_rows_bound < max_rows ? p.expert_rows_bound : max_rows;
      if (rows_bound <= 32) {
        if (mode == MODE_GATEUP) grouped_skinny_lds_kernel<T, WF, MODE_GATEUP, 2><<<grid, 256, 0, st>>>(p, tiles);
        else grouped_skinny_lds_kernel<T, WF, MODE_DOWN, 2><<<grid, 256, 0, st>>>(p, tiles);
      } else {
        if (mode == MODE_GATEUP) grouped_skinny_lds_kernel<T, WF, MODE_GATEUP, 4><<<grid, 256, 0, st>>>(p, tiles);
        else grouped_skinny_lds_kernel<T, WF, MODE_DOWN, 4><<<grid, 256, 0, st>>>(p, tiles);
      }
      return check_launch("grouped_skinny_lds");
    }
  }
  const int waves = pick_waves((int64_t)tiles * p.E, SkinnyOcc<WF>::value);
  dim3 grid((unsigned)(waves / 4));
  if (mode == MODE_GATEUP) grouped_skinny_kernel<T, WF, MODE_GATEUP, 1><<<grid, 256, 0, st>>>(p, tiles, waves, pin);
  else grouped_skinny_kernel<T, WF, MODE_DOWN, 1><<<grid, 256, 0, st>>>(p, tiles, waves, pin);
  return check_launch("grouped_skinny");
}

// Whether launch_skinny has a kernel for a grouped launch of this shape (the tests it applies itself).
bool skinny_takes_grouped(int act_dtype, int wtag, int E, int64_t kred, int64_t n_out, int64_t lda, int64_t ldo) {
  if (E > 64 || kred % 256 != 0 || n_out % 32 != 0 || lda % 8 != 0 || ldo % 4 != 0) return false;
  switch (wtag) {
    case WF_Q8_0: case WF_Q4_1: case WF_FP8_F32D: case WF_Q8_0_P: case WF_Q4_1_P: case WF_FP8_F32D_P:
      return act_dtype == STMOE_F16 || act_dtype == STMOE_BF16;
    case WF_DENSE_F16: return act_dtype == STMOE_F16;
    case WF_DENSE_BF16: return act_dtype == STMOE_BF16;
    default: return false;
  }
}

int launch_skinny(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if ((!p.offsets && p.E != 1) || p.E > 64 || (!p.offsets && p.fixed_rows >= ((int64_t)1 << 31)))
    return set_error(STMOE_ERR_UNSUPPORTED, "skinny kernel: needs per-expert offsets (or a single matrix) and at most 64 experts");
  if (p.kred % 256 != 0 || p.n_out % 32 != 0 || p.lda % 8 != 0 || p.ldo % 4 != 0)
    return set_error(STMOE_ERR_UNSUPPORTED, "skinny kernel: needs K %% 256 == 0 and N %% 32 == 0");
  if (p.choices && (mode != MODE_GATEUP || p.n_choices < 1 || p.n_choices > 64 || p.n_choices != max_rows || !p.offsets || !p.perm ||
                    !p.dispatch_counts || !p.dispatch_inv))
    return set_error(STMOE_ERR_SHAPE, "skinny kernel: a dispatch inside the launch takes 1..64 pairs of a gate/up launch and four arrays to fill");
  if (max_rows == 0) return STMOE_OK;
    if (act_dtype == STMOE_F16) {
    switch (wtag) {
      case WF_Q8_0: return launch_skinny_t<f16_t, WF_Q8_0>(mode, p, max_rows, st);
      case WF_Q4_1: return launch_skinny_t<f16_t, WF_Q4_1>(mode, p, max_rows, st);
      case WF_FP8_F32D: return launch_skinny_t<f16_t, WF_FP8_F32D>(mode, p, max_rows, st);
      case WF_DENSE_F16: return launch_skinny_t<f16_t, WF_DENSE_F16>(mode, p, max_rows, st);
      case WF_Q8_0_P: return launch_skinny_t<f16_t, WF_Q8_0_P>(mode, p, max_rows, st);
      case WF_Q4_1_P: return launch_skinny_t<f16_t, WF_Q4_1_P>(mode, p, max_rows, st);
      case WF_FP8_F32D_P: return launch_skinny_t<f16_t, WF_FP8_F32D_P>(mode, p, max_rows, st);
      default: break;
    }
  } else if (act_dtype == STMOE_BF16) {
    switch (wtag) {
      case WF_Q8_0: return launch_skinny_t<bf16_t, WF_Q8_0>(mode, p, max_rows, st);
      case WF_Q4_1: return launch_skinny_t<bf16_t, WF_Q4_1>(mode, p, max_rows, st);
      case WF_FP8_F32D: return launch_skinny_t<bf16_t, WF_FP8_F32D>(mode, p, max_rows, st);
      case WF_DENSE_BF16: return launch_skinny_t<bf16_t, WF_DENSE_BF16>(mode, p, max_rows, st);
      case WF_Q8_0_P: return launch_skinny_t<bf16_t, WF_Q8_0_P>(mode, p, max_rows, st);
      case WF_Q4_1_P: return launch_skinny_t<bf16_t, WF_Q4_1_P>(mode, p, max_rows, st);
      case WF_FP8_F32D_P: return launch_skinny_t<bf16_t, WF_FP8_F32D_P>(mode, p, max_rows, st);
      default: break;
    }
  }
  return set_error(STMOE_ERR_UNSUPPORTED, "skinny kernel: no instantiation for activation dtype %d with weight tag %d",
                   act_dtype, wtag);
}

}  // namespace stmoe
