// Grouped expert projections over rows sorted by expert.
//
// Two projection shapes cover PreGatherFFNMOE.forward (sharktank/sharktank/layers/ffn_moe_block.py:60-72):
//   GATEUP: z[i, n] = T( T(act(T(x[t] . Wg[e][n]))) * T(x[t] . Wu[e][n]) )   ("mk,menk->men" twice + act + mul)
//   DOWN:   y[i, c] = T( z[i] . Wd[e][c] )                                    ("mek,menk->men")
// where i is a sorted position, t = perm[i] / k its token and e its expert; dot products accumulate in
// fp32 and T(.) is a rounding to the activation dtype where the reference materialises a tensor.
#pragma once
#include "weights.h"

namespace stmoe {

enum : int { MODE_GATEUP = 0, MODE_DOWN = 1 };

struct GemmParams {
  const void* a;          // activations: x [T, lda] (GATEUP) or z [rows, lda] (DOWN)
  int64_t lda;
  const int32_t* perm;    // sorted position -> pair id; source row = perm[i] / k_top.  NULL: source row = i
  int32_t k_top;
  const int32_t* offsets; // [E+1] row ranges per expert; NULL: one expert with `fixed_rows` rows
  int32_t E;
  int64_t fixed_rows;
  WeightView w0, w1;      // GATEUP: gate, up.  DOWN: w0 only
  void* out;
  int64_t ldo;
  const int32_t* out_perm;  // optional: output row of sorted position i is out_perm[i] (scatter back to pair order)
  int64_t n_out;          // rows of the weight matrices
  int64_t kred;           // reduction length
  int32_t act;
  const float* x_scale;   // optional scale applied to the fp32 dot products (fp8 activations)
  const float* out_scale; // fp8 kernel only: quantise the result with this reciprocal scale and store e4m3fn bytes
  // fp8 256 x 256 kernel only: e4m3fn activations / results laid out in blocks of 64 reduction samples, [K / 64][rows][64]
  // with `..._block_rows` rows per block (0: plain rows of lda / ldo bytes).  A wavefront's load of 16 token rows of one K
  // stage is then one contiguous kilobyte instead of sixteen half cache lines.
  int64_t a_block_rows, out_block_rows;
  const float* out_fq;    // GATEUP, 16-bit kernels: fake-quantise the gated product with this reciprocal scale (see below)
  int64_t expert_rows_bound;  // host-side bound of rows per expert (a token gives an expert at most one row)
  float* split_scratch;       // optional fp32 scratch for split reductions (mfma_ws_partial_bytes() bytes)
  bool split_tickets_zeroed;  // the caller vouches that the scratch's ticket words (mfma_ws_tickets_offset()) are zero
  // Streaming GATEUP launches of at most 64 (token, slot) pairs only: the router's expert choice per pair.  When set, every
  // wavefront builds the dispatch itself from these (counting sort by expert, stable in the pair id) and reads neither
  // `offsets` nor `perm`; the first wavefront of the grid also writes the four dispatch arrays (`offsets` and `perm` at the
  // addresses above, counts and inv at the ones below) for the launches that follow, so the forward needs no dispatch launch.
  const int32_t* choices;
  int32_t n_choices;
  int32_t *dispatch_counts, *dispatch_inv;
};

// Row range of expert e; without offsets there is one expert with `fixed_rows` rows.
__device__ __forceinline__ void expert_range(const GemmParams& p, int e, int& row_begin, int& row_end) {
  if (p.offsets) {
    row_begin = p.offsets[e];
    row_end = p.offsets[e + 1];
  } else {
    row_begin = 0;
    row_end = (int)p.fixed_rows;
  }
}

// (expert, first row, end row) of m-tile `slot` when every expert's rows are cut into tiles of BM.
__device__ __forceinline__ bool find_tile(const GemmParams& p, int slot, int BM, int& e, int& row_begin, int& row_end) {
  if (!p.offsets) {
    e = 0;
    row_begin = slot * BM;
    row_end = (int)(p.fixed_rows < (int64_t)row_begin + BM ? p.fixed_rows : (int64_t)row_begin + BM);
    return row_begin < p.fixed_rows;
  }
  int acc = 0;
  for (e = 0; e < p.E; ++e) {
    const int b = p.offsets[e], en = p.offsets[e + 1];
    const int tiles = (en - b + BM - 1) / BM;
    if (slot < acc + tiles) {
      row_begin = b + (slot - acc) * BM;
      row_end = en < row_begin + BM ? en : row_begin + BM;
      return true;
    }
    acc += tiles;
  }
  return false;
}

__device__ __forceinline__ float act_rt(int act, float v) {
  return act == STMOE_ACT_SILU ? act_silu(v) : act_gelu_erf(v);
}

__device__ __forceinline__ int64_t out_row(const GemmParams& p, int i) { return p.out_perm ? (int64_t)p.out_perm[i] : (int64_t)i; }

// A static quantizer of the gated intermediate (the q_input of the down projection) is applied where the intermediate is
// produced: the value written is the quantised and dequantised one (FakeQuant) of the gated product, instead of a second
// pass over the whole intermediate.
__device__ __forceinline__ FakeQuant fq_scale(const GemmParams& p) { return FakeQuant(p.out_fq); }

template <typename T> __device__ __forceinline__ float gateup_epilogue(int act, float g, float u, float scale) {
  const float gr = round_to<T>(g * scale);
  const float a = round_to<T>(act_rt(act, gr));
  const float ur = round_to<T>(u * scale);
  return round_to<T>(__fmul_rn(a, ur));
}
template <typename T> __device__ __forceinline__ float gateup_epilogue(int act, float g, float u, float scale, const FakeQuant& fq) {
  const float v = gateup_epilogue<T>(act, g, u, scale);
  return fq.on() ? fq.one<T>(v) : v;
}

// Epilogue of the prefill kernels for one accumulator quad (4 consecutive features of one token): the same rounding
// points as gateup_epilogue, with the activation fixed at compile time.  SiLU is x * rcp(1 + exp2(-x * log2 e)) on the
// hardware exp2 / rcp (about 1 ulp of fp32 each, far below the rounding to the 16-bit activation dtype that
// follows); for fp16 the last product is a packed fp16 multiply, which rounds the exact product once like the fp32
// multiply followed by the conversion.
template <int ACT> __device__ __forceinline__ float act_fast(float v) {
  if constexpr (ACT == STMOE_ACT_SILU)
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.44269504088896340736f));
  else
    return act_gelu_erf(v);
}
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t v);
template <> __device__ __forceinline__ float unpack_lo<f16_t>(uint32_t v) { return (float)__builtin_bit_cast(f16_t, (uint16_t)(v & 0xffffu)); }
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t v) { return __uint_as_float(v << 16); }
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t v);
template <> __device__ __forceinline__ float unpack_hi<f16_t>(uint32_t v) { return (float)__builtin_bit_cast(f16_t, (uint16_t)(v >> 16)); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
// FakeQuant of four packed values of T
template <typename T> __device__ __forceinline__ uint2 fake_quant_quad(uint2 v, const FakeQuant& fq) {
  float a = unpack_lo<T>(v.x), b = unpack_hi<T>(v.x), c = unpack_lo<T>(v.y), d = unpack_hi<T>(v.y);
  fq.pair<T>(a, b);
  fq.pair<T>(c, d);
  return make_uint2(pack2<T>(a, b), pack2<T>(c, d));
}

template <typename T, int ACT>
__device__ __forceinline__ uint2 gateup_quad(const float (&g)[4], const float (&u)[4]) {
  if constexpr (__is_same(T, f16_t)) {
    uint32_t out[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const half2_t a = {(f16_t)act_fast<ACT>((float)(f16_t)g[2 * h]), (f16_t)act_fast<ACT>((float)(f16_t)g[2 * h + 1])};
      const half2_t uu = {(f16_t)u[2 * h], (f16_t)u[2 * h + 1]};
      out[h] = as_u32(a * uu);
    }
    return make_uint2(out[0], out[1]);
  } else {
    float v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float a = round_to<T>(act_fast<ACT>(round_to<T>(g[q])));
      v[q] = round_to<T>(__fmul_rn(a, round_to<T>(u[q])));
    }
    return make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
  }
}
template <typename T, int ACT>
__device__ __forceinline__ uint2 gateup_quad(const float (&g)[4], const float (&u)[4], const FakeQuant& fq) {
  const uint2 v = gateup_quad<T, ACT>(g, u);
  return fq.on() ? fake_quant_quad<T>(v, fq) : v;
}

}  // namespace stmoe

namespace stmoe {
// Launchers (one per kernel family).  `act_dtype` is the activation dtype enum, `wtag` a WF_* tag,
// `max_rows` an upper bound of the sorted row count known on the host (T*k).  Each returns
// STMOE_ERR_UNSUPPORTED when the family has no instantiation for the combination.
int launch_generic(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
int launch_mfma_tile(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
int launch_mfma_big(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
int launch_mfma_narrow(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
int launch_mfma_ws(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, float* partial, hipStream_t st);
size_t mfma_ws_partial_bytes();
size_t mfma_ws_tickets_offset();  // byte offset of the split units' ticket words inside that scratch
int mfma_ws_ticket_count();
int launch_skinny(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
bool skinny_takes_grouped(int act_dtype, int wtag, int E, int64_t kred, int64_t n_out, int64_t lda, int64_t ldo);
int launch_fp8_tile(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
int launch_fp8_ws(int act_dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st);
}  // namespace stmoe
