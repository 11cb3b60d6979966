// RMS norm and the router (logits, softmax, top-k, gate renormalisation) of MoeBlock.forward
// (sharktank/sharktank/layers/mixture_of_experts_block.py:68-83, norm.py:34-41,
//  sharktank/sharktank/ops/default_impls.py:328-359,402-408).
#include "weights.h"

namespace stmoe {

// ---------------------------------------------------------------------------------------------------
// rms_norm: one workgroup of 512 threads per row.  x32 = float(x); o = x32 * (1 / sqrt(mean(x32^2) + eps));
// o = w * W(o) in W = dtype of w; result rounded to T.
//
// Summation order of the mean of squares (part of the contract, restated by the parity oracle, because the
// router's top-k is only reproducible bit for bit if its input is): thread j adds the squares of elements
// j, j+512, j+1024, ... in that order (square and add rounded separately), the 64 sums of a wavefront are
// combined by the xor butterfly 32..1, and the 8 wavefront sums as ((s0+s1)+(s2+s3))+((s4+s5)+(s6+s7)).
// The fused norm+router kernel below uses the same function.
__device__ __forceinline__ float block512_sum_sq_finish(float ss, float* part) {
  ss = wave_xor_sum(ss);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  return ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
}

template <typename T, typename W>
__global__ void __launch_bounds__(512)
rms_norm_kernel(const T* __restrict__ x, const W* __restrict__ w, int64_t K, float eps, T* __restrict__ out) {
  __shared__ float partial[8];
  const T* row = x + (int64_t)blockIdx.x * K;
  T* orow = out + (int64_t)blockIdx.x * K;
  float ss = 0.0f;
  for (int64_t i = threadIdx.x; i < K; i += 512) {
    const float v = Cvt<T>::to_f32(row[i]);
    ss = __fadd_rn(ss, __fmul_rn(v, v));
  }
  const float total = block512_sum_sq_finish(ss, partial);
  const float rs = rms_scale(total, K, eps);
  for (int64_t i = threadIdx.x; i < K; i += 512) {
    float o = round_to<W>(keep_f32(__fmul_rn(Cvt<T>::to_f32(row[i]), rs)));
    o = round_to<W>(keep_f32(__fmul_rn(Cvt<W>::to_f32(w[i]), o)));
    orow[i] = Cvt<T>::from_f32(o);
  }
}

// ---------------------------------------------------------------------------------------------------
// router: one wavefront per token.
//
// Summation order of a logit (part of the contract, restated by the parity oracle): with c = chunk,
// l = lane, lane l owns the 8 consecutive elements k = (c*64 + l)*8 + j, j = 0..7, of every chunk
// c = 0..ceil(K/512)-1 that lies inside K; it adds their products x[k]*w[e][k] to an fp32 accumulator
// in increasing (c, j) order (multiply and add rounded separately, no FMA contraction), and the 64
// lane sums are then combined by the xor butterfly 32,16,8,4,2,1.  The logit is that fp32 sum rounded
// to the activation dtype, as `torch.matmul` on T tensors returns T.
template <typename T> struct Vec8;
template <> struct Vec8<float> {
  float v[8];
  __device__ __forceinline__ void from_raw(const uint4&) {}  // (16-bit rows only)
  __device__ __forceinline__ void load(const float* p) {
    const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};
template <> struct Vec8<f16_t> {
  float v[8];
  __device__ __forceinline__ void load(const f16_t* p) { from_raw(*reinterpret_cast<const uint4*>(p)); }
  __device__ __forceinline__ void from_raw(const uint4& raw) {
    const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      union { uint16_t u; f16_t h; } lo, hi;
      lo.u = (uint16_t)(r[i] & 0xffffu);
      hi.u = (uint16_t)(r[i] >> 16);
      v[2 * i] = (float)lo.h;
      v[2 * i + 1] = (float)hi.h;
    }
  }
};
template <> struct Vec8<bf16_t> {
  float v[8];
  __device__ __forceinline__ void load(const bf16_t* p) { from_raw(*reinterpret_cast<const uint4*>(p)); }
  __device__ __forceinline__ void from_raw(const uint4& raw) {
    const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(r[i] << 16);
      v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
};

// exp(d) for d = logit - max <= 0 as the softmax needs it.  Below -87 the result is a subnormal fp32 number (or zero);
// the fp32 exponential returns zero there, which would turn distinct tiny probabilities into ties (resolved toward the
// lower expert index) where the reference still tells them apart.  Such values are rare; they are computed as
// exp(d + 32) * exp(-32), whose product is rounded into the subnormal range by the multiplication (d + 32 is exact for
// logits that were rounded to a 16-bit type).
__device__ __forceinline__ float softmax_exp(float d) {
  float r = expf(d);
  if (d < -87.0f) r = expf(d + 32.0f) * 1.2664165549094176e-14f;
  return r;
}

// fp32 softmax over the E logits, top-k of the probabilities and renormalised gates of one token, computed alike by
// every lane from the logits lg[0..E) (already rounded to T); lane 0 writes.
template <typename T, int EP>
__device__ __forceinline__ void softmax_topk_store(const float (&lg)[EP], int E, int k, int64_t t, int lane,
                                                   int32_t* __restrict__ idx_out, int64_t* __restrict__ idx64_out,
                                                   T* __restrict__ gate_out) {
  // fp32 softmax over the E logits (F.softmax(dim=1, dtype=float)).
  float mx = lg[0];
#pragma unroll
  for (int e = 1; e < EP; ++e) mx = fmaxf(mx, lg[e]);
  float ex[EP];
  float denom = 0.0f;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    ex[e] = e < E ? softmax_exp(lg[e] - mx) : 0.0f;
    if (e < E) denom += ex[e];
  }
  // The reference ranks the fp32 probabilities (F.softmax, then torch.topk): so does this kernel, with equal
  // probabilities ordered by increasing expert index.  Distinct logits whose probabilities round to the same fp32 number
  // (logits one ulp apart next to the maximum, say) therefore count as a tie, as they do for the reference.
  float pr[EP];
#pragma unroll
  for (int e = 0; e < EP; ++e) pr[e] = (e < E) ? ex[e] / denom : 0.0f;
  uint64_t taken = 0;
  float vsum = 0.0f;
  float pv[EP];  // selected probabilities in slot order (only the first k are used)
  int pi[EP];
#pragma unroll
  for (int j = 0; j < EP; ++j) {
    if (j < k) {
      int best = -1;
      float bestv = 0.0f;
#pragma unroll
      for (int e = 0; e < EP; ++e) {
        if (e < E && !((taken >> e) & 1ull) && (best < 0 || pr[e] > bestv)) {
          best = e;
          bestv = pr[e];
        }
      }
      taken |= 1ull << best;
      pv[j] = bestv;
      pi[j] = best;
      vsum += bestv;
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < EP; ++j) {
      if (j < k) {
        idx_out[t * k + j] = pi[j];
        if (idx64_out) idx64_out[t * k + j] = pi[j];
        gate_out[t * k + j] = Cvt<T>::from_f32(pv[j] / vsum);
      }
    }
  }
}

template <typename T, int EP>
__global__ void __launch_bounds__(256)
router_topk_kernel(const T* __restrict__ x, const T* __restrict__ wr, int64_t T_tokens, int64_t K, int E, int k,
                   T* __restrict__ logits_out, int32_t* __restrict__ idx_out, int64_t* __restrict__ idx64_out,
                   T* __restrict__ gate_out) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_tokens) return;
  const T* xr = x + t * K;

  float acc[EP];
#pragma unroll
  for (int e = 0; e < EP; ++e) acc[e] = 0.0f;

  for (int64_t k0 = (int64_t)lane * 8; k0 < K; k0 += 512) {
    Vec8<T> xv;
    xv.load(xr + k0);
#pragma unroll
    for (int e = 0; e < EP; ++e) {
      if (e < E) {
        Vec8<T> wv;
        wv.load(wr + (int64_t)e * K + k0);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[e] = __fadd_rn(acc[e], __fmul_rn(xv.v[j], wv.v[j]));
      }
    }
  }

  float lg[EP];
#pragma unroll
  for (int e = 0; e < EP; ++e) lg[e] = (e < E) ? round_to<T>(wave_xor_sum(acc[e])) : -INFINITY;

  if (logits_out) {
#pragma unroll
    for (int e = 0; e < EP; ++e)
      if (e < E && lane == (e & 63)) logits_out[t * E + e] = Cvt<T>::from_f32(lg[e]);
  }

  softmax_topk_store<T, EP>(lg, E, k, t, lane, idx_out, idx64_out, gate_out);
}

// ---------------------------------------------------------------------------------------------------
// router, one workgroup (8 wavefronts) per token, optionally fused with the preceding RMS norm.
//
// Wavefront w computes the logits of experts w, w+8, ... with exactly the per-logit summation order documented
// above (a logit is still produced by one wavefront: lane-owned 8-element pieces per 512-element chunk, then the
// xor butterfly), so its bits are identical to router_topk_kernel's; spreading the experts over wavefronts lets
// all loads of a logit be in flight at once, which is what a 32-token decode batch needs.
// FUSE_NORM: the workgroup first normalises the token row (rms_norm_kernel's arithmetic), writes it to `xn`
// (the expert projections read it) and routes the normalised row kept in LDS.
// Dispatch arrays of a one-token launch (all NULL otherwise): counts [E], offsets [E+1], perm [k], inv [k].
struct SingleTokenDispatch {
  int32_t *counts, *offsets, *perm, *inv;
};

template <typename T, typename W, bool FUSE_NORM, int PRE, bool LATE>
__global__ void __launch_bounds__(512, (PRE && !LATE) ? 4 : 8)
router_wg_kernel(const T* __restrict__ x, const W* __restrict__ norm_w, float eps, T* __restrict__ xn,
                 const T* __restrict__ wr, int64_t K, int E, int k, T* __restrict__ logits_out,
                 int32_t* __restrict__ idx_out, int64_t* __restrict__ idx64_out, T* __restrict__ gate_out,
                 SingleTokenDispatch disp, const float* __restrict__ x_fq) {
  extern __shared__ __align__(16) unsigned char smem[];
  // x_fq (with FUSE_NORM): reciprocal scale of a static e4m3fn quantizer of the expert FFN's input.  The router multiplies
  // the normalised row as it is; the copy written to `xn`, which only the expert projections read, is the quantised and
  // dequantised one (fake_quant_fp8_value), so that no separate pass over the activations is needed.
  const FakeQuant fq(FUSE_NORM ? x_fq : nullptr);
  T* xs = reinterpret_cast<T*>(smem);                                  // [K] the (normalised) token row
  float* lg_s = reinterpret_cast<float*>(smem + ((K * sizeof(T) + 15) / 16) * 16);  // [E] logits, then 8 partials
  float* part = lg_s + 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t t = blockIdx.x;
  const T* xr = x + t * K;

  // The first expert's router-weight row chunks of this wavefront are requested before anything else, so that their
  // latency runs in parallel with the norm (they do not depend on it).  PRE chunks of 512 elements are kept in registers.
  // Rows of at least NC * 512 elements (the usual case) take their first loads without a bounds test per load: loads
  // under separate conditions are waited for one by one, those of a straight line are all in flight together.
  // PRE = 8 (a whole row of 4096) for launches of at most 64 tokens and 4 up to 512 tokens (latency).  Launches of more
  // tokens, where throughput counts and the prefetch registers held through the norm would cost a quarter of the
  // workgroups a CU can hold, request the same 8 chunks only after the norm's registers are free (LATE), in front of the
  // barrier that ends the norm: all in flight together, where a loop over the chunks waits for them one by one.
  constexpr int NC = 8;
  const bool long_row = K >= (int64_t)NC * 512;
  uint4 wpre[PRE ? PRE : 1];
  auto prefetch = [&]() {
    if (PRE > 0 && sizeof(T) == 2 && wave < E) {  // 16-bit rows (a chunk of 8 elements is one 16-byte load)
      const T* wrow = wr + (int64_t)wave * K;
      if (long_row) {
#pragma unroll
        for (int j = 0; j < PRE; ++j) wpre[j] = *reinterpret_cast<const uint4*>(wrow + lane * 8 + j * 512);
      } else {
#pragma unroll
        for (int j = 0; j < PRE; ++j) {
          const int64_t k0 = (int64_t)lane * 8 + (int64_t)j * 512;
          if (k0 < K) wpre[j] = *reinterpret_cast<const uint4*>(wrow + k0);
        }
      }
    }
  };
  if constexpr (!LATE) prefetch();
  if constexpr (FUSE_NORM) {
    // the row's elements tid + 512 j are read once and kept (NC of them) for the second pass; the norm weights are
    // requested before the reduction
    float xv[NC], nw[NC];
    float ss = 0.0f;
    if (long_row) {
      T xraw[NC];
      W wraw[NC];
#pragma unroll
      for (int j = 0; j < NC; ++j) xraw[j] = xr[tid + j * 512];
#pragma unroll
      for (int j = 0; j < NC; ++j) wraw[j] = norm_w[tid + j * 512];
#pragma unroll
      for (int j = 0; j < NC; ++j) {
        xv[j] = Cvt<T>::to_f32(xraw[j]);
        nw[j] = Cvt<W>::to_f32(wraw[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < NC; ++j) {
        const int64_t i = tid + (int64_t)j * 512;
        if (i < K) {
          xv[j] = Cvt<T>::to_f32(xr[i]);
          nw[j] = Cvt<W>::to_f32(norm_w[i]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < NC; ++j)
      if (tid + (int64_t)j * 512 < K) ss = __fadd_rn(ss, __fmul_rn(xv[j], xv[j]));
    for (int64_t i = tid + (int64_t)NC * 512; i < K; i += 512) {
      const float v = Cvt<T>::to_f32(xr[i]);
      ss = __fadd_rn(ss, __fmul_rn(v, v));
    }
    const float total = block512_sum_sq_finish(ss, part);
    const float rs = rms_scale(total, K, eps);
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const int64_t i = tid + (int64_t)j * 512;
      if (i < K) {
        float o = round_to<W>(keep_f32(__fmul_rn(xv[j], rs)));
        o = round_to<W>(keep_f32(__fmul_rn(nw[j], o)));
        const T r = Cvt<T>::from_f32(o);
        xs[i] = r;
        xn[t * K + i] = fq.on() ? Cvt<T>::from_f32(fq.one<T>(Cvt<T>::to_f32(r))) : r;
      }
    }
    for (int64_t i = tid + (int64_t)NC * 512; i < K; i += 512) {
      float o = round_to<W>(keep_f32(__fmul_rn(Cvt<T>::to_f32(xr[i]), rs)));
      o = round_to<W>(keep_f32(__fmul_rn(Cvt<W>::to_f32(norm_w[i]), o)));
      const T r = Cvt<T>::from_f32(o);
      xs[i] = r;
      xn[t * K + i] = fq.on() ? Cvt<T>::from_f32(fq.one<T>(Cvt<T>::to_f32(r))) : r;
    }
  } else {
    for (int64_t i = (int64_t)tid * 8; i < K; i += 512 * 8)
      *reinterpret_cast<uint4*>(reinterpret_cast<unsigned char*>(xs) + i * sizeof(T)) =
          *reinterpret_cast<const uint4*>(reinterpret_cast<const unsigned char*>(xr) + i * sizeof(T));
    if constexpr (sizeof(T) == 4)
      for (int64_t i = (int64_t)tid * 8 + 4; i < K; i += 512 * 8)
        *reinterpret_cast<uint4*>(&xs[i]) = *reinterpret_cast<const uint4*>(&xr[i]);
  }
  if constexpr (LATE) prefetch();
  __syncthreads();

  for (int e = wave; e < E; e += 8) {
    float acc = 0.0f;
    const T* wrow = wr + (int64_t)e * K;
    auto chunk = [&](int64_t k0, const uint4* pre) {
      Vec8<T> xv, wv;
      xv.load(xs + k0);
      if (pre) wv.from_raw(*pre);  // the prefetched chunk (16-bit rows, the wavefront's first expert)
      else wv.load(wrow + k0);
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) acc = __fadd_rn(acc, __fmul_rn(xv.v[jj], wv.v[jj]));
    };
    const bool pre_ok = PRE > 0 && sizeof(T) == 2 && e == wave;
#pragma unroll
    for (int j = 0; j < PRE; ++j) {  // chunks in increasing order, as the summation order requires
      const int64_t k0 = (int64_t)lane * 8 + (int64_t)j * 512;
      if (k0 < K) {
        if (pre_ok) chunk(k0, &wpre[j]);
        else chunk(k0, nullptr);
      }
    }
    int64_t k0 = (int64_t)lane * 8 + (int64_t)PRE * 512;
    if constexpr (sizeof(T) == 2) {
      for (; k0 + 3 * 512 < K; k0 += 4 * 512) {  // four chunks requested together, added in increasing order as before
        uint4 wb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) wb[j] = *reinterpret_cast<const uint4*>(wrow + k0 + j * 512);
#pragma unroll
        for (int j = 0; j < 4; ++j) chunk(k0 + j * 512, &wb[j]);
      }
    }
    for (; k0 < K; k0 += 512) chunk(k0, nullptr);
    const float l = round_to<T>(wave_xor_sum(acc));
    if (lane == 0) {
      lg_s[e] = l;
      if (logits_out) logits_out[t * E + e] = Cvt<T>::from_f32(l);
    }
  }
  __syncthreads();
  if (wave != 0) return;

  // fp32 softmax, top-k of the probabilities (equal ones by increasing index), renormalised gates: same arithmetic and
  // order as router_topk_kernel, done by the first wavefront.  Lane e holds expert e: the exponentials and the divisions
  // are computed side by side; everything whose order matters (the sum of the exponentials, the choice with its
  // lower-index-first rule, the sum of the chosen probabilities) is the serial loop over values read from the lanes, which
  // every lane runs alike.
  const float l = lane < E ? lg_s[lane] : 0.0f;
  float mx = __shfl(l, 0);
  for (int e = 1; e < E; ++e) mx = fmaxf(mx, __shfl(l, e));
  const float ex = softmax_exp(l - mx);
  float denom = 0.0f;
  for (int e = 0; e < E; ++e) denom += __shfl(ex, e);
  const float pr = ex / denom;
  uint64_t taken = 0;
  float vsum = 0.0f;
  int my_best = 0;        // lane j: the j-th choice
  float my_bestv = 0.0f;
  for (int j = 0; j < k; ++j) {
    int best = -1;
    float bestv = 0.0f;
    for (int e = 0; e < E; ++e) {
      const float v = __shfl(pr, e);
      if (!((taken >> e) & 1ull) && (best < 0 || v > bestv)) {
        best = e;
        bestv = v;
      }
    }
    taken |= 1ull << best;
    if (lane == j) {
      my_best = best;
      my_bestv = bestv;
    }
    vsum += bestv;
  }
  if (lane < k) {
    idx_out[t * k + lane] = my_best;
    if (idx64_out) idx64_out[t * k + lane] = my_best;
    gate_out[t * k + lane] = Cvt<T>::from_f32(my_bestv / vsum);
  }

  // A launch of one token can also write that token's dispatch (what dispatch_build_kernel would compute from idx):
  // every chosen expert has one row, the rows are ordered by expert id, pair j sits at the number of chosen experts
  // with a smaller id.  Saves a kernel launch where a forward is a handful of short launches.
  if (disp.counts) {
    if (lane < E) {
      disp.counts[lane] = (int32_t)((taken >> lane) & 1ull);
      disp.offsets[lane] = (int32_t)__popcll(taken & ((1ull << lane) - 1ull));
    }
    if (lane == 0) disp.offsets[E] = k;
    if (lane < k) {
      const int pos = (int)__popcll(taken & ((1ull << my_best) - 1ull));
      disp.perm[pos] = lane;
      disp.inv[lane] = pos;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// ffn_norm + router, one wavefront per token: for launches of many tokens, where the workgroup-per-token kernel above
// holds four tokens per CU at a time and every token pays its chain of latencies (row, reduction, barrier, router rows,
// barrier, softmax) in one of two or more rounds.  Here a CU holds a token per wavefront, all tokens of a usual prefill
// launch are in flight at once, and nothing waits at a barrier.  Same bits as rms_norm_kernel + router_topk_kernel:
//   * sum of squares: rms_norm_kernel's thread j adds elements j, j + 512, ...; its wavefront v is threads 64 v .. 64 v + 63.
//     Lane l here plays thread l + 64 v of every wavefront v = 0..7 in turn: eight running sums over the elements
//     l + 64 v + 512 c in increasing c, eight xor butterflies, and the eight wavefront sums combined in the same order;
//   * a logit is a wavefront's sum anyway (lane-owned pieces of 8 elements per chunk of 512, then the butterfly).
// The row is fetched once in the router's layout (16 bytes per lane and chunk); the norm reads its elements in thread
// order through the wavefront's own piece of LDS; the normalised row is computed, stored and multiplied in the
// router's layout again (normalisation is elementwise).  16-bit rows of NCH * 512 elements.
//
// fp16: a product of two fp16 numbers is exact in fp32 (22 significant bits, exponents far inside the fp32 range), so a
// fused multiply-add rounds once exactly where the separate multiply and add round: same bits, fewer instructions.  bf16
// products can fall into the fp32 subnormal range, where the separate multiply would round: they keep both steps.
template <typename T> __device__ __forceinline__ float mul_add_like_separate(float acc, float a, float b) {
  if constexpr (__is_same(T, f16_t)) return __fmaf_rn(a, b, acc);
  else return __fadd_rn(acc, __fmul_rn(a, b));
}

template <typename T, typename W, int NCH, int EP>
__global__ void __launch_bounds__(256)
norm_router_wave_kernel(const T* __restrict__ x, const W* __restrict__ norm_w, float eps, T* __restrict__ xn,
                        const T* __restrict__ wr, int64_t T_tokens, int E, int k, int32_t* __restrict__ idx_out,
                        T* __restrict__ gate_out, const float* __restrict__ x_fq) {
  static_assert(sizeof(T) == 2, "16-bit rows");
  const FakeQuant fq(x_fq);  // (as in router_wg_kernel: the copy in `xn` is the fake-quantised one)
  constexpr int K = NCH * 512;
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  if (t >= T_tokens) return;  // (no barrier in this kernel: every wavefront works on its own piece of LDS)
  uint4* const xs4 = reinterpret_cast<uint4*>(smem) + wave * (K / 8);
  const T* const xs = reinterpret_cast<const T*>(xs4);
  const uint4* const xr4 = reinterpret_cast<const uint4*>(x + t * K);
  uint4 raw[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) raw[c] = xr4[c * 64 + lane];
  // What does not depend on the row is requested right behind it, so that its latency runs beside the row's: the first
  // expert's router row and the first norm weights.  Loads are issued a whole batch at a time throughout: the wavefront
  // has nobody to hide a latency behind, and loads requested one by one are waited for one by one.
  constexpr int NWB = 4;                 // chunks per batch of norm weights
  constexpr bool DOUBLE = NCH <= 8;      // two router-row buffers (the next expert's row is fetched during this one's sums)
  auto load_router_row = [&](uint4 (&dst)[NCH], int e) {
    const uint4* const w4 = reinterpret_cast<const uint4*>(wr + (int64_t)e * K);
#pragma unroll
    for (int c = 0; c < NCH; ++c) dst[c] = w4[c * 64 + lane];
  };
  auto load_norm_weights = [&](Vec8<W> (&dst)[NWB], int c0) {
#pragma unroll
    for (int i = 0; i < NWB; ++i) dst[i].load(norm_w + ((c0 + i) * 64 + lane) * 8);
  };
  uint4 wa[NCH], wb[DOUBLE ? NCH : 1];
  Vec8<W> nw[NWB];
  load_router_row(wa, 0);
  load_norm_weights(nw, 0);
#pragma unroll
  for (int c = 0; c < NCH; ++c) xs4[c * 64 + lane] = raw[c];
  __builtin_amdgcn_wave_barrier();  // (a wavefront's LDS accesses are served in program order)

  float sv[8];
#pragma unroll
  for (int v = 0; v < 8; ++v) sv[v] = 0.0f;
#pragma unroll
  for (int c = 0; c < NCH; ++c)
#pragma unroll
    for (int v = 0; v < 8; ++v) {
      const float e = Cvt<T>::to_f32(xs[lane + 64 * v + 512 * c]);
      sv[v] = mul_add_like_separate<T>(sv[v], e, e);
    }
#pragma unroll
  for (int v = 0; v < 8; ++v) sv[v] = wave_xor_sum(sv[v]);
  const float total = ((sv[0] + sv[1]) + (sv[2] + sv[3])) + ((sv[4] + sv[5]) + (sv[6] + sv[7]));
  const float rs = rms_scale(total, K, eps);

  float xf[NCH][8];  // the normalised row as the router multiplies it: values of T
  uint4* const xn4 = reinterpret_cast<uint4*>(xn + t * K);
#pragma unroll
  for (int c0 = 0; c0 < NCH; c0 += NWB) {
    if (c0 > 0) load_norm_weights(nw, c0);
#pragma unroll
    for (int i = 0; i < NWB; ++i) {
      const int c = c0 + i;
      Vec8<T> xv;
      xv.from_raw(raw[c]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float o = round_to<W>(keep_f32(__fmul_rn(xv.v[j], rs)));
        o = round_to<W>(keep_f32(__fmul_rn(nw[i].v[j], o)));
        xf[c][j] = round_to<T>(o);
      }
      uint4 packed = make_uint4(pack2<T>(xf[c][0], xf[c][1]), pack2<T>(xf[c][2], xf[c][3]), pack2<T>(xf[c][4], xf[c][5]),
                                pack2<T>(xf[c][6], xf[c][7]));
      if (fq.on()) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = xf[c][j];
#pragma unroll
        for (int j = 0; j < 8; j += 2) fq.pair<T>(v[j], v[j + 1]);
        packed = make_uint4(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]), pack2<T>(v[4], v[5]), pack2<T>(v[6], v[7]));
      }
      xn4[c * 64 + lane] = packed;
    }
  }

  float lg[EP];
  auto logit = [&](const uint4 (&w)[NCH]) {
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      Vec8<T> wv;
      wv.from_raw(w[c]);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc = mul_add_like_separate<T>(acc, xf[c][j], wv.v[j]);
    }
    return round_to<T>(wave_xor_sum(acc));
  };
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    lg[e] = -INFINITY;
    if (e < E) {
      if constexpr (DOUBLE) {
        // expert e sits in wa (even e) or wb (odd e); the other buffer takes expert e + 1 meanwhile
        if (e % 2 == 0) {
          if (e + 1 < E) load_router_row(wb, e + 1);
          lg[e] = logit(wa);
        } else {
          if (e + 1 < E) load_router_row(wa, e + 1);
          lg[e] = logit(wb);
        }
      } else {
        if (e > 0) load_router_row(wa, e);
        lg[e] = logit(wa);
      }
    }
  }
  softmax_topk_store<T, EP>(lg, E, k, t, lane, idx_out, nullptr, gate_out);
}

// Whether the wavefront-per-token kernel takes this launch (16-bit rows of 2048, 4096, 6144 or 8192 elements, at most 16
// experts, 16-byte aligned operands); launches of fewer tokens keep the workgroup-per-token kernel, whose eight
// wavefronts share a token's work and finish it sooner.
static constexpr int64_t kWaveRouterMinTokens = 768;  // (measured at 4096-element rows: 14 us against 13.5 at 512 tokens, 16 against 18 at 1024, 17 against 25 at 2048)
template <typename T, typename W>
static bool launch_norm_router_wave(const void* x, const void* norm_w, float eps, void* xn, const void* wr, int64_t T_tokens,
                                    int64_t K, int E, int k, int32_t* idx, void* gate, hipStream_t st, const float* x_fq) {
  if constexpr (sizeof(T) != 2) {
    return false;
  } else {
    if (T_tokens < kWaveRouterMinTokens || E > 16 || K % 2048 != 0 || K > 8192) return false;
    if (!aligned16(x) || !aligned16(norm_w) || !aligned16(xn) || !aligned16(wr)) return false;
    const dim3 grid((unsigned)((T_tokens + 3) / 4));
    const size_t lds = (size_t)4 * K * 2;
#define STMOE_NRW(NCH, EP)                                                                                              \
  norm_router_wave_kernel<T, W, NCH, EP><<<grid, 256, lds, st>>>((const T*)x, (const W*)norm_w, eps, (T*)xn, (const T*)wr, \
                                                                 T_tokens, E, k, idx, (T*)gate, x_fq)
#define STMOE_NRW_E(NCH)      \
  do {                        \
    if (E <= 8) STMOE_NRW(NCH, 8); \
    else STMOE_NRW(NCH, 16);  \
  } while (0)
    switch (K / 512) {
      case 4: STMOE_NRW_E(4); break;
      case 8: STMOE_NRW_E(8); break;
      case 12: STMOE_NRW_E(12); break;
      default: STMOE_NRW_E(16); break;
    }
#undef STMOE_NRW_E
#undef STMOE_NRW
    return true;
  }
}

template <typename T, typename W, bool FUSE_NORM>
static int launch_router_wg(const void* x, const void* norm_w, float eps, void* xn, const void* wr, int64_t T_tokens,
                            int64_t K, int E, int k, void* logits, int32_t* idx, int64_t* idx64, void* gate, hipStream_t st,
                            SingleTokenDispatch disp = SingleTokenDispatch{nullptr, nullptr, nullptr, nullptr},
                            const float* x_fq = nullptr) {
  const size_t lds = ((K * sizeof(T) + 15) / 16) * 16 + (64 + 8 + 64) * sizeof(float);
  if (lds > 64 * 1024) return set_error(STMOE_ERR_UNSUPPORTED, "router: K=%lld does not fit the per-token LDS row", (long long)K);
  if (T_tokens <= 64)
    router_wg_kernel<T, W, FUSE_NORM, 8, false><<<dim3((unsigned)T_tokens), 512, lds, st>>>(
        (const T*)x, (const W*)norm_w, eps, (T*)xn, (const T*)wr, K, E, k, (T*)logits, idx, idx64, (T*)gate, disp, x_fq);
  else if (T_tokens <= 512)
    router_wg_kernel<T, W, FUSE_NORM, 4, false><<<dim3((unsigned)T_tokens), 512, lds, st>>>(
        (const T*)x, (const W*)norm_w, eps, (T*)xn, (const T*)wr, K, E, k, (T*)logits, idx, idx64, (T*)gate, disp, x_fq);
  else
    router_wg_kernel<T, W, FUSE_NORM, 0, true><<<dim3((unsigned)T_tokens), 512, lds, st>>>(
        (const T*)x, (const W*)norm_w, eps, (T*)xn, (const T*)wr, K, E, k, (T*)logits, idx, idx64, (T*)gate, disp, x_fq);
  return check_launch("router_wg");
}

// ffn_norm + router in one launch (used by the fused layer forward).  norm weight dtype: f32, or the activation dtype.
// With all four dispatch pointers given and T_tokens == 1 the launch also writes the token's dispatch arrays.
int norm_router(const void* h, int dtype, const void* norm_w, int w_dtype, float eps, void* xn, const void* wr,
                int64_t T_tokens, int64_t K, int E, int k, int32_t* idx, void* gate, hipStream_t st,
                int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* inv, const float* x_fq) {
  SingleTokenDispatch disp{nullptr, nullptr, nullptr, nullptr};
  if (T_tokens == 1 && counts && offsets && perm && inv) disp = SingleTokenDispatch{counts, offsets, perm, inv};
#define STMOE_NR(TT, WW)                                                                                                   \
  do {                                                                                                                     \
    if (launch_norm_router_wave<TT, WW>(h, norm_w, eps, xn, wr, T_tokens, K, E, k, idx, gate, st, x_fq)) return check_launch("norm_router_wave"); \
    return launch_router_wg<TT, WW, true>(h, norm_w, eps, xn, wr, T_tokens, K, E, k, nullptr, idx, nullptr, gate, st, disp, x_fq); \
  } while (0)
  if (dtype == STMOE_F32 && w_dtype == STMOE_F32) STMOE_NR(float, float);
  if (dtype == STMOE_F16 && w_dtype == STMOE_F32) STMOE_NR(f16_t, float);
  if (dtype == STMOE_BF16 && w_dtype == STMOE_F32) STMOE_NR(bf16_t, float);
  if (dtype == STMOE_F16 && w_dtype == STMOE_F16) STMOE_NR(f16_t, f16_t);
  if (dtype == STMOE_BF16 && w_dtype == STMOE_BF16) STMOE_NR(bf16_t, bf16_t);
#undef STMOE_NR
  return set_error(STMOE_ERR_DTYPE, "norm_router: dtype %d with weight dtype %d not implemented", dtype, w_dtype);
}

template <typename T>
static int launch_router(const void* x, const void* wr, int64_t T_tokens, int64_t K, int E, int k, void* logits,
                         int32_t* idx, int64_t* idx64, void* gate, hipStream_t st) {
  dim3 grid((unsigned)((T_tokens + 3) / 4));
#define STMOE_ROUTER_CASE(EP)                                                                               \
  router_topk_kernel<T, EP><<<grid, 256, 0, st>>>((const T*)x, (const T*)wr, T_tokens, K, E, k, (T*)logits, \
                                                  idx, idx64, (T*)gate)
  if (E <= 8) STMOE_ROUTER_CASE(8);
  else if (E <= 16) STMOE_ROUTER_CASE(16);
  else if (E <= 32) STMOE_ROUTER_CASE(32);
  else STMOE_ROUTER_CASE(64);
#undef STMOE_ROUTER_CASE
  return check_launch("router_topk");
}

// ---------------------------------------------------------------------------------------------------
// softmax over the last axis, one wavefront per row: values widened to fp32, p = expf(x - max) / sum, rounded to the
// output dtype (torch.nn.functional.softmax(x, dim=-1, dtype=...)).  Rows of at most 64 elements (router logits over the
// experts) are summed in index order by a serial loop over the lanes' values, the router kernels' own arithmetic, so
// that ranking these probabilities gives the router's choice; longer rows add lane-strided partial sums and combine
// them with the xor butterfly.
__device__ __forceinline__ float softmax_load(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case STMOE_F16: return (float)reinterpret_cast<const f16_t*>(p)[i];
    case STMOE_BF16: return bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
    default: return reinterpret_cast<const float*>(p)[i];
  }
}
__device__ __forceinline__ void softmax_store(void* p, int dtype, int64_t i, float v) {
  switch (dtype) {
    case STMOE_F16: reinterpret_cast<f16_t*>(p)[i] = (f16_t)v; break;
    case STMOE_BF16: reinterpret_cast<bf16_t*>(p)[i] = f32_to_bf16(v); break;
    default: reinterpret_cast<float*>(p)[i] = v; break;
  }
}
__global__ void __launch_bounds__(256)
softmax_rows_kernel(const void* __restrict__ x, int x_dtype, int64_t rows, int64_t cols, void* __restrict__ out, int o_dtype) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int64_t base = r * cols;
  if (cols <= 64) {
    const float l = lane < cols ? softmax_load(x, x_dtype, base + lane) : 0.0f;
    float mx = __shfl(l, 0);
    for (int e = 1; e < cols; ++e) mx = fmaxf(mx, __shfl(l, e));
    const float ex = softmax_exp(l - mx);
    float denom = 0.0f;
    for (int e = 0; e < cols; ++e) denom += __shfl(ex, e);
    if (lane < cols) softmax_store(out, o_dtype, base + lane, ex / denom);
    return;
  }
  float mx = -INFINITY;
  for (int64_t c = lane; c < cols; c += 64) mx = fmaxf(mx, softmax_load(x, x_dtype, base + c));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
  float sum = 0.0f;
  for (int64_t c = lane; c < cols; c += 64) sum += softmax_exp(softmax_load(x, x_dtype, base + c) - mx);
  sum = wave_xor_sum(sum);
  for (int64_t c = lane; c < cols; c += 64) softmax_store(out, o_dtype, base + c, softmax_exp(softmax_load(x, x_dtype, base + c) - mx) / sum);
}

}  // namespace stmoe

using namespace stmoe;

extern "C" int stmoe_rms_norm(const void* x, int dtype, const void* w, int w_dtype, int64_t T, int64_t K, float eps,
                              void* out, stmoe_stream_t stream) {
  STMOE_REQUIRE(T >= 0 && K > 0, STMOE_ERR_SHAPE, "rms_norm: T=%lld K=%lld", (long long)T, (long long)K);
  if (T == 0) return STMOE_OK;
  STMOE_REQUIRE(x && w && out, STMOE_ERR_NULL, "rms_norm: NULL pointer");
  STMOE_REQUIRE(T < 0x7fffffffLL, STMOE_ERR_SHAPE, "rms_norm: T too large");
  hipStream_t st = as_stream(stream);
  dim3 g((unsigned)T);
#define STMOE_RMS(TT, WW) rms_norm_kernel<TT, WW><<<g, 512, 0, st>>>((const TT*)x, (const WW*)w, K, eps, (TT*)out)
  if (dtype == STMOE_F32 && w_dtype == STMOE_F32) STMOE_RMS(float, float);
  else if (dtype == STMOE_F16 && w_dtype == STMOE_F32) STMOE_RMS(f16_t, float);
  else if (dtype == STMOE_BF16 && w_dtype == STMOE_F32) STMOE_RMS(bf16_t, float);
  else if (dtype == STMOE_F16 && w_dtype == STMOE_F16) STMOE_RMS(f16_t, f16_t);
  else if (dtype == STMOE_BF16 && w_dtype == STMOE_BF16) STMOE_RMS(bf16_t, bf16_t);
  else return set_error(STMOE_ERR_DTYPE, "rms_norm: dtype %d with weight dtype %d not implemented", dtype, w_dtype);
#undef STMOE_RMS
  return check_launch("rms_norm");
}

extern "C" int stmoe_router_topk(const void* x, const void* w_router, int dtype, int64_t T, int64_t K, int E, int k,
                                 void* logits_out, int32_t* idx_out, int64_t* idx64_out, void* gate_out,
                                 stmoe_stream_t stream) {
  STMOE_REQUIRE(T >= 0 && K > 0 && K % 8 == 0, STMOE_ERR_SHAPE, "router_topk: T=%lld, K=%lld (K must be a positive multiple of 8)",
                (long long)T, (long long)K);
  STMOE_REQUIRE(E >= 1 && E <= 64, STMOE_ERR_SHAPE, "router_topk: expert count %d outside 1..64", E);
  STMOE_REQUIRE(k >= 1 && k <= E, STMOE_ERR_SHAPE, "router_topk: top-k %d outside 1..%d", k, E);
  if (T == 0) return STMOE_OK;
  STMOE_REQUIRE(x && w_router && idx_out && gate_out, STMOE_ERR_NULL, "router_topk: NULL pointer");
  STMOE_REQUIRE(aligned16(x) && aligned16(w_router), STMOE_ERR_ALIGN, "router_topk: x and w_router must be 16-byte aligned");
  hipStream_t st = as_stream(stream);
  if (T < 0x7fffffffLL && K * dtype_size(dtype) <= 48 * 1024) {  // one workgroup per token: lower latency
    switch (dtype) {
      case STMOE_F32: return launch_router_wg<float, float, false>(x, nullptr, 0.f, nullptr, w_router, T, K, E, k, logits_out, idx_out, idx64_out, gate_out, st);
      case STMOE_F16: return launch_router_wg<f16_t, float, false>(x, nullptr, 0.f, nullptr, w_router, T, K, E, k, logits_out, idx_out, idx64_out, gate_out, st);
      case STMOE_BF16: return launch_router_wg<bf16_t, float, false>(x, nullptr, 0.f, nullptr, w_router, T, K, E, k, logits_out, idx_out, idx64_out, gate_out, st);
      default: return set_error(STMOE_ERR_DTYPE, "router_topk: dtype %d is not f32/f16/bf16", dtype);
    }
  }
  switch (dtype) {
    case STMOE_F32: return launch_router<float>(x, w_router, T, K, E, k, logits_out, idx_out, idx64_out, gate_out, st);
    case STMOE_F16: return launch_router<f16_t>(x, w_router, T, K, E, k, logits_out, idx_out, idx64_out, gate_out, st);
    case STMOE_BF16: return launch_router<bf16_t>(x, w_router, T, K, E, k, logits_out, idx_out, idx64_out, gate_out, st);
    default: return set_error(STMOE_ERR_DTYPE, "router_topk: dtype %d is not f32/f16/bf16", dtype);
  }
}

extern "C" int stmoe_softmax(const void* x, int x_dtype, int64_t rows, int64_t cols, void* out, int out_dtype, stmoe_stream_t stream) {
  STMOE_REQUIRE(rows >= 0 && cols > 0 && rows < 0x7fffffffLL * 4, STMOE_ERR_SHAPE, "softmax: rows=%lld cols=%lld", (long long)rows, (long long)cols);
  auto is_float = [](int d) { return d == STMOE_F32 || d == STMOE_F16 || d == STMOE_BF16; };
  STMOE_REQUIRE(is_float(x_dtype) && is_float(out_dtype), STMOE_ERR_DTYPE, "softmax: dtypes %d -> %d", x_dtype, out_dtype);
  if (rows == 0) return STMOE_OK;
  STMOE_REQUIRE(x && out, STMOE_ERR_NULL, "softmax: NULL pointer");
  softmax_rows_kernel<<<dim3((unsigned)((rows + 3) / 4)), 256, 0, as_stream(stream)>>>(x, x_dtype, rows, cols, out, out_dtype);
  return check_launch("softmax");
}
