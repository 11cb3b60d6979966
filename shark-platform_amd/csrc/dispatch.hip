// Token-to-expert dispatch (histogram, exclusive scan, stable permutation) and the weighted combine.
//
// The reference has no dispatch step: it gathers expert weights per token
// (sharktank/sharktank/layers/ffn_moe_block.py:37-41).  Grouping rows by expert instead needs a
// permutation; it is defined as the stable counting sort of the pairs p = t*k + j by expert id, so it
// is a pure function of the routing indices and can be checked bit for bit.
#include "stmoe_common.h"

namespace stmoe {

static constexpr int kDispatchThreads = 1024;
static constexpr int kDispatchWaves = kDispatchThreads / 64;

// One workgroup walks the pairs in chunks of 1024, in order.  LDS: base[E] (next free position of each
// expert) and wcnt[16][E] (per-wave counts of the current chunk).
__global__ void __launch_bounds__(kDispatchThreads)
dispatch_build_kernel(const int32_t* __restrict__ idx, int64_t n, int E, int32_t* __restrict__ counts,
                      int32_t* __restrict__ offsets, int32_t* __restrict__ perm, int32_t* __restrict__ inv,
                      int32_t* __restrict__ zero_words, int n_zero) {
  extern __shared__ int32_t sm[];
  int32_t* base = sm;
  int32_t* wcnt = sm + E;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (the fused layer forward has the ticket words of the projections' split reductions cleared here: a launch it makes anyway)
  if (tid < n_zero) zero_words[tid] = 0;

  for (int e = tid; e < E; e += kDispatchThreads) base[e] = 0;
  __syncthreads();
  for (int64_t i = tid; i < n; i += kDispatchThreads) {
    int e = idx[i];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);  // out-of-range ids are a caller error; clamp to stay in bounds
    atomicAdd(&base[e], 1);                // integer LDS atomics: the counts do not depend on their order
  }
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
      const int32_t c = base[e];
      counts[e] = c;
      offsets[e] = run;
      base[e] = run;
      run += c;
    }
    offsets[E] = run;
  }
  __syncthreads();

  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int64_t c0 = 0; c0 < n; c0 += kDispatchThreads) {
    const int64_t i = c0 + tid;
    int e = -1;
    if (i < n) {
      e = idx[i];
      e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    }
    int my_rank = 0;
    for (int ee = 0; ee < E; ++ee) {
      const uint64_t mask = __ballot(e == ee);
      if (e == ee) my_rank = __popcll(mask & lt_mask);
      if (lane == 0) wcnt[wave * E + ee] = __popcll(mask);
    }
    __syncthreads();
    if (i < n) {
      int32_t pos = base[e] + my_rank;
      for (int w = 0; w < wave; ++w) pos += wcnt[w * E + e];
      perm[pos] = (int32_t)i;
      inv[i] = pos;
    }
    __syncthreads();
    for (int ee = tid; ee < E; ee += kDispatchThreads) {
      int32_t s = 0;
      for (int w = 0; w < kDispatchWaves; ++w) s += wcnt[w * E + ee];
      base[ee] += s;
    }
    __syncthreads();
  }
}

// The same result for launches of at most 8 chunks of 1024 pairs and at most 64 experts (a prefill batch of 4096 tokens
// with top-2 routing), with three barriers in all instead of three per chunk: every thread fetches its pair of every
// chunk at once (one memory latency instead of one per chunk and pass), the per-wavefront counts of all chunks go to
// LDS in one sweep, one thread per expert turns its column of counts (chunk by chunk, wavefront by wavefront: the order
// of the pairs) into running positions, and after the scan over the experts every pair knows its place.
static constexpr int kDispatchRegChunks = 8;
static constexpr int kDispatchRegExperts = 64;
__global__ void __launch_bounds__(kDispatchThreads)
dispatch_build_reg_kernel(const int32_t* __restrict__ idx, int n, int E, int32_t* __restrict__ counts,
                          int32_t* __restrict__ offsets, int32_t* __restrict__ perm, int32_t* __restrict__ inv,
                          int32_t* __restrict__ zero_words, int n_zero) {
  extern __shared__ int32_t sm[];
  int32_t* cnt = sm;  // [chunk][wavefront][E]: count, then the position of the wavefront's first pair inside its expert
  int32_t* first = sm + kDispatchRegChunks * kDispatchWaves * E;  // [E] first row of each expert
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid < n_zero) zero_words[tid] = 0;
  const int chunks = (n + kDispatchThreads - 1) / kDispatchThreads;
  int e[kDispatchRegChunks], rank[kDispatchRegChunks];
#pragma unroll
  for (int c = 0; c < kDispatchRegChunks; ++c) {
    const int i = c * kDispatchThreads + tid;
    e[c] = i < n ? idx[i] : -1;
  }
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int c = 0; c < kDispatchRegChunks; ++c) {
    if (c < chunks) {
      if (e[c] >= E) e[c] = E - 1;  // out-of-range ids are a caller error; clamp to stay in bounds
      if (e[c] < 0 && c * kDispatchThreads + tid < n) e[c] = 0;
      rank[c] = 0;
      for (int ee = 0; ee < E; ++ee) {
        const uint64_t mask = __ballot(e[c] == ee);
        if (e[c] == ee) rank[c] = __popcll(mask & lt_mask);
        if (lane == 0) cnt[(c * kDispatchWaves + wave) * E + ee] = __popcll(mask);
      }
    }
  }
  __syncthreads();
  if (tid < E) {
    int32_t run = 0;
    for (int c = 0; c < chunks; ++c) {
      int32_t v[kDispatchWaves];  // a chunk's sixteen counts are read together, not one after the other
#pragma unroll
      for (int w = 0; w < kDispatchWaves; ++w) v[w] = cnt[(c * kDispatchWaves + w) * E + tid];
#pragma unroll
      for (int w = 0; w < kDispatchWaves; ++w) {
        cnt[(c * kDispatchWaves + w) * E + tid] = run;
        run += v[w];
      }
    }
    counts[tid] = run;
    first[tid] = run;
  }
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0;
    for (int ee = 0; ee < E; ++ee) {
      const int32_t c = first[ee];
      offsets[ee] = run;
      first[ee] = run;
      run += c;
    }
    offsets[E] = run;
  }
  __syncthreads();
#pragma unroll
  for (int c = 0; c < kDispatchRegChunks; ++c) {
    const int i = c * kDispatchThreads + tid;
    if (i < n) {
      const int32_t pos = first[e[c]] + cnt[(c * kDispatchWaves + wave) * E + e[c]] + rank[c];
      perm[pos] = i;
      inv[i] = pos;
    }
  }
}

// The same result for at most 64 pairs and 64 experts (a decode step of 32 tokens with top-2 routing): one wavefront, lane i
// owns pair i, no LDS and no barrier.  For every expert a ballot gives its count (kept by lane `expert`) and the rank of
// each of its pairs; the scan over the experts runs on values read from the lanes.
__global__ void __launch_bounds__(64)
dispatch_build_wave_kernel(const int32_t* __restrict__ idx, int n, int E, int32_t* __restrict__ counts,
                           int32_t* __restrict__ offsets, int32_t* __restrict__ perm, int32_t* __restrict__ inv,
                           int32_t* __restrict__ zero_words, int n_zero) {
  const int lane = threadIdx.x;
  for (int i = lane; i < n_zero; i += 64) zero_words[i] = 0;
  int e = lane < n ? idx[lane] : -1;
  if (lane < n) e = e < 0 ? 0 : (e >= E ? E - 1 : e);  // out-of-range ids are a caller error; clamp to stay in bounds
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  int rank = 0, count = 0;  // of pair `lane` inside its expert; of expert `lane`
  for (int ee = 0; ee < E; ++ee) {
    const uint64_t mask = __ballot(e == ee);
    if (e == ee) rank = __popcll(mask & lt_mask);
    if (lane == ee) count = __popcll(mask);
  }
  int first = 0, run = 0;  // first row of expert `lane`
  for (int ee = 0; ee < E; ++ee) {
    if (lane == ee) first = run;
    run += __builtin_amdgcn_readlane(count, ee);
  }
  if (lane < E) {
    counts[lane] = count;
    offsets[lane] = first;
  }
  if (lane == 0) offsets[E] = run;
  const int first_of_mine = __shfl(first, e < 0 ? 0 : e, 64);
  if (lane < n) {
    const int pos = first_of_mine + rank;
    perm[pos] = lane;
    inv[lane] = pos;
  }
}

// One workgroup per token; every thread owns 8 consecutive features (16-byte loads for 16-bit types).
// o = sum over slots of round(gate * y) (fp32 sum in slot order, rounded to T); optional RMS norm of o;
// optional residual add.
template <typename T> struct Row8 {
  float v[8];
  __device__ __forceinline__ void load(const T* p) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = Cvt<T>::to_f32(p[i]);
  }
  __device__ __forceinline__ void store(T* p) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) p[i] = Cvt<T>::from_f32(v[i]);
  }
};

template <typename T, typename W>
__global__ void __launch_bounds__(256)
combine_kernel(const T* __restrict__ y, const T* __restrict__ gate, const int32_t* __restrict__ inv, int k,
               int64_t K, const W* __restrict__ norm_w, float eps, const T* __restrict__ residual,
               T* __restrict__ out) {
  __shared__ float partial[4];
  const int64_t t = blockIdx.x;
  T* orow = out + t * K;
  float ss = 0.0f;
  for (int64_t i = (int64_t)threadIdx.x * 8; i < K; i += 256 * 8) {
    float acc[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) acc[q] = 0.0f;
    for (int j = 0; j < k; ++j) {
      const int64_t r = inv[t * k + j];
      const float g = Cvt<T>::to_f32(gate[t * k + j]);
      Row8<T> yv;
      yv.load(y + r * K + i);
#pragma unroll
      for (int q = 0; q < 8; ++q) acc[q] += round_to<T>(__fmul_rn(g, yv.v[q]));
    }
    Row8<T> o;
#pragma unroll
    for (int q = 0; q < 8; ++q) o.v[q] = round_to<T>(acc[q]);
    if (norm_w) {
#pragma unroll
      for (int q = 0; q < 8; ++q) ss = fmaf(o.v[q], o.v[q], ss);
    } else if (residual) {
      Row8<T> h;
      h.load(residual + t * K + i);
#pragma unroll
      for (int q = 0; q < 8; ++q) o.v[q] = round_to<T>(h.v[q] + o.v[q]);
    }
    o.store(orow + i);
  }
  if (!norm_w) return;
  ss = wave_xor_sum(ss);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float rs = rms_scale(total, K, eps);
  for (int64_t i = (int64_t)threadIdx.x * 8; i < K; i += 256 * 8) {  // each thread re-reads only what it wrote itself
    Row8<T> o;
    o.load(orow + i);
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      float v = round_to<W>(keep_f32(__fmul_rn(o.v[q], rs)));
      v = round_to<T>(round_to<W>(keep_f32(__fmul_rn(Cvt<W>::to_f32(norm_w[i + q]), v))));
      if (residual) v = round_to<T>(Cvt<T>::to_f32(residual[t * K + i + q]) + v);
      o.v[q] = v;
    }
    o.store(orow + i);
  }
}

// out[r, :] = round(g[r] * y[r, :]) ("me,men->men": the gate weighting before the slot sum)
template <typename T>
__global__ void __launch_bounds__(256)
scale_rows_kernel(const T* __restrict__ y, const T* __restrict__ g, int64_t K, T* __restrict__ out) {
  const int64_t r = blockIdx.x;
  const float gv = Cvt<T>::to_f32(g[r]);
  for (int64_t i = threadIdx.x; i < K; i += 256)
    out[r * K + i] = Cvt<T>::from_f32(keep_f32(__fmul_rn(gv, Cvt<T>::to_f32(y[r * K + i]))));
}

int dispatch_build(const int32_t* idx, int64_t n_pairs, int E, int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* inv,
                   int32_t* zero_words, int n_zero, hipStream_t st) {
  STMOE_REQUIRE(n_pairs >= 0 && n_pairs < 0x7fffffffLL, STMOE_ERR_SHAPE, "dispatch_build: n_pairs=%lld", (long long)n_pairs);
  STMOE_REQUIRE(E >= 1 && E <= 1024, STMOE_ERR_SHAPE, "dispatch_build: expert count %d outside 1..1024", E);
  STMOE_REQUIRE(counts && offsets, STMOE_ERR_NULL, "dispatch_build: counts/offsets NULL");
  STMOE_REQUIRE(n_pairs == 0 || (idx && perm && inv), STMOE_ERR_NULL, "dispatch_build: idx/perm/inv NULL");
  STMOE_REQUIRE(n_zero >= 0 && n_zero <= kDispatchThreads && (n_zero == 0 || zero_words), STMOE_ERR_SHAPE, "dispatch_build: %d words to clear", n_zero);
  if (n_pairs <= 64 && E <= 64) {
    dispatch_build_wave_kernel<<<1, 64, 0, st>>>(idx, (int)n_pairs, E, counts, offsets, perm, inv, zero_words, n_zero);
    return check_launch("dispatch_build");
  }
  if (n_pairs <= kDispatchRegChunks * kDispatchThreads && E <= kDispatchRegExperts) {
    const size_t lds = sizeof(int32_t) * (size_t)E * (kDispatchRegChunks * kDispatchWaves + 1);
    dispatch_build_reg_kernel<<<1, kDispatchThreads, lds, st>>>(idx, (int)n_pairs, E, counts, offsets, perm, inv, zero_words, n_zero);
    return check_launch("dispatch_build");
  }
  const size_t lds = sizeof(int32_t) * (size_t)E * (1 + kDispatchWaves);
  dispatch_build_kernel<<<1, kDispatchThreads, lds, st>>>(idx, n_pairs, E, counts, offsets, perm, inv, zero_words, n_zero);
  return check_launch("dispatch_build");
}

// out[r, c] = O(y[r, c] + bias[c]): the bias add of `linear` (sharktank/sharktank/ops/default_impls.py:328-341), each
// operand widened to fp32 (exact), one fp32 add, one rounding to the promoted dtype O, as eager torch computes it.
__device__ __forceinline__ float load_f32(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case STMOE_F16: return (float)reinterpret_cast<const f16_t*>(p)[i];
    case STMOE_BF16: return bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
    default: return reinterpret_cast<const float*>(p)[i];
  }
}
__device__ __forceinline__ void store_f32(void* p, int dtype, int64_t i, float v) {
  switch (dtype) {
    case STMOE_F16: reinterpret_cast<f16_t*>(p)[i] = (f16_t)v; break;
    case STMOE_BF16: reinterpret_cast<bf16_t*>(p)[i] = f32_to_bf16(v); break;
    default: reinterpret_cast<float*>(p)[i] = v; break;
  }
}
__global__ void __launch_bounds__(256)
add_bias_kernel(const void* __restrict__ y, int y_dtype, const void* __restrict__ bias, int b_dtype, int64_t cols,
                void* __restrict__ out, int o_dtype) {
  const int64_t r = blockIdx.x;
  for (int64_t c = threadIdx.x; c < cols; c += 256)
    store_f32(out, o_dtype, r * cols + c, __fadd_rn(load_f32(y, y_dtype, r * cols + c), load_f32(bias, b_dtype, c)));
}

}  // namespace stmoe

using namespace stmoe;

extern "C" int stmoe_scale_rows(const void* y, const void* g, int dtype, int64_t rows, int64_t K, void* out,
                                stmoe_stream_t stream) {
  STMOE_REQUIRE(rows >= 0 && K > 0 && rows < 0x7fffffffLL, STMOE_ERR_SHAPE, "scale_rows: rows=%lld K=%lld", (long long)rows, (long long)K);
  if (rows == 0) return STMOE_OK;
  STMOE_REQUIRE(y && g && out, STMOE_ERR_NULL, "scale_rows: NULL pointer");
  hipStream_t st = as_stream(stream);
  dim3 grid((unsigned)rows);
  switch (dtype) {
    case STMOE_F32: scale_rows_kernel<float><<<grid, 256, 0, st>>>((const float*)y, (const float*)g, K, (float*)out); break;
    case STMOE_F16: scale_rows_kernel<f16_t><<<grid, 256, 0, st>>>((const f16_t*)y, (const f16_t*)g, K, (f16_t*)out); break;
    case STMOE_BF16: scale_rows_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)y, (const bf16_t*)g, K, (bf16_t*)out); break;
    default: return set_error(STMOE_ERR_DTYPE, "scale_rows: dtype %d is not f32/f16/bf16", dtype);
  }
  return check_launch("scale_rows");
}

extern "C" int stmoe_add_bias(const void* y, int y_dtype, const void* bias, int bias_dtype, int64_t rows, int64_t cols, void* out,
                              int out_dtype, stmoe_stream_t stream) {
  STMOE_REQUIRE(rows >= 0 && cols > 0 && rows < 0x7fffffffLL, STMOE_ERR_SHAPE, "add_bias: rows=%lld cols=%lld", (long long)rows, (long long)cols);
  auto is_float = [](int d) { return d == STMOE_F32 || d == STMOE_F16 || d == STMOE_BF16; };
  STMOE_REQUIRE(is_float(y_dtype) && is_float(bias_dtype) && is_float(out_dtype), STMOE_ERR_DTYPE, "add_bias: dtypes %d + %d -> %d", y_dtype, bias_dtype, out_dtype);
  // torch's promotion: equal dtypes stay, everything else (f16 + bf16 included) goes to f32
  const int promoted = y_dtype == bias_dtype ? y_dtype : STMOE_F32;
  STMOE_REQUIRE(out_dtype == promoted, STMOE_ERR_DTYPE, "add_bias: dtypes %d + %d give %d, not %d", y_dtype, bias_dtype, promoted, out_dtype);
  if (rows == 0) return STMOE_OK;
  STMOE_REQUIRE(y && bias && out, STMOE_ERR_NULL, "add_bias: NULL pointer");
  add_bias_kernel<<<dim3((unsigned)rows), 256, 0, as_stream(stream)>>>(y, y_dtype, bias, bias_dtype, cols, out, out_dtype);
  return check_launch("add_bias");
}

extern "C" int stmoe_dispatch_build(const int32_t* idx, int64_t n_pairs, int E, int32_t* counts, int32_t* offsets,
                                    int32_t* perm, int32_t* inv, stmoe_stream_t stream) {
  return dispatch_build(idx, n_pairs, E, counts, offsets, perm, inv, nullptr, 0, as_stream(stream));
}

extern "C" int stmoe_combine(const void* y_sorted, const void* gate, const int32_t* inv, int dtype, int64_t T, int k,
                             int64_t K, const void* out_norm_w, int w_dtype, float eps, const void* residual,
                             void* out, stmoe_stream_t stream) {
  STMOE_REQUIRE(T >= 0 && K > 0 && K % 8 == 0 && k >= 1, STMOE_ERR_SHAPE, "combine: T=%lld K=%lld (a multiple of 8) k=%d",
                (long long)T, (long long)K, k);
  if (T == 0) return STMOE_OK;
  STMOE_REQUIRE(y_sorted && gate && inv && out, STMOE_ERR_NULL, "combine: NULL pointer");
  STMOE_REQUIRE(T < 0x7fffffffLL, STMOE_ERR_SHAPE, "combine: T too large");
  hipStream_t st = as_stream(stream);
  dim3 g((unsigned)T);
  const int wd = out_norm_w ? w_dtype : STMOE_F32;
#define STMOE_COMBINE(TT, WW)                                                                               \
  combine_kernel<TT, WW><<<g, 256, 0, st>>>((const TT*)y_sorted, (const TT*)gate, inv, k, K, (const WW*)out_norm_w, \
                                            eps, (const TT*)residual, (TT*)out)
  if (dtype == STMOE_F32 && wd == STMOE_F32) STMOE_COMBINE(float, float);
  else if (dtype == STMOE_F16 && wd == STMOE_F32) STMOE_COMBINE(f16_t, float);
  else if (dtype == STMOE_BF16 && wd == STMOE_F32) STMOE_COMBINE(bf16_t, float);
  else if (dtype == STMOE_F16 && wd == STMOE_F16) STMOE_COMBINE(f16_t, f16_t);
  else if (dtype == STMOE_BF16 && wd == STMOE_BF16) STMOE_COMBINE(bf16_t, bf16_t);
  else return set_error(STMOE_ERR_DTYPE, "combine: dtype %d with norm weight dtype %d not implemented", dtype, w_dtype);
#undef STMOE_COMBINE
  return check_launch("combine");
}
