/*
 * C ABI of the MI355X (gfx950) quantized mixture-of-experts kernels.
 *
 * The library computes what sharktank's eager `MoeBlock` / `PreGatherFFNMOE`
 * compute (sharktank/sharktank/layers/mixture_of_experts_block.py:64-90,
 * sharktank/sharktank/layers/ffn_moe_block.py:60-74) and what its IREE custom
 * ops `mmt_block_scaled_q8`, `mmt_block_scaled_offset_q4_unsigned` and
 * `einsum_2args_q4` compute (sharktank/sharktank/kernels/ *.py), on device
 * pointers, without any torch type in a signature.
 *
 * Conventions for every entry point:
 *   - all pointers are device pointers unless the comment says "host";
 *   - tensors are dense row-major; quantized planes are the planar planes of
 *     the reference layouts (`d`, `qs`, `m`), made contiguous by the caller;
 *   - the caller owns all memory, including the workspace; the library
 *     allocates nothing, never synchronises and only enqueues on `stream`
 *     (a hipStream_t passed as void*; NULL is the default stream);
 *   - host-side state is limited to a thread-local error string, one flag per
 *     device and kernel that records that the kernel's LDS reservation has been
 *     raised (hipFuncSetAttribute, on the kernel's first launch on that device:
 *     run every shape once eagerly before capturing launches into a HIP graph),
 *     and the per-device address of the built-in workspace of
 *     stmoe_moe_forward_static;
 *   - the return value is a stmoe_status; stmoe_last_error() returns a
 *     thread-local, human-readable description of the last non-zero status.
 */
#ifndef SHARKTANK_MOE_HIP_H_
#define SHARKTANK_MOE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* stmoe_stream_t;

typedef enum {
  STMOE_OK = 0,
  STMOE_ERR_NULL = 1,        /* a required pointer is NULL */
  STMOE_ERR_SHAPE = 2,       /* a size is negative, zero where it may not be, or not a multiple the kernel needs */
  STMOE_ERR_DTYPE = 3,       /* dtype enum out of range or combination not implemented */
  STMOE_ERR_ALIGN = 4,       /* a pointer is not aligned to 16 bytes */
  STMOE_ERR_UNSUPPORTED = 5, /* layout / format combination not implemented */
  STMOE_ERR_WORKSPACE = 6,   /* workspace smaller than *_workspace_bytes() */
  STMOE_ERR_LAUNCH = 7       /* hipGetLastError() after a launch was not hipSuccess */
} stmoe_status;

typedef enum {
  STMOE_F32 = 0,
  STMOE_F16 = 1,
  STMOE_BF16 = 2,
  STMOE_F8E4M3FN = 3, /* OCP e4m3 (torch.float8_e4m3fn), the fp8 format of gfx950 MFMA */
  STMOE_I8 = 4,
  STMOE_U8 = 5
} stmoe_dtype;

typedef enum {
  STMOE_ACT_SILU = 0,    /* torch.nn.functional.silu */
  STMOE_ACT_GELU_ERF = 1 /* torch.nn.functional.gelu, exact erf form */
} stmoe_act;

typedef enum {
  STMOE_W_DENSE = 0, /* DefaultPrimitiveTensor: qs = elements of `dtype` */
  STMOE_W_Q8_0 = 1,  /* BlockScaledLayout, block 32: d fp16 [.,K/32], qs int8 [.,K/32,32] */
  STMOE_W_Q4_1 = 2,  /* BlockScaledI4Layout, block 32, unsigned: d,m fp16 [.,K/32], qs u8 [.,K/32,16] */
                     /* (the matrix-multiply kernels on the PACKED form need finite block scales with |d| < 64:
                      * they remove the nibbles' exponent bias with one fused multiply-add whose constant term is
                      * 1024 * d in fp16.  Larger scales give NaN there without an error; the planar form and the
                      * dequant entry points have no such limit.  The Python binding checks the scale plane once
                      * before it prepacks a tensor and keeps tensors beyond the limit planar; a C caller that
                      * cannot rule such scales out does the same.) */
  STMOE_W_FP8 = 3,   /* TensorScaledLayout: qs e4m3fn [.,K], d = d_count scales of `dtype` (f32 or f16) */
  /* The same bytes re-ordered by stmoe_prepack() into the order the matrix-core kernels stream (every wavefront
   * load is one contiguous kilobyte; see stmoe_prepack).  Plane sizes are unchanged. */
  STMOE_W_Q8_0_PACKED = 4,
  STMOE_W_Q4_1_PACKED = 5,
  STMOE_W_FP8_PACKED = 6
} stmoe_wfmt;

/* One stacked expert weight `[experts, rows, cols]`, used as x @ W[e]^T. */
typedef struct stmoe_weight {
  int32_t format;  /* stmoe_wfmt */
  int32_t dtype;   /* DENSE: element dtype (F32/F16/BF16); FP8: dtype of d (F32/F16); else ignored */
  int64_t experts; /* E; 1 for a plain matrix */
  int64_t rows;    /* output features of the projection */
  int64_t cols;    /* reduction length; multiple of 32 for the block formats */
  const void* qs;
  const void* d;   /* NULL for DENSE */
  const void* m;   /* Q4_1 only */
  int64_t d_count; /* FP8: 1 (one scale per tensor) or `experts` (one per expert) */
} stmoe_weight;

const char* stmoe_last_error(void);
int stmoe_abi_version(void);

/* ---- dequantization (bit-exact with the reference layouts' dequant()) ---------------------- */

/* BlockScaledLayout.dequant (sharktank/sharktank/types/layouts.py:274-290):
 * out[b,i] = D(d[b]) * D(qs[b,i]) (+ D(m[b])), every step rounded in out_dtype D. */
int stmoe_dequant_block_scaled(const void* d, const void* m /*nullable*/, int dm_dtype,
                               const int8_t* qs, int64_t n_blocks, int block_size,
                               void* out, int out_dtype, stmoe_stream_t stream);

/* BlockScaledI4Layout.dequant (layouts.py:302-357 + layout_utils.py:67-86): nibbles in linear
 * little-endian order (element 2i = low nibble of byte i), unsigned or sign-extended. */
int stmoe_dequant_block_scaled_i4(const void* d, const void* m /*nullable*/, int dm_dtype,
                                  const uint8_t* qs_packed, int64_t n_blocks, int block_size,
                                  int is_signed, void* out, int out_dtype, stmoe_stream_t stream);

/* promote_linear_i4_block_to_i8 (layout_utils.py:67-86): n_bytes packed bytes -> 2*n_bytes (u)int8. */
int stmoe_promote_i4(const uint8_t* qs_packed, int64_t n_bytes, int is_signed, void* out,
                     stmoe_stream_t stream);

/* TensorScaledLayout.dequant (layouts.py:163-181): out = ((D(qs) - m) * d).to(out_dtype) with
 * D = d_dtype. `d`/`m` hold d_count values; value j applies to elements [j*n/d_count, (j+1)*n/d_count). */
int stmoe_dequant_tensor_scaled(const void* qs, int qs_dtype, const void* d, const void* m /*nullable*/,
                                int d_dtype, int64_t d_count, int64_t n, void* out, int out_dtype,
                                stmoe_stream_t stream);

/* StaticScaledQuantizer per-tensor quantize to fp8 (sharktank/sharktank/types/quantizers.py:153-183 with
 * saturate_cast, layout_utils.py:150-176): out = e4m3fn(clamp(x / rscale, -448, 448)); the quotient is
 * computed in fp32 and rounded to x's dtype before the clamp.  `rscale` points to one device float. */
int stmoe_quantize_fp8(const void* x, int x_dtype, const float* rscale, int64_t n, void* out_fp8,
                       stmoe_stream_t stream);

/* StaticScaledQuantizer per-axis quantize to fp8 (sharktank/sharktank/types/quantizers.py:184-230): with j the index along
 * the scaled axis (`axis_len` entries, `inner` elements behind it: element i has j = (i / inner) % axis_len),
 * out = e4m3fn(clamp(x * scale[j], -448, 448)); the product is computed in the dtype eager torch gives the two tensors'
 * product: x's dtype when the scales have it, fp32 otherwise (scale_dtype f32).  The matching TensorScaledLayout holds
 * d = reciprocal scales, broadcast along the same axis: stmoe_dequant_tensor_scaled_per_axis. */
int stmoe_quantize_fp8_per_axis(const void* x, int x_dtype, const void* scale, int scale_dtype, int64_t axis_len,
                                int64_t inner, int64_t n, void* out_fp8, stmoe_stream_t stream);

/* TensorScaledLayout.dequant (layouts.py:163-181) with d (and m) of `axis_len` values broadcast along one axis that has
 * `inner` elements behind it: out = ((D(qs) - m[j]) * d[j]).to(out_dtype), j = (i / inner) % axis_len, D = d_dtype. */
int stmoe_dequant_tensor_scaled_per_axis(const void* qs, int qs_dtype, const void* d, const void* m /*nullable*/,
                                         int d_dtype, int64_t axis_len, int64_t inner, int64_t n, void* out,
                                         int out_dtype, stmoe_stream_t stream);

/* DynamicScaledQuantizer._quantize_raw_tensor for float8_e4m3fn (sharktank/sharktank/types/quantizers.py:368-389):
 * amax = max|x|; scale = T(T(1 / max(amax, eps)) * 448) (torch evaluates the reference's `finfo.max / amax.clamp(eps)`, a
 * number over a tensor, as reciprocal times number), eps = finfo(float8_e4m3fn).eps = 0.125; rscale = T(1 / scale);
 * out = e4m3fn(clamp(T(x * scale))), every step in x's dtype T as eager torch computes it.  scale_rscale_out receives
 * {scale, rscale} (the T values, widened to fp32); `scratch` is device memory of at least
 * stmoe_dynamic_quantize_fp8_scratch_bytes() bytes.  Two launches, no synchronisation. */
size_t stmoe_dynamic_quantize_fp8_scratch_bytes(void);
int stmoe_dynamic_quantize_fp8(const void* x, int dtype, int64_t n, void* out_fp8, float* scale_rscale_out, void* scratch,
                               size_t scratch_bytes, stmoe_stream_t stream);

/* quantize(x).unpack().dequant() of the same quantizer in one pass (the fake-quantised activations of
 * sharktank/sharktank/layers/linear.py:72-78): out = T(f32(e4m3fn(clamp(T(x / rscale)))) * rscale), T = `dtype`. */
int stmoe_fake_quant_fp8(const void* x, int dtype, const float* rscale, int64_t n, void* out, stmoe_stream_t stream);

/* Load-time re-ordering of a planar quantized weight into the streaming order (and back).  For every tile of 16
 * consecutive rows: samples as [K/64][lane = 16*g + n][16 B] (Q8_0, fp8: row n, k = 64*kb + 16*g..+15) or
 * [K/128][lane][16 B] (Q4_1: row n, block 4*kb + g; inside every dword the even elements fill the low half-word and
 * the odd ones the high half-word); block scales/offsets as [K/256][16 rows][8] fp16.  A pure permutation of bytes
 * (of nibbles for Q4_1): stmoe_unpack(stmoe_prepack(w)) == w bit for bit.  `planar` and `packed` describe the same
 * [experts, rows, cols] with formats X and X_PACKED and caller-owned planes of equal sizes; rows % 16 == 0 and
 * cols % 256 == 0.  The reference has no counterpart (its planes come from GGUF blocks,
 * sharktank/sharktank/types/gguf_interop/layouts.py:51-60,285-300, and are consumed row-major). */
int stmoe_prepack(const stmoe_weight* planar, const stmoe_weight* packed_out, stmoe_stream_t stream);
int stmoe_unpack(const stmoe_weight* packed, const stmoe_weight* planar_out, stmoe_stream_t stream);

typedef enum {
  STMOE_GGUF_Q8_0 = 0, /* ggml block_q8_0 {f16 d; i8 qs[32]}, 34 bytes */
  STMOE_GGUF_Q4_1 = 1  /* ggml block_q4_1 {f16 d; f16 m; u8 qs[16]}, 20 bytes; byte i = element i (low nibble), i + 16 (high) */
} stmoe_gguf_type;

/* Raw GGUF blocks -> weight planes in one pass: Q8_0.unpack (sharktank/sharktank/types/gguf_interop/layouts.py:51-60)
 * and Q4_1.unpack (:285-300) with linearize_interleaved_i4_block (sharktank/sharktank/types/layout_utils.py:20-44).
 * `raw_blocks` holds experts*rows*cols/32 blocks, row-major, 2-byte aligned.  `out` describes caller-owned planes of
 * format STMOE_W_Q8_0 / STMOE_W_Q4_1 (the reference's planar planes, bit for bit) or of the matching _PACKED format
 * (the streaming order of stmoe_prepack, written directly: rows % 16 == 0 and cols % 256 == 0). */
int stmoe_gguf_ingest(const void* raw_blocks, int gguf_type, const stmoe_weight* out, stmoe_stream_t stream);

/* ---- layer pieces ----------------------------------------------------------------------------- */

/* RMSNormLayer.forward (sharktank/sharktank/layers/norm.py:34-41) with rms_norm_default
 * (sharktank/sharktank/ops/default_impls.py:402-408): fp32 statistics, weight `w` of w_dtype, result
 * rounded to the dtype of x.  x, out: [T, K]. */
int stmoe_rms_norm(const void* x, int dtype, const void* w, int w_dtype, int64_t T, int64_t K, float eps,
                   void* out, stmoe_stream_t stream);

/* Router of MoeBlock.forward (mixture_of_experts_block.py:70-83): logits = x @ Wr^T rounded to `dtype`,
 * fp32 softmax over E, top-k of the fp32 probabilities (descending; equal probabilities -> lower expert index first,
 * also where distinct logits round to one probability), gates renormalised
 * in fp32 then rounded to `dtype`.  Wr [E,K] is given in `dtype`.  K % 8 == 0, E <= 64, k <= E.
 * logits_out ([T,E], `dtype`) and idx64_out ([T,k], int64) may be NULL. */
int stmoe_router_topk(const void* x, const void* w_router, int dtype, int64_t T, int64_t K, int E, int k,
                      void* logits_out, int32_t* idx_out, int64_t* idx64_out, void* gate_out,
                      stmoe_stream_t stream);

/* Token-to-expert dispatch: a stable counting sort of the n_pairs = T*k (token, slot) pairs
 * p = t*k + j by expert id.  counts[E]; offsets[E+1] = exclusive scan; perm[offsets[e]+r] = the r-th
 * pair of expert e in increasing p; inv[perm[i]] = i.  The reference has no such step (it gathers
 * weights per token instead, ffn_moe_block.py:37-41); this is what replaces it.
 * Expert ids outside 0..E-1 are clamped into the range, not reported (the reference's weights[experts] would raise
 * IndexError): a caller that cannot trust its ids checks them first; the Python layer does when
 * TURBINE_LLM_DEBUG=enable_nan_checks is set. */
int stmoe_dispatch_build(const int32_t* idx, int64_t n_pairs, int E, int32_t* counts, int32_t* offsets,
                         int32_t* perm, int32_t* inv, stmoe_stream_t stream);

/* Workspace for stmoe_grouped_ffn / stmoe_moe_forward (bytes; depends on sizes only).  A single matrix (E == 1) of
 * 33..128 rows runs up to 1.5 times faster when the caller appends stmoe_mmt_workspace_bytes(T * k) bytes to the size
 * stmoe_grouped_ffn_workspace_bytes returns (scratch for reductions split over several workgroups; launches of more than
 * 128 rows have it inside the queried size, smaller grouped launches do not use any). */
size_t stmoe_grouped_ffn_workspace_bytes(int64_t T, int k, int64_t K, int64_t N, int dtype);
size_t stmoe_moe_forward_workspace_bytes(int64_t T, int k, int E, int64_t K, int64_t N, int dtype);

/* Gated expert FFN of PreGatherFFNMOE.forward (ffn_moe_block.py:60-72) over rows grouped by expert:
 * for sorted position i (pair p = perm[i], token t = p / k, expert e with offsets[e] <= i < offsets[e+1])
 *   y[i,:] = Wd[e] . ( act(Wg[e] . x[t]) * (Wu[e] . x[t]) )
 * with each intermediate rounded to `dtype` where the reference materialises a tensor.  x [T,K];
 * y [T*k, K] in `dtype`.
 * Quantised activations: `x_scale` / `z_scale` (nullable; each one device float) are the reciprocal scales of static
 * per-tensor e4m3fn quantizers (StaticScaledQuantizer, quantizers.py:153-183) applied to x before the gate/up
 * projections and to the intermediate before the down projection.  The reference semantics is quantise then
 * dequantise (`quantize(x).unpack().dequant()`, sharktank/sharktank/layers/linear.py:72-78) followed by the
 * floating-point path: quantise, dequantise, 16-bit kernels, every rounding where the reference rounds (the quantizers are
 * applied by the kernels that produce the tensors).  With FP8 weights the other arithmetic is to feed both operands to the
 * fp8 matrix cores as bytes and scale the fp32 dot product once by scale_x * d_w, which skips the rounding of the
 * dequantised operands to `dtype` (variant 5; variant 7: the same on the general 128x128 tile kernel only).  Variant 0
 * takes the matrix-core arithmetic where it is both much faster and well inside the fp8 tolerance of 2e-2 (packed FP8
 * weights with fp32 scales, both quantizers, F16 activations, at least 320 rows, K and N multiples of 256) and the
 * step-by-step arithmetic everywhere else (BF16 activations included); variant 8 never leaves the step-by-step arithmetic.
 * x itself is always given unquantised in `dtype`.
 * `perm` may be NULL when k == 1 and the rows of x are already grouped by expert (sorted row i is row i of x): with
 * E == 1 this is the plain feed-forward network of one expert (FFNMOE,
 * sharktank/sharktank/layers/ffn_moe_block.py:77-127; FFN, sharktank/sharktank/layers/ffn_block.py:21-51), and `offsets`
 * may then be NULL (the expert owns all T rows): no device array has to be built for the call.
 * `variant` 0 picks the kernel by shape (8: the same, restricted to the reference's arithmetic); other values force one
 * (see the kernel list in ffn.hip). */
int stmoe_grouped_ffn(const void* x, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                      const stmoe_weight* w_gate, const stmoe_weight* w_up, const stmoe_weight* w_down,
                      int act, const int32_t* offsets, const int32_t* perm, const float* x_scale /*nullable*/,
                      const float* z_scale /*nullable*/, void* y_sorted, void* workspace, size_t workspace_bytes,
                      int variant, stmoe_stream_t stream);

/* The two halves of stmoe_grouped_ffn as calls of their own, for callers that need the gated intermediate between them:
 * a dynamic or per-axis quantizer of the input of `ffn_down_exps` (DynamicScaledQuantizer,
 * sharktank/sharktank/types/quantizers.py:338-389; LinearLayer applies a q_input in front of its matmul,
 * sharktank/sharktank/layers/linear.py:72-78) needs the whole intermediate before it can scale any of it.
 *   stmoe_grouped_gate_up: z[i,:] = act(Wg[e] . x[t]) * (Wu[e] . x[t]) for every sorted position i; z [T*k, N] in `dtype`,
 *                          rows in dispatch order.  x_scale as in stmoe_grouped_ffn.
 *   stmoe_grouped_down:    y[i,:] = Wd[e] . z[i,:]; z is read as it is (the caller has quantised and dequantised it if it
 *                          wants that; a scale it computed stays in device memory, nothing comes back to the host).
 * Workspace: stmoe_grouped_ffn_workspace_bytes(T, k, K, N, dtype) for either.  Variants 5 and 7 are not available here. */
int stmoe_grouped_gate_up(const void* x, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                          const stmoe_weight* w_gate, const stmoe_weight* w_up, int act, const int32_t* offsets,
                          const int32_t* perm, const float* x_scale /*nullable*/, void* z_sorted, void* workspace,
                          size_t workspace_bytes, int variant, stmoe_stream_t stream);
int stmoe_grouped_down(const void* z_sorted, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                       const stmoe_weight* w_down, const int32_t* offsets, void* y_sorted, void* workspace,
                       size_t workspace_bytes, int variant, stmoe_stream_t stream);

/* One gathered-expert projection over all (token, slot) pairs, without the [T,k,rows,cols] weight gather of
 * `weights[experts]` + einsum_2args (ffn_moe_block.py:37-41; sharktank/sharktank/ops/default_impls.py:72-94):
 *   out[p, :] = W[idx[p]] . a[src(p), :],  p = t*k + j,  src(p) = t  (a [T, cols],   "mk,menk->men")   if !a_per_pair
 *                                                           src(p) = p  (a [T*k, cols], "mek,menk->men")  if a_per_pair
 * out [T*k, rows] in pair order (i.e. [T, k, rows]); offsets/perm from stmoe_dispatch_build on idx. */
int stmoe_grouped_mmt(const void* a, int dtype, int64_t T, int k, int a_per_pair, const stmoe_weight* w,
                      const int32_t* offsets, const int32_t* perm, void* out, int variant, stmoe_stream_t stream);

/* out[r, :] = g[r] * y[r, :] rounded to `dtype`: einsum "me,men->men" (default_impls.py:97-105) on flattened pairs. */
int stmoe_scale_rows(const void* y, const void* g, int dtype, int64_t rows, int64_t K, void* out, stmoe_stream_t stream);

/* out[r, c] = y[r, c] + bias[c]: the bias of `linear` (sharktank/sharktank/ops/default_impls.py:328-341, `result + bias`).
 * y [rows, cols]; dtypes F32/F16/BF16; out_dtype must be torch's promotion of the two (equal dtypes stay, mixed ones
 * give F32); operands are widened to fp32, added, rounded once.  out may alias y when the dtypes are equal. */
int stmoe_add_bias(const void* y, int y_dtype, const void* bias, int bias_dtype, int64_t rows, int64_t cols, void* out,
                   int out_dtype, stmoe_stream_t stream);

/* softmax over the last axis of x [rows, cols] (`ops.softmax`, sharktank/sharktank/ops/signatures.py:974-993, default
 * implementation F.softmax, default_impls.py:426-432; MoeBlock applies it to the router logits with dtype=float,
 * mixture_of_experts_block.py:72-74): values widened to fp32, p = exp(x - max) / sum (results below the smallest normal
 * fp32 number are kept, not flushed to zero), rounded to out_dtype.  Rows of at
 * most 64 elements are summed in index order, as the router kernel sums them: ranking these probabilities reproduces
 * stmoe_router_topk's choice bit for bit. */
int stmoe_softmax(const void* x, int x_dtype, int64_t rows, int64_t cols, void* out, int out_dtype, stmoe_stream_t stream);

/* Weighted combine (ffn_moe_block.py:73-74) and the layer tail (mixture_of_experts_block.py:86-90):
 *   o[t,:] = sum_j round(gate[t,j] * y[inv[t*k+j],:])   (slot order, fp32 sum, rounded to `dtype`)
 *   o = rms_norm(o; out_norm_w, eps) if out_norm_w != NULL     (layer_output_norm)
 *   out[t,:] = residual[t,:] + o[t,:] if residual != NULL      (h + moe_output)   */
int stmoe_combine(const void* y_sorted, const void* gate, const int32_t* inv, int dtype, int64_t T, int k,
                  int64_t K, const void* out_norm_w /*nullable*/, int w_dtype, float eps,
                  const void* residual /*nullable*/, void* out, stmoe_stream_t stream);

/* Whole MoeBlock.forward (mixture_of_experts_block.py:64-90) on h [T,K] -> out [T,K]:
 * ffn_norm -> router -> dispatch -> grouped FFN -> combine (+ layer_output_norm) + residual.
 * ffn_norm_w / out_norm_w are of w_dtype; out_norm_w may be NULL.  idx_out/gate_out ([T,k]) may be NULL.
 * x_scale / z_scale: activation quantizers of the expert FFN as in stmoe_grouped_ffn (NULL: none).
 * The stages are not always launches of their own: ffn_norm rides in the router launch when a token row fits its LDS
 * row; the dispatch of a single token is written by the router launch and that of at most 64 (token, slot) pairs is
 * built inside a streamed gate/up launch (the same stable counting sort as stmoe_dispatch_build, bit for bit). */
int stmoe_moe_forward(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                      const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                      const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                      const stmoe_weight* w_down, int act, const float* x_scale /*nullable*/,
                      const float* z_scale /*nullable*/, void* out, int32_t* idx_out, void* gate_out,
                      void* workspace, size_t workspace_bytes, int variant, stmoe_stream_t stream);

/* stmoe_moe_forward with per-stage timing for benchmarks: `events` is a host array of 12 hipEvent_t created by
 * the caller (entries may be NULL); stage s is bracketed on `stream` by events[2s] and events[2s+1], with
 * s = 0 ffn_norm, 1 router, 2 dispatch, 3 gate/up projection, 4 down projection, 5 combine.  No counterpart in
 * the reference; it exists so a benchmark can time each kernel inside its timed region. */
#define STMOE_FORWARD_STAGES 6
int stmoe_moe_forward_timed(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                            const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                            const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                            const stmoe_weight* w_down, int act, const float* x_scale /*nullable*/,
                            const float* z_scale /*nullable*/, void* out, int32_t* idx_out, void* gate_out,
                            void* workspace, size_t workspace_bytes, int variant, stmoe_stream_t stream,
                            void** events);

/* stmoe_moe_forward without a workspace argument, for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The workspace is a
 * fixed array of STMOE_STATIC_SCRATCH_BYTES in device memory that belongs to the library (one copy on every GPU the
 * library runs on, held until the process ends); the call itself allocates nothing.  Shapes whose
 * stmoe_moe_forward_workspace_bytes() exceeds that size (prefill-sized batches) are refused with STMOE_ERR_WORKSPACE.
 * All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race; serialise them.
 * The first call on a device looks the array's address up (hipGetSymbolAddress): make it outside graph capture. */
#define STMOE_STATIC_SCRATCH_BYTES (16u << 20)
int stmoe_moe_forward_static(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                             const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                             const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                             const stmoe_weight* w_down, int act, const float* x_scale /*nullable*/,
                             const float* z_scale /*nullable*/, void* out, int32_t* idx_out, void* gate_out,
                             int variant, stmoe_stream_t stream);

/* Measurement aid, no counterpart in the reference: one launch of nothing but independent matrix-core instructions on
 * operands held in registers (kind 0: v_mfma_f32_16x16x32_f16, kind 1: v_mfma_scale_f32_32x32x64_f8f6f4 on e4m3 bytes;
 * random_operands 0: constant bits, 1: hashed bits), 2 wavefronts per SIMD on 256 CUs, `iters` (a multiple of 4) loop
 * passes.  *flop (host, nullable) receives the floating-point operations of the launch; the caller times it.  The chip
 * lowers its clock with the matrix cores' activity and with the switching of the operand bits, so this rate, not the
 * data-sheet one, is what a matrix-core-bound kernel can approach on this machine.  `sink`: 4 writable device bytes. */
int stmoe_probe_mfma(int kind, int random_operands, int iters, float* sink, double* flop /*host, nullable*/,
                     stmoe_stream_t stream);

/* x @ W^T for one quantised (or dense) matrix W [rows, cols]: the operand set of the reference's
 * `mmt_block_scaled_q8(a,d,qs)` (sharktank/sharktank/kernels/mmt_block_scaled_q8.py:30) and
 * `mmt_block_scaled_offset_q4_unsigned(a,d,qs,m)` (mmt_block_scaled_offset_q4.py:31), reached from
 * ops.matmul(Tensor, QuantizedTensor, transpose_rhs=True) (sharktank/sharktank/ops/custom_impls.py:66-103).
 * a [M,K], out [M,rows], both `dtype`; fp32 accumulation.
 * `workspace` (nullable; stmoe_mmt_workspace_bytes(M) bytes, 16-byte aligned): scratch for reductions split over several
 * workgroups, which lets a launch of a few hundred rows (too few 256 x 256 units for 256 CUs) use the whole chip; without
 * it the result is the same up to the grouping of the fp32 sums, the launch only slower.  (Launches of 129 rows and more
 * whose tiles of 64 output features x 256 rows fit the 256 CUs run on such tiles instead and use no workspace.)  The workspace ends in a few
 * counters that elect the workgroup which adds a split unit's chunks; every call leaves them at zero.
 * `workspace_ready` != 0: the caller vouches that the workspace was zero-filled before its first use and has since been
 * written only by calls of this function (on one stream at a time); 0: the counters are cleared first, one small launch
 * more (5 us). */
size_t stmoe_mmt_workspace_bytes(int64_t M);
int stmoe_mmt(const void* a, int dtype, int64_t M, const stmoe_weight* w, void* out, void* workspace /*nullable*/,
              size_t workspace_bytes, int workspace_ready, int variant, stmoe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SHARKTANK_MOE_HIP_H_ */
