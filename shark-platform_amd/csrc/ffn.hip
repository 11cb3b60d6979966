// C-ABI entry points of the grouped expert FFN, the fused layer forward and the single-matrix mmt.
#include <atomic>
#include "ffn_kernels.h"

namespace stmoe {

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

static int check_weight(const stmoe_weight* w, const char* who, int64_t E, int64_t rows, int64_t cols) {
  STMOE_REQUIRE(w, STMOE_ERR_NULL, "%s: weight descriptor is NULL", who);
  STMOE_REQUIRE(w->qs, STMOE_ERR_NULL, "%s: qs plane is NULL", who);
  STMOE_REQUIRE(w->experts == E && w->rows == rows && w->cols == cols, STMOE_ERR_SHAPE,
                "%s: weight is [%lld,%lld,%lld], expected [%lld,%lld,%lld]", who, (long long)w->experts,
                (long long)w->rows, (long long)w->cols, (long long)E, (long long)rows, (long long)cols);
  STMOE_REQUIRE(aligned16(w->qs), STMOE_ERR_ALIGN, "%s: qs plane must be 16-byte aligned", who);
  if (w->format >= STMOE_W_Q8_0_PACKED && w->format <= STMOE_W_FP8_PACKED)
    STMOE_REQUIRE(rows % 16 == 0 && cols % 256 == 0, STMOE_ERR_SHAPE, "%s: packed formats need rows %% 16 == 0 and cols %% 256 == 0", who);
  switch (w->format) {
    case STMOE_W_Q8_0:
    case STMOE_W_Q8_0_PACKED:
      STMOE_REQUIRE(w->d, STMOE_ERR_NULL, "%s: Q8_0 needs d", who);
      STMOE_REQUIRE(w->m == nullptr, STMOE_ERR_UNSUPPORTED, "%s: Q8 block scaled with offset is not implemented", who);
      STMOE_REQUIRE(cols % 32 == 0, STMOE_ERR_SHAPE, "%s: Q8_0 needs cols %% 32 == 0", who);
      break;
    case STMOE_W_Q4_1:
    case STMOE_W_Q4_1_PACKED:
      STMOE_REQUIRE(w->d && w->m, STMOE_ERR_NULL, "%s: Q4_1 needs d and m", who);
      STMOE_REQUIRE(cols % 32 == 0, STMOE_ERR_SHAPE, "%s: Q4_1 needs cols %% 32 == 0", who);
      break;
    case STMOE_W_FP8:
    case STMOE_W_FP8_PACKED:
      STMOE_REQUIRE(w->d, STMOE_ERR_NULL, "%s: FP8 needs d", who);
      STMOE_REQUIRE(w->d_count == 1 || w->d_count == E, STMOE_ERR_SHAPE, "%s: FP8 d_count must be 1 or experts", who);
      STMOE_REQUIRE(cols % 16 == 0, STMOE_ERR_SHAPE, "%s: FP8 needs cols %% 16 == 0", who);
      break;
    case STMOE_W_DENSE:
      STMOE_REQUIRE(cols % 16 == 0, STMOE_ERR_SHAPE, "%s: dense weights need cols %% 16 == 0", who);
      break;
    default:
      return set_error(STMOE_ERR_UNSUPPORTED, "%s: unknown weight format %d", who, w->format);
  }
  STMOE_REQUIRE(weight_tag(w) >= 0, STMOE_ERR_DTYPE, "%s: dtype %d not valid for format %d", who, w->dtype, w->format);
  return STMOE_OK;
}

// variant: 0 auto, 1 generic (vector ALU), 2 MFMA 128x128 tile, 3 skinny streaming kernel (decode),
//          4 MFMA 256x256 tile (prefill; packed Q8_0), 5 fp8 matrix cores (fp8 weights and quantised activations),
//          6 MFMA 256x256 tile with specialised producer/consumer wavefronts (prefill; packed formats),
//          7 fp8 matrix cores, 128x128 tile kernel only (5 uses the 256x256 LDS-direct kernel where it applies),
//          8 auto among the kernels that follow the reference's arithmetic step by step (never the fp8 matrix cores)
//          9 MFMA 64 x 256 tile, the narrow form of 4 (a single matrix with a few hundred rows; packed formats)
// Automatic choice with fp8 weights and static quantizers on both activations: a prefill-sized launch with fp16
// activations goes to the fp8 matrix cores (variant 5: both operands as bytes, the fp32 dot product scaled once; 1.8 times
// faster than dequantise-then-multiply, and 6e-3 from it on the layer output at the Mixtral shape, inside the 2e-2 the fp8
// configuration is held to).  bf16 activations stay on the step-by-step path: there the two arithmetics are up to 4e-2
// apart (the reference rounds the dequantised operands to 8 significant bits first).  Smaller launches stream the
// weights and are bound by memory either way.
static int effective_variant(int variant, int dtype, int64_t rows, int64_t K, int64_t N, const stmoe_weight* w_gate,
                             const stmoe_weight* w_up, const stmoe_weight* w_down, const float* x_scale, const float* z_scale) {
  if (variant == 8) return 0;
  if (variant != 0) return variant;
  const bool fp8_all = w_gate && w_up && w_down && w_gate->format == STMOE_W_FP8_PACKED && w_up->format == STMOE_W_FP8_PACKED &&
                       w_down->format == STMOE_W_FP8_PACKED && w_gate->dtype == STMOE_F32 && w_up->dtype == STMOE_F32 &&
                       w_down->dtype == STMOE_F32;
  if (fp8_all && x_scale && z_scale && dtype == STMOE_F16 && rows >= 320 && K % 256 == 0 && N % 256 == 0) return 5;
  return 0;
}
// Automatic choice of a grouped launch (the host knows the row total and the token count, not the rows per expert):
// the streaming kernel when no expert can get more than 32 rows (token count <= 32), when the launch has at most 128 rows
// in all (such launches get no scratch for split reductions, without which the prefill kernel leaves most CUs idle), or
// when experts get 16 rows or fewer on average (28 with at most 4 experts); everything else goes to the
// specialised-wavefront prefill kernel.  Measured on the Mixtral layer (top-2, Q8_0 fp16, whole layer, us; streaming /
// prefill kernel with split scratch): 8 experts at 64 / 80 / 96 / 128 / 160 tokens 297 / 340 / 360 / 436 / 559 against
// 307 / 310 / 315 / 321 / 331 (Q4_1 bf16: 285 / 330 / 358 / 434 / 565 against 332 / 334 / 335 / 339 / 346); 4 experts at
// 48 / 56 / 64 / 80 tokens 168 / 172 / 235 / 295 against 183 / 184 / 186 / 190; 2 experts at 40 / 64 tokens 171 / 185
// against 127 / 131 (with scratch, which launches of that size do not get).  Since token tiles of at most 128 rows run
// with eight loader wavefronts the prefill kernel is nearly flat from 48 to 256 tokens.
// The streaming kernel walks an expert's rows in passes of 32 and re-reads the expert's weights for every pass, so inside
// its window a routing that puts all T tokens on a few experts costs those experts ceil(T / 32) passes instead of one.
static constexpr int64_t kSkinnyMaxRowsPerExpert = 32;
static constexpr int64_t kSkinnyMaxRows = 128;  // == the largest T * k without split scratch (carve_ffn)
static inline int64_t skinny_max_avg_rows(int E) { return E <= 4 ? 28 : 16; }
// A single matrix (no grouping): the streaming kernel re-reads the weights once per 32 rows and wins up to 48 rows
// (24 / 38 / 45 / 58 us at 32 / 48 / 64 / 80 rows of a [14336, 4096] Q8_0 matrix, against 37 / 38 / 40 / 48 us for the
// 256 x 256 kernel, which takes 50 us at 96-128 rows and 74-82 us from 129 to 512).  With scratch for split reductions
// the 256 x 256 kernel cuts its 56 units into 224 chunks and takes 30 / 39 / 58 / 77 us at 64 / 128 / 256 / 512 rows
// (Q4_1: 33 / 43 / 60 / 79): it then wins from 33 rows on.
static constexpr int64_t kSkinnyMaxRowsSingle = 48;
static constexpr int64_t kSkinnyMaxRowsSingleSplit = 32;
// A single matrix with 129 rows or more and few output features: tiles of 64 output features x 256 rows (the narrow form of
// the 256 x 256 kernel, variant 9) fill the CUs where 256 x 256 units cannot, without cutting the reduction.  It pays while
// its tiles fit one round over the 256 CUs and, against the split reduction, while the reduction is short: a narrow tile
// takes 0.6 us per K step of 64, a quarter of a split unit's reduction 0.25 us per step of the whole plus 40-45 us for the
// fp32 partial tiles and their sum.  Measured ([out, in] Q8_0 fp16, narrow / split, us): [14336, 4096] 192 rows 42 / 58,
// 256 rows 45 / 64 (0.67 PFLOP/s), 384 rows 81 / 73; [4096, 4096] 192 ... 1024 rows 33 ... 47 / 42 ... 67; [8192, 8192] 256
// rows 75 / 69; [4096, 14336] 256 rows 123 / 86.  Without scratch the 256 x 256 kernel takes 1.15 us per step unsplit.
static bool narrow_pays(int mode, const GemmParams& p, int64_t rows) {
  if (rows <= 128) return false;
  const int64_t features = mode == MODE_GATEUP ? 32 : 64;
  if (p.n_out % features != 0) return false;
  if (p.n_out / features * ((rows + 255) / 256) > 256) return false;
  return p.split_scratch == nullptr || p.kred <= 6144;
}
// fp8 activations x fp8 weights on the fp8 matrix cores: the 256 x 256 kernel for packed weights and launches with
// enough rows to fill its tiles (variant 5), the 128 x 128 kernel otherwise (and always with variant 7).
// Whether the 256 x 256 kernel takes a projection (its token rows must come without a gather: see fp8_ws_takes' caller).
static bool fp8_ws_takes(int variant, int wtag, int mode, int64_t kred, int64_t lda, int64_t ldo, int64_t n_out, bool offsets, int E,
                         int64_t max_rows) {
  return variant == 5 && wtag == WF_FP8_F32D_P && max_rows >= 320 && kred % 256 == 0 && lda % 16 == 0 && ldo % 4 == 0 &&
         n_out % (mode == MODE_GATEUP ? 128 : 256) == 0 && (!offsets || E < 64) && max_rows * lda < ((int64_t)1 << 32);
}
static int run_fp8_projection(int variant, int dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (!p.perm && fp8_ws_takes(variant, wtag, mode, p.kred, p.lda, p.ldo, p.n_out, p.offsets != nullptr, p.E, max_rows))
    return launch_fp8_ws(dtype, wtag, mode, p, max_rows, st);
  return launch_fp8_tile(dtype, wtag, mode, p, max_rows, st);
}

static int run_projection(int variant, int dtype, int wtag, int mode, const GemmParams& p, int64_t max_rows, hipStream_t st) {
  if (p.choices) {
    // (only the streaming kernel builds its own dispatch; the caller has checked that it takes the launch)
    const int rc = launch_skinny(dtype, wtag, mode, p, max_rows, st);
    return rc != STMOE_ERR_UNSUPPORTED ? rc : set_error(STMOE_ERR_UNSUPPORTED, "grouped_ffn: no streaming kernel for a launch that builds its own dispatch");
  }
  if (variant == 0) {
    if (dtype == STMOE_F32) variant = 1;
    // (one matrix, with or without an offsets array around its rows)
    else if (p.E == 1) variant = max_rows <= (p.split_scratch ? kSkinnyMaxRowsSingleSplit : kSkinnyMaxRowsSingle) ? 3
                                 : narrow_pays(mode, p, max_rows) ? 9 : 6;
    else if (p.offsets && ((p.expert_rows_bound > 0 && p.expert_rows_bound <= kSkinnyMaxRowsPerExpert) ||
                           max_rows <= kSkinnyMaxRows || max_rows <= skinny_max_avg_rows(p.E) * p.E)) variant = 3;
    // Everything else goes to the 256 x 256 kernel (which hands shapes it does not take down to the 128 x 128 one).
    else variant = 6;
  }
  if (variant == 9) {
    int rc = launch_mfma_narrow(dtype, wtag, mode, p, max_rows, st);
    if (rc != STMOE_ERR_UNSUPPORTED) return rc;
    variant = 6;
  }
  if (variant == 6) {
    int rc = launch_mfma_ws(dtype, wtag, mode, p, max_rows, p.split_scratch, st);
    if (rc != STMOE_ERR_UNSUPPORTED) return rc;
    variant = 4;
  }
  if (variant == 4) {
    int rc = launch_mfma_big(dtype, wtag, mode, p, max_rows, st);
    if (rc != STMOE_ERR_UNSUPPORTED) return rc;
    variant = 2;
  }
  if (variant == 3) {
    int rc = launch_skinny(dtype, wtag, mode, p, max_rows, st);
    if (rc != STMOE_ERR_UNSUPPORTED) return rc;
    variant = 2;
  }
  if (variant == 2) {
    int rc = launch_mfma_tile(dtype, wtag, mode, p, max_rows, st);
    if (rc != STMOE_ERR_UNSUPPORTED) return rc;
    variant = 1;  // combination without a matrix-core instantiation: the vector-ALU kernel covers it
  }
  if (variant == 1) return launch_generic(dtype, wtag, mode, p, max_rows, st);
  return set_error(STMOE_ERR_UNSUPPORTED, "grouped_ffn: unknown kernel variant %d", variant);
}

}  // namespace stmoe

using namespace stmoe;

// Workspace of the grouped FFN: the intermediate z [T*k, N] in `dtype`, then (used only with quantised activations)
// the quantised or re-dequantised copy of x [T, K] and the quantised intermediate [T*k, N] bytes.
struct FfnWs {
  size_t z, xa, zq, split, total;
};
static FfnWs carve_ffn(int64_t T, int k, int64_t K, int64_t N, int dtype) {
  FfnWs w{};
  const size_t es = dtype_size(dtype);
  w.z = 0;
  w.xa = align_up((size_t)T * k * N * es, 256);
  // (the fp8 matrix-core path keeps one quantised row per (token, slot) pair there, grouped by expert)
  w.zq = w.xa + align_up(std::max((size_t)T * K * es, (size_t)T * k * K), 256);
  w.split = w.zq + align_up((size_t)T * k * N, 256);
  // fp32 partial tiles of split reductions (prefill kernels only)
  w.total = w.split + (T * k > 128 ? align_up(mfma_ws_partial_bytes(), 256) : 0);  // kSkinnyMaxRows: smaller launches stream
  return w;
}

extern "C" size_t stmoe_grouped_ffn_workspace_bytes(int64_t T, int k, int64_t K, int64_t N, int dtype) {
  if (T <= 0 || k <= 0 || N <= 0 || K <= 0) return 0;
  return carve_ffn(T, k, K, N, dtype).total;
}

static inline void mark(void** events, int i, hipStream_t st) {
  if (events && events[i]) (void)hipEventRecord(reinterpret_cast<hipEvent_t>(events[i]), st);
}

// stages: 1 = gate/up projection only (the gated intermediate goes to `z_io`), 2 = down projection only (reads `z_io`),
// 3 = both (the intermediate lives in the workspace).  offsets == NULL: one expert that owns all T * k rows.
static int grouped_ffn_impl(const void* x, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                            const stmoe_weight* w_gate, const stmoe_weight* w_up, const stmoe_weight* w_down,
                            int act, const int32_t* offsets, const int32_t* perm, const float* x_scale,
                            const float* z_scale, void* y_sorted, void* workspace, size_t workspace_bytes, int variant,
                            stmoe_stream_t stream, void** events, bool tickets_zeroed = false, int stages = 3,
                            void* z_io = nullptr, bool x_is_fake_quantized = false, const int32_t* choices = nullptr,
                            int32_t* dispatch_counts = nullptr, int32_t* dispatch_inv = nullptr) {
  STMOE_REQUIRE(T >= 0 && K > 0 && N > 0 && E >= 1 && k >= 1, STMOE_ERR_SHAPE, "grouped_ffn: T=%lld K=%lld N=%lld E=%d k=%d",
                (long long)T, (long long)K, (long long)N, E, k);
  STMOE_REQUIRE(dtype == STMOE_F32 || dtype == STMOE_F16 || dtype == STMOE_BF16, STMOE_ERR_DTYPE,
                "grouped_ffn: activation dtype %d is not f32/f16/bf16", dtype);
  STMOE_REQUIRE(act == STMOE_ACT_SILU || act == STMOE_ACT_GELU_ERF, STMOE_ERR_UNSUPPORTED, "grouped_ffn: activation %d", act);
  const bool do_in = (stages & 1) != 0, do_out = (stages & 2) != 0;
  if (variant == 8) variant = 0;  // (the entry points have resolved the automatic choice: effective_variant)
  int rc;
  if (do_in) {
    if ((rc = check_weight(w_gate, "grouped_ffn(ffn_gate_exps)", E, N, K))) return rc;
    if ((rc = check_weight(w_up, "grouped_ffn(ffn_up_exps)", E, N, K))) return rc;
    STMOE_REQUIRE(weight_tag(w_gate) == weight_tag(w_up), STMOE_ERR_UNSUPPORTED,
                  "grouped_ffn: gate and up weights must share one format");
  }
  if (do_out && (rc = check_weight(w_down, "grouped_ffn(ffn_down_exps)", E, K, N))) return rc;
  if (T == 0) return STMOE_OK;
  STMOE_REQUIRE(offsets || E == 1, STMOE_ERR_NULL, "grouped_ffn: offsets may only be NULL with a single expert");
  STMOE_REQUIRE((!do_in || (x && (perm || k == 1))) && (!do_out || y_sorted) && (stages == 3 || z_io), STMOE_ERR_NULL,
                "grouped_ffn: NULL pointer");
  STMOE_REQUIRE((!do_in || aligned16(x)) && (!do_out || aligned16(y_sorted)) && aligned16(workspace) && aligned16(z_io),
                STMOE_ERR_ALIGN, "grouped_ffn: x, y_sorted, the intermediate and the workspace must be 16-byte aligned");
  STMOE_REQUIRE((K * dtype_size(dtype)) % 16 == 0 && (N * dtype_size(dtype)) % 16 == 0, STMOE_ERR_SHAPE,
                "grouped_ffn: rows of x and of the intermediate must be multiples of 16 bytes");
  const size_t need = stmoe_grouped_ffn_workspace_bytes(T, k, K, N, dtype);
  STMOE_REQUIRE(workspace && workspace_bytes >= need, STMOE_ERR_WORKSPACE, "grouped_ffn: workspace %zu < %zu bytes",
                workspace_bytes, need);
  hipStream_t st = as_stream(stream);
  const int64_t rows = T * k;
  const FfnWs ws = carve_ffn(T, k, K, N, dtype);
  char* base = (char*)workspace;
  void* z = stages == 3 ? (void*)(base + ws.z) : z_io;
  void* xa = base + ws.xa;
  void* zq = base + ws.zq;

  // Quantised activations (fp8 e4m3fn, static per-tensor scale).  By default the samples are re-dequantised (the
  // reference's own formulation: quantize, dequantize, multiply in the activation dtype) and the 16-bit kernels run
  // unchanged: the streaming kernel is bound by the weight stream anyway, and the 16-bit prefill kernel with its
  // producer/consumer pipeline is currently faster than the fp8 matrix-core kernel.  Variant 5 sends both operands to
  // the fp8 matrix cores as bytes and scales the fp32 dot product once.
  const bool want_mfma8 = (variant == 5 || variant == 7) && stages == 3;
  STMOE_REQUIRE(!(variant == 5 || variant == 7) || stages == 3, STMOE_ERR_UNSUPPORTED,
                "grouped_ffn: variants 5 and 7 (fp8 matrix cores) run both projections in one call");
  const bool fp8_w_in = want_mfma8 && (w_gate->format == STMOE_W_FP8 || w_gate->format == STMOE_W_FP8_PACKED);
  const bool fp8_w_out = want_mfma8 && (w_down->format == STMOE_W_FP8 || w_down->format == STMOE_W_FP8_PACKED);
  STMOE_REQUIRE(!want_mfma8 || (x_scale && z_scale), STMOE_ERR_UNSUPPORTED, "grouped_ffn: variants 5 and 7 (fp8 matrix cores) need x_scale and z_scale");
  const bool t16 = dtype == STMOE_F16 || dtype == STMOE_BF16;
  const bool mfma8_in = t16 && x_scale && fp8_w_in && w_gate->dtype == STMOE_F32 && K % 16 == 0 && want_mfma8;
  const bool mfma8_out = t16 && z_scale && fp8_w_out && w_down->dtype == STMOE_F32 && N % 16 == 0 && want_mfma8;
  const int v16 = (variant == 5 || variant == 7) ? 0 : variant;
  // Scratch of the split reductions: part of the workspace for launches of more than 128 rows.  Smaller grouped launches
  // stream and need none; a single matrix of 33..128 rows runs the prefill kernel and is up to 1.5 times faster with it, so
  // a caller may append it (a workspace of the queried size plus stmoe_mmt_workspace_bytes(rows)).
  const size_t split_bytes = align_up(mfma_ws_partial_bytes(), 256);
  const bool appended = E == 1 && rows > kSkinnyMaxRowsSingleSplit && workspace_bytes >= ws.split + split_bytes;
  float* const split = ws.total > ws.split || appended ? reinterpret_cast<float*>(base + ws.split) : nullptr;
  const int32_t n_experts = offsets ? E : 1;
  const bool z_blocked = mfma8_in && mfma8_out &&
                         fp8_ws_takes(variant, weight_tag(w_gate), MODE_GATEUP, K, K, N, N, offsets != nullptr, n_experts, rows) &&
                         fp8_ws_takes(variant, weight_tag(w_down), MODE_DOWN, N, N, K, K, offsets != nullptr, n_experts, rows);

  if (do_in) {
    GemmParams p{};
    p.a = x; p.lda = K; p.perm = perm; p.k_top = k; p.offsets = offsets; p.E = n_experts; p.fixed_rows = offsets ? 0 : rows;
    p.w0 = make_view(w_gate); p.w1 = make_view(w_up);
    p.out = z; p.ldo = N; p.n_out = N; p.kred = K; p.act = act; p.x_scale = nullptr; p.expert_rows_bound = T;
    p.split_scratch = split;
    p.split_tickets_zeroed = tickets_zeroed;
    if (choices) {  // `offsets` and `perm` are filled by the gate/up launch itself (see GemmParams::choices)
      p.choices = choices; p.n_choices = (int32_t)rows; p.dispatch_counts = dispatch_counts; p.dispatch_inv = dispatch_inv;
    }
    mark(events, 0, st);
    if (x_scale && !(x_is_fake_quantized && !mfma8_in)) {  // (the fused forward's norm launch may have done it already)
      // The 256 x 256 fp8 kernel streams its token rows in sorted order: the quantising pass writes them grouped by expert
      // (one row per pair) and the projection needs no gather.  The 128 x 128 kernel gathers itself.
      const bool sorted_rows = mfma8_in && perm &&
                               fp8_ws_takes(variant, weight_tag(w_gate), MODE_GATEUP, K, K, N, N, offsets != nullptr, n_experts, rows);
      if (sorted_rows) rc = quantize_fp8_gather(x, dtype, x_scale, perm, k, rows, K, xa, rows, st);
      else if (mfma8_in) rc = stmoe_quantize_fp8(x, dtype, x_scale, T * K, xa, stream);
      else rc = stmoe_fake_quant_fp8(x, dtype, x_scale, T * K, xa, stream);
      if (rc) return rc;
      p.a = xa;
      if (sorted_rows) { p.perm = nullptr; p.k_top = 1; p.a_block_rows = rows; }
    }
    // the quantizer of the intermediate is applied by the gate/up kernels themselves (16-bit kernels; the fp8 matrix-core
    // kernels write real e4m3fn samples instead)
    if (z_scale && stages == 3 && !mfma8_out && !mfma8_in) p.out_fq = z_scale;
    if (mfma8_in) {
      p.x_scale = x_scale;
      if (mfma8_out) {
        p.out = zq;
        p.out_scale = z_scale;
        // the quantised intermediate goes from one 256 x 256 fp8 launch to the other in blocks of 64 reduction samples
        if (z_blocked) p.out_block_rows = rows;
      }
      rc = run_fp8_projection(variant, dtype, weight_tag(w_gate), MODE_GATEUP, p, rows, st);
    } else {
      rc = run_projection(v16, dtype, weight_tag(w_gate), MODE_GATEUP, p, rows, st);
    }
    if (rc) return rc;
    mark(events, 1, st);
  }
  if (!do_out) return STMOE_OK;

  GemmParams q{};
  q.a = z; q.lda = N; q.perm = nullptr; q.k_top = 1; q.offsets = offsets; q.E = n_experts; q.fixed_rows = offsets ? 0 : rows;
  q.w0 = make_view(w_down); q.w1 = q.w0;
  q.out = y_sorted; q.ldo = K; q.n_out = K; q.kred = N; q.act = act; q.x_scale = nullptr; q.expert_rows_bound = T;
  q.split_scratch = split;
  q.split_tickets_zeroed = tickets_zeroed;  // (a launch that uses the tickets leaves them at zero)
  mark(events, 2, st);
  if (z_scale) {
    STMOE_REQUIRE(stages == 3, STMOE_ERR_UNSUPPORTED, "grouped_ffn: the down projection on its own takes the intermediate as it is");
    if (mfma8_out && !mfma8_in) rc = stmoe_quantize_fp8(z, dtype, z_scale, rows * N, zq, stream);
    else if (!mfma8_out && mfma8_in) rc = stmoe_fake_quant_fp8(z, dtype, z_scale, rows * N, z, stream);  // in place
    else rc = STMOE_OK;  // (done by the gate/up launch, or the fp8 kernel has written e4m3fn samples)
    if (rc) return rc;
  }
  if (mfma8_out) {
    q.a = zq;
    q.x_scale = z_scale;
    if (z_blocked) q.a_block_rows = rows;
    rc = run_fp8_projection(variant, dtype, weight_tag(w_down), MODE_DOWN, q, rows, st);
  } else {
    rc = run_projection(v16, dtype, weight_tag(w_down), MODE_DOWN, q, rows, st);
  }
  mark(events, 3, st);
  return rc;
}

extern "C" int stmoe_grouped_ffn(const void* x, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                                 const stmoe_weight* w_gate, const stmoe_weight* w_up, const stmoe_weight* w_down,
                                 int act, const int32_t* offsets, const int32_t* perm, const float* x_scale,
                                 const float* z_scale, void* y_sorted, void* workspace, size_t workspace_bytes,
                                 int variant, stmoe_stream_t stream) {
  variant = effective_variant(variant, dtype, T * k, K, N, w_gate, w_up, w_down, x_scale, z_scale);
  return grouped_ffn_impl(x, dtype, T, K, N, E, k, w_gate, w_up, w_down, act, offsets, perm, x_scale, z_scale, y_sorted,
                          workspace, workspace_bytes, variant, stream, nullptr);
}

extern "C" int stmoe_grouped_gate_up(const void* x, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                                     const stmoe_weight* w_gate, const stmoe_weight* w_up, int act, const int32_t* offsets,
                                     const int32_t* perm, const float* x_scale, void* z_sorted, void* workspace,
                                     size_t workspace_bytes, int variant, stmoe_stream_t stream) {
  return grouped_ffn_impl(x, dtype, T, K, N, E, k, w_gate, w_up, nullptr, act, offsets, perm, x_scale, nullptr, nullptr, workspace,
                          workspace_bytes, variant, stream, nullptr, false, 1, z_sorted);
}

extern "C" int stmoe_grouped_down(const void* z_sorted, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                                  const stmoe_weight* w_down, const int32_t* offsets, void* y_sorted, void* workspace,
                                  size_t workspace_bytes, int variant, stmoe_stream_t stream) {
  return grouped_ffn_impl(nullptr, dtype, T, K, N, E, k, nullptr, nullptr, w_down, STMOE_ACT_SILU, offsets, nullptr, nullptr, nullptr,
                          y_sorted, workspace, workspace_bytes, variant, stream, nullptr, false, 2, const_cast<void*>(z_sorted));
}

extern "C" size_t stmoe_mmt_workspace_bytes(int64_t M) {
  // fp32 partial tiles of split reductions: only launches between the streaming kernel's window and a chip-filling number
  // of units can use them (see stmoe_mmt)
  return M > kSkinnyMaxRowsSingleSplit ? align_up(mfma_ws_partial_bytes(), 256) : 0;
}

extern "C" int stmoe_mmt(const void* a, int dtype, int64_t M, const stmoe_weight* w, void* out, void* workspace,
                         size_t workspace_bytes, int workspace_ready, int variant, stmoe_stream_t stream) {
  STMOE_REQUIRE(w, STMOE_ERR_NULL, "mmt: weight descriptor is NULL");
  STMOE_REQUIRE(M >= 0, STMOE_ERR_SHAPE, "mmt: M=%lld", (long long)M);
  STMOE_REQUIRE(dtype == STMOE_F32 || dtype == STMOE_F16 || dtype == STMOE_BF16, STMOE_ERR_DTYPE,
                "mmt: activation dtype %d is not f32/f16/bf16", dtype);
  int rc;
  if ((rc = check_weight(w, "mmt", 1, w->rows, w->cols))) return rc;
  if (M == 0) return STMOE_OK;
  STMOE_REQUIRE(a && out, STMOE_ERR_NULL, "mmt: NULL pointer");
  STMOE_REQUIRE(aligned16(a) && aligned16(out), STMOE_ERR_ALIGN, "mmt: a and out must be 16-byte aligned");
  STMOE_REQUIRE((w->cols * dtype_size(dtype)) % 16 == 0 && (w->rows * dtype_size(dtype)) % 8 == 0, STMOE_ERR_SHAPE,
                "mmt: row sizes must keep 16-byte (input) and 8-byte (output) alignment");
  GemmParams p{};
  p.a = a; p.lda = w->cols; p.perm = nullptr; p.k_top = 1; p.offsets = nullptr; p.E = 1; p.fixed_rows = M;
  p.w0 = make_view(w); p.w1 = p.w0;
  p.out = out; p.ldo = w->rows; p.n_out = w->rows; p.kred = w->cols; p.act = 0; p.x_scale = nullptr;
  // With a workspace the prefill kernel cuts the units that do not fill a round over the CUs along the reduction (256 rows
  // of a [14336, 4096] matrix are 56 units for 256 CUs: four chunks each make 224 workgroups).
  if (workspace && workspace_bytes >= stmoe_mmt_workspace_bytes(M) && stmoe_mmt_workspace_bytes(M) > 0) {
    STMOE_REQUIRE(aligned16(workspace), STMOE_ERR_ALIGN, "mmt: workspace must be 16-byte aligned");
    p.split_scratch = reinterpret_cast<float*>(workspace);
    p.split_tickets_zeroed = workspace_ready != 0;
  }
  return run_projection(variant, dtype, weight_tag(w), MODE_DOWN, p, M, as_stream(stream));
}

extern "C" int stmoe_grouped_mmt(const void* a, int dtype, int64_t T, int k, int a_per_pair, const stmoe_weight* w,
                                 const int32_t* offsets, const int32_t* perm, void* out, int variant,
                                 stmoe_stream_t stream) {
  STMOE_REQUIRE(w, STMOE_ERR_NULL, "grouped_mmt: weight descriptor is NULL");
  STMOE_REQUIRE(T >= 0 && k >= 1, STMOE_ERR_SHAPE, "grouped_mmt: T=%lld k=%d", (long long)T, k);
  STMOE_REQUIRE(dtype == STMOE_F32 || dtype == STMOE_F16 || dtype == STMOE_BF16, STMOE_ERR_DTYPE,
                "grouped_mmt: activation dtype %d is not f32/f16/bf16", dtype);
  int rc;
  if ((rc = check_weight(w, "grouped_mmt", w->experts, w->rows, w->cols))) return rc;
  if (T == 0) return STMOE_OK;
  STMOE_REQUIRE(a && offsets && perm && out, STMOE_ERR_NULL, "grouped_mmt: NULL pointer");
  STMOE_REQUIRE(aligned16(a) && aligned16(out), STMOE_ERR_ALIGN, "grouped_mmt: a and out must be 16-byte aligned");
  STMOE_REQUIRE((w->cols * dtype_size(dtype)) % 16 == 0 && (w->rows * dtype_size(dtype)) % 8 == 0, STMOE_ERR_SHAPE,
                "grouped_mmt: row sizes must keep 16-byte (input) and 8-byte (output) alignment");
  GemmParams p{};
  p.a = a; p.lda = w->cols; p.perm = perm; p.k_top = a_per_pair ? 1 : k; p.offsets = offsets; p.E = (int32_t)w->experts;
  p.w0 = make_view(w); p.w1 = p.w0;
  p.out = out; p.ldo = w->rows; p.out_perm = perm; p.n_out = w->rows; p.kred = w->cols; p.act = 0; p.x_scale = nullptr;
  p.expert_rows_bound = T;
  return run_projection(variant, dtype, weight_tag(w), MODE_DOWN, p, T * k, as_stream(stream));
}

// ---- whole layer ----------------------------------------------------------------------------------
// Workspace carve-up (each piece 256-byte aligned):
//   xn [T,K] T | logits-free | idx i32 [T,k] | gate T [T,k] | counts i32 [E] | offsets i32 [E+1] |
//   perm i32 [T*k] | inv i32 [T*k] | y [T*k, K] T | ffn workspace
struct LayerWs {
  size_t xn, idx, gate, counts, offsets, perm, inv, y, ffn, total;
};
static LayerWs carve(int64_t T, int k, int E, int64_t K, int64_t N, int dtype) {
  LayerWs w{};
  const size_t es = dtype_size(dtype);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes ? bytes : 1, 256); return o; };
  w.xn = take((size_t)T * K * es);
  w.idx = take((size_t)T * k * 4);
  w.gate = take((size_t)T * k * es);
  w.counts = take((size_t)E * 4);
  w.offsets = take((size_t)(E + 1) * 4);
  w.perm = take((size_t)T * k * 4);
  w.inv = take((size_t)T * k * 4);
  w.y = take((size_t)T * k * K * es);
  w.ffn = take(stmoe_grouped_ffn_workspace_bytes(T, k, K, N, dtype));
  w.total = off;
  return w;
}

extern "C" size_t stmoe_moe_forward_workspace_bytes(int64_t T, int k, int E, int64_t K, int64_t N, int dtype) {
  if (T <= 0 || k <= 0 || E <= 0 || K <= 0 || N <= 0) return 0;
  return carve(T, k, E, K, N, dtype).total;
}

static int moe_forward_impl(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                            const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                            const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                            const stmoe_weight* w_down, int act, const float* x_scale, const float* z_scale, void* out,
                            int32_t* idx_out, void* gate_out, void* workspace, size_t workspace_bytes, int variant,
                            stmoe_stream_t stream, void** events) {
  STMOE_REQUIRE(T >= 0 && K > 0 && N > 0 && E >= 1 && k >= 1 && k <= E, STMOE_ERR_SHAPE,
                "moe_forward: T=%lld K=%lld N=%lld E=%d k=%d", (long long)T, (long long)K, (long long)N, E, k);
  if (T == 0) return STMOE_OK;
  STMOE_REQUIRE(h && ffn_norm_w && w_router && out, STMOE_ERR_NULL, "moe_forward: NULL pointer");
  const LayerWs ws = carve(T, k, E, K, N, dtype);
  STMOE_REQUIRE(workspace && workspace_bytes >= ws.total, STMOE_ERR_WORKSPACE, "moe_forward: workspace %zu < %zu bytes",
                workspace_bytes, ws.total);
  STMOE_REQUIRE(aligned16(workspace), STMOE_ERR_ALIGN, "moe_forward: workspace must be 16-byte aligned");
  char* base = (char*)workspace;
  void* xn = base + ws.xn;
  int32_t* idx = idx_out ? idx_out : (int32_t*)(base + ws.idx);
  void* gate = gate_out ? gate_out : (void*)(base + ws.gate);
  int32_t* counts = (int32_t*)(base + ws.counts);
  int32_t* offsets = (int32_t*)(base + ws.offsets);
  int32_t* perm = (int32_t*)(base + ws.perm);
  int32_t* inv = (int32_t*)(base + ws.inv);
  void* y = base + ws.y;
  int rc;
  hipStream_t st = as_stream(stream);
  // stages: 0 rms_norm, 1 router, 2 dispatch, 3 gate/up projection, 4 down projection, 5 combine;
  // stage s is bracketed by events[2s] and events[2s+1]
  // ffn_norm and the router run as one launch when the token row fits the router's LDS row (stage 0 then has
  // zero length in the event brackets); otherwise as two.
  const bool fused_front = T < 0x7fffffffLL && K * dtype_size(dtype) <= 48 * 1024 && K % 8 == 0 && E <= 64 && aligned16(w_router);
  mark(events, 0, st);
  if (!fused_front && (rc = stmoe_rms_norm(h, dtype, ffn_norm_w, w_dtype, T, K, eps, xn, stream))) return rc;
  mark(events, 1, st);
  mark(events, 2, st);
  // a single token's dispatch is written by the router launch itself
  const bool router_dispatches = fused_front && T == 1;
  variant = effective_variant(variant, dtype, T * k, K, N, w_gate, w_up, w_down, x_scale, z_scale);
  // a static quantizer of the experts' input rides in the norm launch (which writes the rows the experts read) unless the
  // fp8 matrix-core kernels want real e4m3fn samples
  const float* x_fq = (fused_front && x_scale && variant != 5 && variant != 7) ? x_scale : nullptr;
  if (fused_front) rc = norm_router(h, dtype, ffn_norm_w, w_dtype, eps, xn, w_router, T, K, E, k, idx, gate, st,
                                    router_dispatches ? counts : nullptr, offsets, perm, inv, x_fq);
  else rc = stmoe_router_topk(xn, w_router, dtype, T, K, E, k, nullptr, idx, nullptr, gate, stream);
  if (rc) return rc;
  mark(events, 3, st);
  mark(events, 4, st);
  // A forward of at most 64 (token, slot) pairs that streams its weights has no dispatch launch either: every wavefront of
  // the gate/up launch sorts the router's choices itself (a few ballots) and the first one leaves the arrays for the down
  // and combine launches.
  const bool gate_up_dispatches =
      fused_front && T > 1 && T * k <= 64 && E >= 2 && (variant == 0 || variant == 3) && (dtype == STMOE_F16 || dtype == STMOE_BF16) &&
      w_gate && w_up && weight_tag(w_gate) == weight_tag(w_up) && !(x_scale && !x_fq) &&
      skinny_takes_grouped(dtype, weight_tag(w_gate), E, K, N, K, N);
  // the dispatch launch also clears the ticket words of the projections' split reductions (if this shape has any)
  const FfnWs fws = carve_ffn(T, k, K, N, dtype);
  const bool has_tickets = fws.total > fws.split && !router_dispatches;
  int32_t* tickets = has_tickets ? reinterpret_cast<int32_t*>(base + ws.ffn + fws.split + mfma_ws_tickets_offset()) : nullptr;
  if (!router_dispatches && !gate_up_dispatches &&
      (rc = dispatch_build(idx, T * k, E, counts, offsets, perm, inv, tickets, has_tickets ? mfma_ws_ticket_count() : 0, st)))
    return rc;
  mark(events, 5, st);
  if ((rc = grouped_ffn_impl(xn, dtype, T, K, N, E, k, w_gate, w_up, w_down, act, offsets, perm, x_scale, z_scale, y,
                             base + ws.ffn, workspace_bytes - ws.ffn, variant, stream, events ? events + 6 : nullptr, has_tickets, 3,
                             nullptr, x_fq != nullptr, gate_up_dispatches ? idx : nullptr, counts, inv)))
    return rc;
  mark(events, 10, st);
  rc = stmoe_combine(y, gate, inv, dtype, T, k, K, out_norm_w, w_dtype, eps, h, out, stream);
  mark(events, 11, st);
  return rc;
}

extern "C" int stmoe_moe_forward(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                                 const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                                 const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                                 const stmoe_weight* w_down, int act, const float* x_scale, const float* z_scale,
                                 void* out, int32_t* idx_out, void* gate_out, void* workspace, size_t workspace_bytes,
                                 int variant, stmoe_stream_t stream) {
  return moe_forward_impl(h, dtype, T, K, N, E, k, ffn_norm_w, out_norm_w, w_dtype, eps, w_router, w_gate, w_up, w_down,
                          act, x_scale, z_scale, out, idx_out, gate_out, workspace, workspace_bytes, variant, stream, nullptr);
}

extern "C" int stmoe_moe_forward_timed(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                                       const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                                       const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                                       const stmoe_weight* w_down, int act, const float* x_scale, const float* z_scale,
                                       void* out, int32_t* idx_out, void* gate_out, void* workspace,
                                       size_t workspace_bytes, int variant, stmoe_stream_t stream, void** events) {
  return moe_forward_impl(h, dtype, T, K, N, E, k, ffn_norm_w, out_norm_w, w_dtype, eps, w_router, w_gate, w_up, w_down,
                          act, x_scale, z_scale, out, idx_out, gate_out, workspace, workspace_bytes, variant, stream, events);
}

// ---- whole layer, workspace inside the library ---------------------------------------------------------
// For callers that cannot allocate (code under HIP graph capture, tight serving loops): the same forward with its
// workspace in a fixed array in device memory that belongs to the library, so the call needs no allocation by anyone.
// Every GPU the library runs on holds its own copy of the array until the process ends.  `scratch` below is the
// host-side handle of that array, not a device address: the address on the current device comes from
// hipGetSymbolAddress, is looked up once per device and is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[STMOE_STATIC_SCRATCH_BYTES];

static constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static int static_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return set_error(STMOE_ERR_LAUNCH, "moe_forward_static: no current device");
  STMOE_REQUIRE(dev >= 0 && dev < kMaxDevices, STMOE_ERR_UNSUPPORTED, "moe_forward_static: device ordinal %d is beyond %d", dev, kMaxDevices - 1);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return set_error(STMOE_ERR_LAUNCH, "moe_forward_static: hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // two threads racing here store the same address
  }
  *out = ptr;
  return STMOE_OK;
}

extern "C" int stmoe_moe_forward_static(const void* h, int dtype, int64_t T, int64_t K, int64_t N, int E, int k,
                                        const void* ffn_norm_w, const void* out_norm_w, int w_dtype, float eps,
                                        const void* w_router, const stmoe_weight* w_gate, const stmoe_weight* w_up,
                                        const stmoe_weight* w_down, int act, const float* x_scale, const float* z_scale,
                                        void* out, int32_t* idx_out, void* gate_out, int variant, stmoe_stream_t stream) {
  STMOE_REQUIRE(T >= 0 && K > 0 && N > 0 && E >= 1 && k >= 1 && k <= E, STMOE_ERR_SHAPE,
                "moe_forward_static: T=%lld K=%lld N=%lld E=%d k=%d", (long long)T, (long long)K, (long long)N, E, k);
  if (T == 0) return STMOE_OK;
  const size_t need = carve(T, k, E, K, N, dtype).total;
  STMOE_REQUIRE(need <= (size_t)STMOE_STATIC_SCRATCH_BYTES, STMOE_ERR_WORKSPACE,
                "moe_forward_static: this shape needs a workspace of %zu bytes, the built-in one holds %zu (use stmoe_moe_forward "
                "with a caller-owned workspace)", need, (size_t)STMOE_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // Nothing in the workspace has to start at zero: every piece (normalised rows, routing, dispatch arrays, the two
  // intermediates) is written by one kernel of the forward before another one reads it.
  return moe_forward_impl(h, dtype, T, K, N, E, k, ffn_norm_w, out_norm_w, w_dtype, eps, w_router, w_gate, w_up, w_down,
                          act, x_scale, z_scale, out, idx_out, gate_out, ws, (size_t)STMOE_STATIC_SCRATCH_BYTES, variant, stream,
                          nullptr);
}
