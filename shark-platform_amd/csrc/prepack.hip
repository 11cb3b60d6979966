// One-time re-ordering of quantized expert weights into the streaming order the matrix-core kernels read.
//
// The planar planes of the reference layouts are row-major ([.., K/32, 32] int8, ...).  A wavefront that feeds
// MFMA operands straight from such rows touches 16 rows x 64 bytes per load instruction.  The packed order
// stores, for every tile of 16 consecutive weight rows, the bytes of one load instruction contiguously
// (1 KB: lane l = 16*g + n holds row n of the tile, 16 bytes of reduction group g), so that every wavefront
// load is one contiguous kilobyte, and stores the block scales of 256 reduction elements of the 16 rows as one
// contiguous 256-byte piece.  It is a permutation of the same bytes (nibbles for Q4_1): unpacking restores the planes bit for bit.
//
//   Q8_0 / fp8 samples: qs_p[rt][K/64][64 lanes][16 B]   lane (n,g): row 16*rt+n, k = 64*kb + 16*g .. +15
//   Q4_1 samples:       qs_p[rt][K/128][64 lanes][16 B]  lane (n,g): row 16*rt+n, k = 128*kb + 32*g .. +31 (one block);
//                       inside every dword (8 elements) the even elements fill the low half-word and the odd ones the
//                       high half-word (element 2p at bits 4p, 2p+1 at bits 16+4p): a pair comes out with one shift
//                       and one and-or
//   scales / offsets:   d_p[rt][K/256][16 rows][8] fp16  (8 consecutive blocks of one row)
// with rt running over all E*rows/16 row tiles.  Requires rows % 16 == 0 and cols % 256 == 0.
#include "weights.h"

namespace stmoe {

// kind 0: 1-byte samples, kind 1: Q4_1 nibbles, kind 2: fp16 block scales.  dir 0: pack, 1: unpack.
template <int KIND, int DIR>
__global__ void __launch_bounds__(256)
repack_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16, int64_t cols) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index of a 16-byte piece in packed order
  if (i >= n16) return;
  int64_t planar;  // index of the same 16-byte piece in planar order
  if (KIND == 0) {
    const int lane = (int)(i & 63), n = lane & 15, g = lane >> 4;
    const int64_t blk = i >> 6, kbs = cols >> 6, rt = blk / kbs, kb = blk - rt * kbs;
    planar = ((rt * 16 + n) * cols + kb * 64 + g * 16) >> 4;
  } else if (KIND == 1) {
    const int lane = (int)(i & 63), n = lane & 15, g = lane >> 4;
    const int64_t blk = i >> 6, kbs = cols >> 7, rt = blk / kbs, kb = blk - rt * kbs;
    planar = ((rt * 16 + n) * (cols >> 1) + kb * 64 + g * 16) >> 4;
  } else {
    const int n = (int)(i & 15);
    const int64_t blk = i >> 4, cs = cols >> 8, rt = blk / cs, c = blk - rt * cs;
    planar = ((rt * 16 + n) * (cols >> 5) + c * 8) >> 3;
  }
  uint4 v = DIR == 0 ? src[planar] : src[i];
  if (KIND == 1) {  // nibbles of every dword: linear order <-> even elements low / odd elements high
    if (DIR == 0) v = make_uint4(q4_dword_to_packed(v.x), q4_dword_to_packed(v.y), q4_dword_to_packed(v.z), q4_dword_to_packed(v.w));
    else v = make_uint4(q4_dword_to_linear(v.x), q4_dword_to_linear(v.y), q4_dword_to_linear(v.z), q4_dword_to_linear(v.w));
  }
  if (DIR == 0) dst[i] = v;
  else dst[planar] = v;
}

template <int KIND>
static int repack(const void* src, void* dst, int64_t bytes, int64_t cols, int dir, hipStream_t st) {
  const int64_t n16 = bytes >> 4;
  if (n16 == 0) return STMOE_OK;
  dim3 grid((unsigned)((n16 + 255) / 256));
  if (dir == 0) repack_kernel<KIND, 0><<<grid, 256, 0, st>>>((const uint4*)src, (uint4*)dst, n16, cols);
  else repack_kernel<KIND, 1><<<grid, 256, 0, st>>>((const uint4*)src, (uint4*)dst, n16, cols);
  return check_launch("repack");
}

static int repack_weight(const stmoe_weight* src, const stmoe_weight* dst, int dir, stmoe_stream_t stream) {
  const stmoe_weight* planar = dir == 0 ? src : dst;
  const stmoe_weight* packed = dir == 0 ? dst : src;
  STMOE_REQUIRE(src && dst, STMOE_ERR_NULL, "prepack: NULL descriptor");
  STMOE_REQUIRE(planar->experts == packed->experts && planar->rows == packed->rows && planar->cols == packed->cols,
                STMOE_ERR_SHAPE, "prepack: shapes differ");
  STMOE_REQUIRE(planar->rows % 16 == 0 && planar->cols % 256 == 0, STMOE_ERR_SHAPE,
                "prepack: needs rows %% 16 == 0 and cols %% 256 == 0 (got %lld x %lld)", (long long)planar->rows,
                (long long)planar->cols);
  STMOE_REQUIRE(src->qs && dst->qs && aligned16(src->qs) && aligned16(dst->qs), STMOE_ERR_ALIGN,
                "prepack: qs planes must be non-NULL and 16-byte aligned");
  const int64_t elems = planar->experts * planar->rows * planar->cols;
  hipStream_t st = as_stream(stream);
  int rc;
  if (planar->format == STMOE_W_Q8_0 && packed->format == STMOE_W_Q8_0_PACKED) {
    STMOE_REQUIRE(src->d && dst->d, STMOE_ERR_NULL, "prepack: d plane is NULL");
    if ((rc = repack<0>(src->qs, const_cast<void*>(dst->qs), elems, planar->cols, dir, st))) return rc;
    return repack<2>(src->d, const_cast<void*>(dst->d), elems / 16, planar->cols, dir, st);
  }
  if (planar->format == STMOE_W_Q4_1 && packed->format == STMOE_W_Q4_1_PACKED) {
    STMOE_REQUIRE(src->d && dst->d && src->m && dst->m, STMOE_ERR_NULL, "prepack: d/m plane is NULL");
    if ((rc = repack<1>(src->qs, const_cast<void*>(dst->qs), elems / 2, planar->cols, dir, st))) return rc;
    if ((rc = repack<2>(src->d, const_cast<void*>(dst->d), elems / 16, planar->cols, dir, st))) return rc;
    return repack<2>(src->m, const_cast<void*>(dst->m), elems / 16, planar->cols, dir, st);
  }
  if (planar->format == STMOE_W_FP8 && packed->format == STMOE_W_FP8_PACKED) {
    return repack<0>(src->qs, const_cast<void*>(dst->qs), elems, planar->cols, dir, st);  // the scale(s) are shared, not copied
  }
  return set_error(STMOE_ERR_UNSUPPORTED, "prepack: format pair %d -> %d has no packed order", src->format, dst->format);
}

// ---- raw ggml blocks -> planes (planar or streaming order) ---------------------------------------------
// One thread per 32-element block.  Q8_0 block: {f16 d; i8 qs[32]} (34 bytes); Q4_1 block: {f16 d; f16 m; u8 qs[16]}
// (20 bytes) with element i in the low nibble of byte i and element i + 16 in the high nibble.  The raw buffer is only
// 2-byte aligned, so it is read as half-words.  This kernel writes the planar planes.
template <int Q4>
__global__ void __launch_bounds__(256)
gguf_ingest_kernel(const uint16_t* __restrict__ raw, uint8_t* __restrict__ qs, uint16_t* __restrict__ d, uint16_t* __restrict__ m,
                   int64_t n_blocks, int64_t cols) {
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;  // block index in row-major [rows_total][cols / 32]
  if (b >= n_blocks) return;
  constexpr int HW = Q4 ? 10 : 17;  // half-words per raw block
  const uint16_t* src = raw + b * HW;
  d[b] = src[0];
  if (Q4) {
    m[b] = src[1];
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)src[2 + 2 * i] | ((uint32_t)src[3 + 2 * i] << 16);
    // linear order: element e at nibble e; elements 0..15 are the low nibbles of the 16 raw bytes, 16..31 the high ones
    uint32_t lin[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint32_t lo = 0, hi = 0;  // 8 consecutive low (high) nibbles of raw bytes 8 i .. 8 i + 7
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t byte = (w[2 * i + (j >> 2)] >> (8 * (j & 3))) & 0xffu;
        lo |= (byte & 0xfu) << (4 * j);
        hi |= (byte >> 4) << (4 * j);
      }
      lin[i] = lo;
      lin[2 + i] = hi;
    }
    reinterpret_cast<uint4*>(qs)[b] = make_uint4(lin[0], lin[1], lin[2], lin[3]);
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint32_t w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = (uint32_t)src[1 + 8 * h + 2 * i] | ((uint32_t)src[2 + 8 * h + 2 * i] << 16);
      reinterpret_cast<uint4*>(qs)[2 * b + h] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
}

// Streaming order, one thread per 16-byte piece of the output: a wavefront writes one contiguous kilobyte (lane 16 g + n
// = row n of the row tile, 16-element group g of the K step for Q8_0, block g of the four for Q4_1) and reads, per row,
// 68 (Q8_0) or 80 (Q4_1) consecutive raw bytes; the workgroups that follow continue the same cache lines.  Writing
// block by block as the kernel above does scatters 16-byte stores over the pieces and reaches 2.4 TB/s.
template <int Q4>
__global__ void __launch_bounds__(256)
gguf_ingest_packed_kernel(const uint16_t* __restrict__ raw, uint8_t* __restrict__ qs, uint16_t* __restrict__ d,
                          uint16_t* __restrict__ m, int64_t n_pieces, int64_t cols) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;  // output piece: [row tile][K step][lane]
  if (t >= n_pieces) return;
  const int lane = (int)(t & 63), n = lane & 15, g = lane >> 4;
  const int64_t step = t >> 6, bpr = cols >> 5;
  const int64_t steps_per_tile = Q4 ? (cols >> 7) : (cols >> 6);
  const int64_t rt = step / steps_per_tile, ks = step - rt * steps_per_tile;
  const int64_t kb32 = Q4 ? 4 * ks + g : 2 * ks + (g >> 1);  // 32-element block inside the row
  const int64_t b = (rt * 16 + n) * bpr + kb32;
  const int64_t dpos = ((rt * (cols >> 8) + (kb32 >> 3)) * 16 + n) * 8 + (kb32 & 7);
  if (Q4) {
    const uint16_t* src = raw + b * 10;
    d[dpos] = src[0];
    m[dpos] = src[1];
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)src[2 + 2 * i] | ((uint32_t)src[3 + 2 * i] << 16);
    uint32_t lin[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t byte = (w[2 * i + (j >> 2)] >> (8 * (j & 3))) & 0xffu;
        lo |= (byte & 0xfu) << (4 * j);
        hi |= (byte >> 4) << (4 * j);
      }
      lin[i] = lo;
      lin[2 + i] = hi;
    }
    reinterpret_cast<uint4*>(qs)[t] = make_uint4(q4_dword_to_packed(lin[0]), q4_dword_to_packed(lin[1]),
                                                 q4_dword_to_packed(lin[2]), q4_dword_to_packed(lin[3]));
  } else {
    const uint16_t* src = raw + b * 17;
    const int h = g & 1;
    if (h == 0) d[dpos] = src[0];
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)src[1 + 8 * h + 2 * i] | ((uint32_t)src[2 + 8 * h + 2 * i] << 16);
    reinterpret_cast<uint4*>(qs)[t] = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

static int gguf_ingest(const void* raw, int gguf_type, const stmoe_weight* out, stmoe_stream_t stream) {
  STMOE_REQUIRE(raw && out, STMOE_ERR_NULL, "gguf_ingest: NULL argument");
  STMOE_REQUIRE((reinterpret_cast<uintptr_t>(raw) & 1) == 0, STMOE_ERR_ALIGN, "gguf_ingest: raw blocks must be 2-byte aligned");
  STMOE_REQUIRE(out->experts >= 0 && out->rows >= 0 && out->cols >= 0 && out->cols % 32 == 0, STMOE_ERR_SHAPE,
                "gguf_ingest: cols must be a multiple of the block size 32 (got %lld)", (long long)out->cols);
  const bool q4 = gguf_type == STMOE_GGUF_Q4_1;
  STMOE_REQUIRE(q4 || gguf_type == STMOE_GGUF_Q8_0, STMOE_ERR_UNSUPPORTED, "gguf_ingest: unknown block type %d", gguf_type);
  const int planar_fmt = q4 ? STMOE_W_Q4_1 : STMOE_W_Q8_0, packed_fmt = q4 ? STMOE_W_Q4_1_PACKED : STMOE_W_Q8_0_PACKED;
  STMOE_REQUIRE(out->format == planar_fmt || out->format == packed_fmt, STMOE_ERR_UNSUPPORTED,
                "gguf_ingest: block type %d cannot become weight format %d", gguf_type, out->format);
  const bool packed = out->format == packed_fmt;
  if (packed)
    STMOE_REQUIRE(out->rows % 16 == 0 && out->cols % 256 == 0, STMOE_ERR_SHAPE,
                  "gguf_ingest: the streaming order needs rows %% 16 == 0 and cols %% 256 == 0 (got %lld x %lld)",
                  (long long)out->rows, (long long)out->cols);
  const int64_t n_blocks = out->experts * out->rows * (out->cols / 32);
  if (n_blocks == 0) return STMOE_OK;
  STMOE_REQUIRE(out->qs && out->d && (!q4 || out->m), STMOE_ERR_NULL, "gguf_ingest: output plane is NULL");
  STMOE_REQUIRE(aligned16(out->qs), STMOE_ERR_ALIGN, "gguf_ingest: qs plane must be 16-byte aligned");
  STMOE_REQUIRE((n_blocks + 255) / 256 < ((int64_t)1 << 31), STMOE_ERR_SHAPE, "gguf_ingest: too many blocks");
  hipStream_t st = as_stream(stream);
  dim3 grid((unsigned)((n_blocks + 255) / 256));
  auto* qs = static_cast<uint8_t*>(const_cast<void*>(out->qs));
  auto* d = static_cast<uint16_t*>(const_cast<void*>(out->d));
  auto* m = static_cast<uint16_t*>(const_cast<void*>(out->m));
  const auto* r = static_cast<const uint16_t*>(raw);
  if (packed) {
    const int64_t n_pieces = q4 ? n_blocks : 2 * n_blocks;
    STMOE_REQUIRE((n_pieces + 255) / 256 < ((int64_t)1 << 31), STMOE_ERR_SHAPE, "gguf_ingest: too many blocks");
    dim3 pgrid((unsigned)((n_pieces + 255) / 256));
    if (q4) gguf_ingest_packed_kernel<1><<<pgrid, 256, 0, st>>>(r, qs, d, m, n_pieces, out->cols);
    else gguf_ingest_packed_kernel<0><<<pgrid, 256, 0, st>>>(r, qs, d, nullptr, n_pieces, out->cols);
  } else if (q4) {
    gguf_ingest_kernel<1><<<grid, 256, 0, st>>>(r, qs, d, m, n_blocks, out->cols);
  } else {
    gguf_ingest_kernel<0><<<grid, 256, 0, st>>>(r, qs, d, nullptr, n_blocks, out->cols);
  }
  return check_launch("gguf_ingest");
}

}  // namespace stmoe

extern "C" int stmoe_gguf_ingest(const void* raw_blocks, int gguf_type, const stmoe_weight* out, stmoe_stream_t stream) {
  return stmoe::gguf_ingest(raw_blocks, gguf_type, out, stream);
}

extern "C" int stmoe_prepack(const stmoe_weight* planar, const stmoe_weight* packed_out, stmoe_stream_t stream) {
  return stmoe::repack_weight(planar, packed_out, 0, stream);
}

extern "C" int stmoe_unpack(const stmoe_weight* packed, const stmoe_weight* planar_out, stmoe_stream_t stream) {
  return stmoe::repack_weight(packed, planar_out, 1, stream);
}
