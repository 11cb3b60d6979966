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

}  // namespace stmoe

extern "C" int stmoe_prepack(const stmoe_weight* planar, const stmoe_weight* packed_out, stmoe_stream_t stream) {
  return stmoe::repack_weight(planar, packed_out, 0, stream);
}

extern "C" int stmoe_unpack(const stmoe_weight* packed, const stmoe_weight* planar_out, stmoe_stream_t stream) {
  return stmoe::repack_weight(packed, planar_out, 1, stream);
}
