// Standalone int4 -> fp16 group-quantization decompress for gfx950.
//
// Replaces the two device passes of the reference lowering
// (group_quantize_decompressx.cpp:51-109: unpack vertex, then popops::map(_1*_2+_3))
// with one pass.  HBM-bound: per element 0.5 B of codes + 4/group_size B of scale/bias are
// read and 2 B are written.
//
// Numerics (group_quantize_decompress.py:133-134): value = f16(f16(code * scale) + bias).
// This translation unit is compiled with -ffp-contract=off so the multiply and the add
// stay two separately rounded packed-fp16 instructions; the build checks the ISA for that.
#include "gq_common.h"

namespace gq {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t as_u32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

// One 32-bit word = two little-endian uint16 = eight codes.  Memory order of the results:
// word bits 15:12, 11:8, 7:4, 3:0, then 31:28, 27:24, 23:20, 19:16 (most significant
// nibble of each uint16 first, group_quantize_decompress.py:130).
// Codes are made exact in fp16 by or-ing the nibble into the mantissa of 1024.0 (0x6400)
// and subtracting 1024; each step handles the pair (element j, element j + 4).
__device__ __forceinline__ uint4_t expand_word(uint32_t w, half2_t s2, half2_t b2) {
  const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
  half2_t r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t pair = ((w >> (12 - 4 * j)) & 0x000F000Fu) | 0x64006400u;
    const half2_t code = as_half2(pair) - k1024;  // exact
    const half2_t prod = code * s2;               // rounded to fp16
    r[j] = prod + b2;                             // rounded to fp16 (no fma: contraction is off)
  }
  // r[j] = (element j, element j + 4)  ->  dwords (0,1) (2,3) (4,5) (6,7)
  uint4_t o;
  o.x = __builtin_amdgcn_perm(as_u32(r[1]), as_u32(r[0]), 0x05040100u);
  o.y = __builtin_amdgcn_perm(as_u32(r[3]), as_u32(r[2]), 0x05040100u);
  o.z = __builtin_amdgcn_perm(as_u32(r[1]), as_u32(r[0]), 0x07060302u);
  o.w = __builtin_amdgcn_perm(as_u32(r[3]), as_u32(r[2]), 0x07060302u);
  return o;
}

// Fast path.  One lane = one 32-bit word of the flattened packed tensor (8 codes) -> one 16-byte
// store: every load instruction of a wave covers 256 contiguous bytes and every store 1 KiB.
// Loads are ordinary cached loads (8 lanes share a scale/bias pair), stores are non-temporal.
// One pass over the tensor, 512 threads per workgroup (measured against 64..1024 threads, wider
// items per lane, non-temporal loads and persistent grids: all slower).
constexpr int kFastThreads = 512;
__global__ __launch_bounds__(kFastThreads) void decompress_kernel(const uint32_t *__restrict__ packed,
                                                                  const half_t *__restrict__ scale,
                                                                  const half_t *__restrict__ bias,
                                                                  uint4_t *__restrict__ out, int64_t n_items,
                                                                  int items_per_group_shift) {
  const int64_t item = (int64_t)blockIdx.x * kFastThreads + threadIdx.x;
  if (item >= n_items) return;
  const uint32_t w = packed[item];
  const int64_t group = item >> items_per_group_shift;
  const half_t s = scale[group], b = bias[group];
  const half2_t s2 = {s, s}, b2 = {b, b};
  __builtin_nontemporal_store(expand_word(w, s2, b2), out + item);
}

// Any shape and any 2-byte alignment: one uint16 (four codes) per lane.
__global__ __launch_bounds__(kThreads) void decompress_scalar_kernel(const uint16_t *__restrict__ packed,
                                                                     const half_t *__restrict__ scale,
                                                                     const half_t *__restrict__ bias,
                                                                     half_t *__restrict__ out, int64_t n_words,
                                                                     int64_t n_ids) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n_words) return;
  const uint32_t w = packed[i];
  const int64_t group = i / n_ids;
  const half_t s = scale[group], b = bias[group];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const half_t code = (half_t)(float)((w >> (12 - 4 * j)) & 15u);
    const half_t prod = code * s;
    out[i * 4 + j] = prod + b;
  }
}

// Transposed result out_t[c][r] (c = column of the decompressed row).  A workgroup expands a
// tile of 64 rows x 16 uint16 (64 columns) into LDS and writes it out with rows contiguous.
constexpr int kTileRows = 64, kTileWords = 16, kTileCols = kTileWords * 4;
__global__ __launch_bounds__(kThreads) void decompress_transposed_kernel(
    const uint16_t *__restrict__ packed, const half_t *__restrict__ scale, const half_t *__restrict__ bias,
    half_t *__restrict__ out_t, int64_t rows, int64_t words_per_row, int64_t n_ids) {
  __shared__ half_t tile[kTileCols][kTileRows + 2];
  const int64_t row0 = (int64_t)blockIdx.y * kTileRows, word0 = (int64_t)blockIdx.x * kTileWords;
  const int64_t n_groups = words_per_row / n_ids;
  for (int t = threadIdx.x; t < kTileRows * kTileWords; t += kThreads) {
    const int r = t / kTileWords, wi = t % kTileWords;
    const int64_t row = row0 + r, word = word0 + wi;
    if (row < rows && word < words_per_row) {
      const uint32_t w = packed[row * words_per_row + word];
      const int64_t group = row * n_groups + word / n_ids;
      const half_t s = scale[group], b = bias[group];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half_t code = (half_t)(float)((w >> (12 - 4 * j)) & 15u);
        const half_t prod = code * s;
        tile[wi * 4 + j][r] = prod + b;
      }
    }
  }
  __syncthreads();
  for (int t = threadIdx.x; t < kTileCols * kTileRows; t += kThreads) {
    const int c = t / kTileRows, r = t % kTileRows;
    const int64_t row = row0 + r, col = word0 * 4 + c;
    if (row < rows && col < words_per_row * 4) out_t[col * rows + row] = tile[c][r];
  }
}

// Transposed result, fast path: a workgroup expands a tile of 128 rows x 128 columns.
// Phase 1: thread (quarter q, row pair rp) loads the 16 bytes = 32 codes of quarter q of rows
// 2 rp and 2 rp + 1, and computes every column for both rows at once as the two halves of
// packed fp16 instructions (their scales and biases differ: s2 = (row a, row b)); the pair goes
// to LDS column c as one 32-bit word.  Phase 2: a thread reads 8 consecutive rows of a column
// (16 bytes) and stores them; 16 threads cover the 256 contiguous bytes of a column of the tile.
// LDS: column c starts at c * 272 bytes; the row pair rp of a column of quarter q sits at word
// rp ^ (16 q), so that the 64 lanes of a wave (4 quarters x 16 row pairs) write 64 different banks.
constexpr int kFastTile = 128, kFastStride = 272;
__global__ __launch_bounds__(256) void decompress_transposed_tile_kernel(
    const uint16_t *__restrict__ packed, const half_t *__restrict__ scale, const half_t *__restrict__ bias,
    half_t *__restrict__ out_t, int64_t rows, int64_t words_per_row, int n_ids) {
  __shared__ __attribute__((aligned(16))) char tile[kFastTile * kFastStride];
  const int t = threadIdx.x, q = t & 3, rp = t >> 2;
  // (row tiles vary fastest: workgroups that run together write neighbouring stretches of the same columns)
  const int64_t row0 = (int64_t)blockIdx.x * kFastTile, word0 = (int64_t)blockIdx.y * (kFastTile / 4);
  const int64_t n_groups = words_per_row / n_ids;
  {
    // rows past the end repeat the last one (their results are never stored)
    const int64_t ra = min(row0 + 2 * rp, rows - 1), rb = min(row0 + 2 * rp + 1, rows - 1);
    const int64_t word = word0 + q * 8, group = word / n_ids;
    const uint4_t da = *reinterpret_cast<const uint4_t *>(packed + ra * words_per_row + word);
    const uint4_t db = *reinterpret_cast<const uint4_t *>(packed + rb * words_per_row + word);
    const half2_t s2 = {scale[ra * n_groups + group], scale[rb * n_groups + group]};
    const half2_t b2 = {bias[ra * n_groups + group], bias[rb * n_groups + group]};
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    char *dst = tile + (q * 32) * kFastStride + (rp ^ (q << 4)) * 4;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      // uint16 word 2k (low halves) and 2k + 1 (high halves) of both rows: (row a, row b)
      const uint32_t both[2] = {__builtin_amdgcn_perm(db[k], da[k], 0x05040100u),
                                __builtin_amdgcn_perm(db[k], da[k], 0x07060302u)};
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t pair = ((both[u] >> (12 - 4 * j)) & 0x000F000Fu) | 0x64006400u;
          const half2_t code = as_half2(pair) - k1024;  // exact
          const half2_t prod = code * s2;               // rounded to fp16
          const half2_t v = prod + b2;                  // rounded to fp16
          *reinterpret_cast<uint32_t *>(dst + ((2 * k + u) * 4 + j) * kFastStride) = as_u32(v);
        }
    }
  }
  __syncthreads();
  const int rg = t & 15;  // rows 8 rg .. 8 rg + 7 of the tile
  const int64_t row = row0 + rg * 8;
  if (row >= rows) return;  // (rows is a multiple of 8)
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = (t >> 4) + 16 * i;
    const uint4_t v = *reinterpret_cast<const uint4_t *>(tile + c * kFastStride + ((4 * rg) ^ ((c >> 5) << 4)) * 4);
    __builtin_nontemporal_store(v, reinterpret_cast<uint4_t *>(out_t + (word0 * 4 + c) * rows + row));
  }
}

}  // namespace

int launch_decompress(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, uint16_t *out,
                      int64_t rows, int64_t n_groups, int64_t n_ids, bool transposed, hipStream_t stream) {
  const int64_t n_words = rows * n_groups * n_ids;
  if (n_words == 0) return GQ_OK;
  if (transposed) {
    const int64_t words_per_row = n_groups * n_ids;
    // tiles of 128 x 128 with 16-byte accesses throughout
    if (words_per_row % (kFastTile / 4) == 0 && n_ids % 8 == 0 && rows % 8 == 0 && (uintptr_t)packed % 16 == 0 &&
        (uintptr_t)out % 16 == 0) {
      const int64_t gx = words_per_row / (kFastTile / 4), gy = (rows + kFastTile - 1) / kFastTile;
      if (gx > 65535 || gy > 0x7fffffff)
        return fail(GQ_ERR_UNSUPPORTED, "transposed decompress: tensor too large (columns=%lld)", (long long)words_per_row * 4);
      decompress_transposed_tile_kernel<<<dim3((unsigned)gy, (unsigned)gx), dim3(256), 0, stream>>>(
          packed, reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
          reinterpret_cast<half_t *>(out), rows, words_per_row, (int)n_ids);
      return check_launch("decompress_transposed_tile_kernel");
    }
    const int64_t gx = (words_per_row + kTileWords - 1) / kTileWords, gy = (rows + kTileRows - 1) / kTileRows;
    if (gy > 65535) return fail(GQ_ERR_UNSUPPORTED, "transposed decompress: rows=%lld exceeds 65535*64", (long long)rows);
    decompress_transposed_kernel<<<dim3((unsigned)gx, (unsigned)gy), dim3(kThreads), 0, stream>>>(
        packed, reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
        reinterpret_cast<half_t *>(out), rows, words_per_row, n_ids);
    return check_launch("decompress_transposed_kernel");
  }
  // the fast kernel needs whole 32-bit words that tile a group (a power-of-two count per group,
  // so that the group index is a shift), a 4-byte aligned input and a 16-byte aligned output
  const int64_t words_per_group = n_ids / 2;
  const bool fast = n_ids % 2 == 0 && (words_per_group & (words_per_group - 1)) == 0 && (uintptr_t)packed % 4 == 0 &&
                    (uintptr_t)out % 16 == 0;
  if ((n_words + 1) / 2 / kThreads >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "decompress: tensor too large");
  if (!fast) {
    const int64_t blocks = (n_words + kThreads - 1) / kThreads;
    decompress_scalar_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
        packed, reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
        reinterpret_cast<half_t *>(out), n_words, n_ids);
    return check_launch("decompress_scalar_kernel");
  }
  const int shift = __builtin_ctzll((unsigned long long)words_per_group);
  const int64_t n_items = n_words / 2;
  const int64_t blocks = (n_items + kFastThreads - 1) / kFastThreads;
  decompress_kernel<<<dim3((unsigned)blocks), dim3(kFastThreads), 0, stream>>>(
      reinterpret_cast<const uint32_t *>(packed), reinterpret_cast<const half_t *>(scale),
      reinterpret_cast<const half_t *>(bias), reinterpret_cast<uint4_t *>(out), n_items, shift);
  return check_launch("decompress_kernel");
}

}  // namespace gq
