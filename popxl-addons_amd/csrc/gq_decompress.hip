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

template <bool NT>
__device__ __forceinline__ void store16(uint4_t *p, uint4_t v) {
  if (NT)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

template <typename T, bool NT>
__device__ __forceinline__ T load_packed(const T *p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}

// Fast path.  One work item = WORDS consecutive 32-bit words of the flattened packed tensor
// (WORDS in {1, 2, 4}: a 4/8/16-byte load) -> WORDS 16-byte stores.  All words of an item
// lie in one group (the launcher guarantees WORDS divides the words per group), so an item
// needs one (scale, bias) pair.  Items are dealt to lanes so that consecutive lanes take
// consecutive items: with WORDS == 1 every load and store instruction of a wave covers one
// contiguous span (256 B read, 1 KiB written).  A workgroup walks the tensor with a grid
// stride of THREADS * UNROLL items; the launcher picks the grid (one pass or persistent).
template <int THREADS, int WORDS, int UNROLL, bool NT_LOAD, bool NT_STORE>
__global__ __launch_bounds__(THREADS) void decompress_kernel(const uint32_t *__restrict__ packed,
                                                             const half_t *__restrict__ scale,
                                                             const half_t *__restrict__ bias,
                                                             uint4_t *__restrict__ out, int64_t n_items,
                                                             int items_per_group_shift) {
  typedef uint32_t vec_t __attribute__((ext_vector_type(WORDS)));
  const int64_t stride = (int64_t)gridDim.x * (THREADS * UNROLL);
  for (int64_t base = (int64_t)blockIdx.x * (THREADS * UNROLL) + threadIdx.x; base < n_items; base += stride) {
    vec_t w[UNROLL];
    half_t s[UNROLL], b[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t item = base + (int64_t)u * THREADS;
      if (item < n_items) {
        w[u] = load_packed<vec_t, NT_LOAD>(reinterpret_cast<const vec_t *>(packed) + item);
        const int64_t group = item >> items_per_group_shift;
        s[u] = scale[group];
        b[u] = bias[group];
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t item = base + (int64_t)u * THREADS;
      if (item < n_items) {
        const half2_t s2 = {s[u], s[u]}, b2 = {b[u], b[u]};
        uint4_t *dst = out + item * WORDS;
#pragma unroll
        for (int k = 0; k < WORDS; ++k) store16<NT_STORE>(dst + k, expand_word(w[u][k], s2, b2));
      }
    }
  }
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

template <int THREADS, int WORDS, int UNROLL, bool NT_LOAD, bool NT_STORE>
void launch_fast(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, uint16_t *out,
                 int64_t n_words16, int shift, int64_t max_blocks, hipStream_t stream) {
  const int64_t n_items = n_words16 / (2 * WORDS);
  const int64_t per_block = (int64_t)THREADS * UNROLL;
  int64_t blocks = (n_items + per_block - 1) / per_block;
  if (max_blocks > 0 && blocks > max_blocks) blocks = max_blocks;
  decompress_kernel<THREADS, WORDS, UNROLL, NT_LOAD, NT_STORE><<<dim3((unsigned)blocks), dim3(THREADS), 0, stream>>>(
      reinterpret_cast<const uint32_t *>(packed), reinterpret_cast<const half_t *>(scale),
      reinterpret_cast<const half_t *>(bias), reinterpret_cast<uint4_t *>(out), n_items, shift);
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
        (uintptr_t)out % 16 == 0 && option_decompress_variant() != 900) {
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
  const uintptr_t pa = (uintptr_t)packed, oa = (uintptr_t)out;
  const bool out16 = (oa % 16) == 0;
  const int variant = option_decompress_variant();
  // 32-bit words per work item: 1 unless a diagnostic variant asks for wider items.  Items must
  // tile a group (power-of-two count per group so the group index is a shift) and be aligned.
  auto usable = [&](int words) {
    if (!out16 || n_ids % (2 * words) != 0 || pa % (4 * words) != 0) return false;
    const int64_t ipg = n_ids / (2 * words);
    return (ipg & (ipg - 1)) == 0;
  };
  int words = usable(1) ? 1 : 0;
  if (variant >= 200 && variant < 300 && usable(2)) words = 2;
  if (variant >= 400 && variant < 500 && usable(4)) words = 4;
  if ((n_words + 1) / 2 / kThreads >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "decompress: tensor too large");
  if (words == 0) {
    const int64_t blocks = (n_words + kThreads - 1) / kThreads;
    decompress_scalar_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
        packed, reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
        reinterpret_cast<half_t *>(out), n_words, n_ids);
    return check_launch("decompress_scalar_kernel");
  }
  const int shift = __builtin_ctzll((unsigned long long)(n_ids / (2 * words)));
  const int sub = variant % 100;
#define GQ_ARGS packed, scale, bias, out, n_words, shift
  if (words == 4) {
    launch_fast<256, 4, 1, false, false>(GQ_ARGS, 0, stream);
  } else if (words == 2) {
    launch_fast<256, 2, 1, false, true>(GQ_ARGS, 0, stream);
  } else {
    switch (sub) {
      case 1: launch_fast<256, 1, 1, false, false>(GQ_ARGS, 0, stream); break;
      case 2: launch_fast<256, 1, 1, true, false>(GQ_ARGS, 0, stream); break;
      case 3: launch_fast<256, 1, 1, false, true>(GQ_ARGS, 0, stream); break;
      case 4: launch_fast<256, 1, 1, true, true>(GQ_ARGS, 0, stream); break;
      case 5: launch_fast<512, 1, 1, false, true>(GQ_ARGS, 0, stream); break;
      case 6: launch_fast<1024, 1, 1, false, true>(GQ_ARGS, 0, stream); break;
      case 7: launch_fast<128, 1, 1, false, true>(GQ_ARGS, 0, stream); break;
      case 8: launch_fast<64, 1, 1, false, true>(GQ_ARGS, 0, stream); break;
      case 9: launch_fast<256, 1, 2, false, true>(GQ_ARGS, 0, stream); break;
      case 10: launch_fast<256, 1, 4, false, true>(GQ_ARGS, 0, stream); break;
      case 11: launch_fast<256, 1, 1, false, true>(GQ_ARGS, 256 * 8, stream); break;
      case 12: launch_fast<256, 1, 1, false, true>(GQ_ARGS, 256 * 16, stream); break;
      case 13: launch_fast<256, 1, 1, false, true>(GQ_ARGS, 256 * 32, stream); break;
      case 14: launch_fast<512, 1, 1, false, true>(GQ_ARGS, 256 * 4, stream); break;
      case 15: launch_fast<512, 1, 1, false, true>(GQ_ARGS, 256 * 8, stream); break;
      case 16: launch_fast<1024, 1, 1, false, true>(GQ_ARGS, 256 * 2, stream); break;
      case 17: launch_fast<256, 1, 2, false, true>(GQ_ARGS, 256 * 8, stream); break;
      case 18: launch_fast<256, 1, 2, false, true>(GQ_ARGS, 256 * 16, stream); break;
      case 19: launch_fast<512, 1, 2, false, true>(GQ_ARGS, 0, stream); break;
      case 20: launch_fast<128, 1, 2, false, true>(GQ_ARGS, 0, stream); break;
      default: launch_fast<512, 1, 1, false, true>(GQ_ARGS, 0, stream); break;
    }
  }
#undef GQ_ARGS
  return check_launch("decompress_kernel");
}

}  // namespace gq
