// Fused int4 dequant + GEMM (prefill-sized batches) on fp16 MFMA for gfx950.
//
// y[m][n] = sum_k x[m][k] * W[n][k] (+ out_bias[n]),  W[n][k] = code * scale[n][k/gs] + bias[n][k/gs]
// -- LinearGQ.build with dim=0 (popxl_addons/layers/linear_gq.py:99-109); the fp16 weight only
// ever exists in LDS/registers.  Bound by the fp16 dense MFMA rate for m_rows >= 512.
#include "gq_common.h"

namespace gq {

int launch_gemv_generic_rows(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                             const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                             int64_t k_in, int64_t group_size, hipStream_t stream);

namespace {

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t as_u32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

// 8 codes of one packed word -> 8 fp16 weights in memory order (see gq_decompress.hip for the
// nibble order).  Codes are exact; scale and bias are applied with one packed fma.
__device__ __forceinline__ uint4_t dequant_word_ordered(uint32_t w, half2_t s2, half2_t b2) {
  const half2_t kNeg1024 = {(half_t)-1024.0f, (half_t)-1024.0f};
  const half2_t kSixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  const half2_t kNeg64 = {(half_t)-64.0f, (half_t)-64.0f};
  const uint32_t hi = w >> 8;
  const half2_t c0 = __builtin_elementwise_fma(as_half2((hi & 0x00F000F0u) | 0x64006400u), kSixteenth, kNeg64);
  const half2_t c1 = as_half2((hi & 0x000F000Fu) | 0x64006400u) + kNeg1024;
  const half2_t c2 = __builtin_elementwise_fma(as_half2((w & 0x00F000F0u) | 0x64006400u), kSixteenth, kNeg64);
  const half2_t c3 = as_half2((w & 0x000F000Fu) | 0x64006400u) + kNeg1024;
  const uint32_t r0 = as_u32(__builtin_elementwise_fma(c0, s2, b2));  // elements (0,4)
  const uint32_t r1 = as_u32(__builtin_elementwise_fma(c1, s2, b2));  // (1,5)
  const uint32_t r2 = as_u32(__builtin_elementwise_fma(c2, s2, b2));  // (2,6)
  const uint32_t r3 = as_u32(__builtin_elementwise_fma(c3, s2, b2));  // (3,7)
  uint4_t o;
  o.x = __builtin_amdgcn_perm(r1, r0, 0x05040100u);
  o.y = __builtin_amdgcn_perm(r3, r2, 0x05040100u);
  o.z = __builtin_amdgcn_perm(r1, r0, 0x07060302u);
  o.w = __builtin_amdgcn_perm(r3, r2, 0x07060302u);
  return o;
}

// ---------------------------------------------------------------------------------------
// Tile kernel.  Workgroup = 4 waves (2 x 2), tile 128 (m) x 128 (n) x 64 (k).  The x tile and
// the dequantised weight tile sit in LDS as fp16 with padded rows; each wave owns a 64 x 64
// sub-tile = 2 x 2 v_mfma_f32_32x32x16_f16 accumulators.  Global loads for tile t+1 are issued
// before the MFMAs of tile t.
// ---------------------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 64, LDK = BK + 8;

__global__ __launch_bounds__(256) void gemm_tile_kernel(const half_t *__restrict__ x, int m_rows,
                                                        const uint4_t *__restrict__ packed,
                                                        const half_t *__restrict__ scale,
                                                        const half_t *__restrict__ bias,
                                                        const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                        int n_out, int k_in, int gs_shift) {
  __shared__ __attribute__((aligned(16))) half_t As[BM][LDK];
  __shared__ __attribute__((aligned(16))) half_t Bs[BN][LDK];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int groups_per_row = k_in >> gs_shift;

  // global -> register staging assignments
  const int a_col = (tid & 7) * 8;  // 8 fp16 = 16 bytes
  const int a_row = tid >> 3;       // + 32 * i
  const int b_row = tid >> 1, b_half = tid & 1;
  const int b_grow = min(n0 + b_row, n_out - 1);
  const uint4_t *b_src = packed + (int64_t)b_grow * (k_in >> 5) + b_half;
  const half_t *s_src = scale + (int64_t)b_grow * groups_per_row;
  const half_t *z_src = bias + (int64_t)b_grow * groups_per_row;
  const half_t *a_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) a_src[i] = x + (int64_t)min(m0 + a_row + 32 * i, m_rows - 1) * k_in + a_col;

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  uint4_t a_reg[4], b_reg;
  half_t s_reg, z_reg;
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) a_reg[i] = *reinterpret_cast<const uint4_t *>(a_src[i] + k0);
    b_reg = b_src[k0 >> 5];
    const int g = (k0 + b_half * 32) >> gs_shift;
    s_reg = s_src[g];
    z_reg = z_src[g];
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4_t *>(&As[a_row + 32 * i][a_col]) = a_reg[i];
    const half2_t s2 = {s_reg, s_reg}, z2 = {z_reg, z_reg};
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<uint4_t *>(&Bs[b_row][b_half * 32 + q * 8]) = dequant_word_ordered(b_reg[q], s2, z2);
  };

  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
  load_tile(0);
  for (int k0 = 0; k0 < k_in; k0 += BK) {
    __syncthreads();
    store_tile();
    __syncthreads();
    if (k0 + BK < k_in) load_tile(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      half8_t a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i] = *reinterpret_cast<const half8_t *>(&As[wm * 64 + i * 32 + frag_row][ks + frag_k]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        b[j] = *reinterpret_cast<const half8_t *>(&Bs[wn * 64 + j * 32 + frag_row][ks + frag_k]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }

  // D[m][n]: lane holds n = lane % 32 and m = 8 * (e / 4) + 4 * (lane / 32) + e % 4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + (lane & 31);
      if (n >= n_out) continue;
      const float ob = out_bias ? (float)out_bias[n] : 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (m < m_rows) y[(int64_t)m * n_out + n] = (half_t)(acc[i][j][e] + ob);
      }
    }
}

}  // namespace

int launch_gemm(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, hipStream_t stream) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  const bool fast_ok = pow2 && group_size >= 32 && k_in % BK == 0 && k_in > 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)packed % 16) == 0;
  if (!fast_ok || option_gemm_variant() == 1)
    return launch_gemv_generic_rows(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, stream);
  const int gs_shift = __builtin_ctzll((unsigned long long)group_size);
  const dim3 grid((unsigned)((n_out + BN - 1) / BN), (unsigned)((m_rows + BM - 1) / BM));
  if (grid.y > 65535) return fail(GQ_ERR_UNSUPPORTED, "gq_gemm_f16: m_rows=%lld too large", (long long)m_rows);
  gemm_tile_kernel<<<grid, dim3(256), 0, stream>>>(
      reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const uint4_t *>(packed),
      reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
      reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, gs_shift);
  return check_launch("gemm_tile_kernel");
}

}  // namespace gq
