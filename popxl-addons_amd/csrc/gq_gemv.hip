// Fused int4 dequant + GEMV (decode-sized batches, 1 <= m_rows <= 16) for gfx950.
//
// y[m][n] = sum_k x[m][k] * W[n][k] (+ out_bias[n]) with W[n][k] = code * scale[n][k/gs] + bias[n][k/gs]
// -- LinearGQ.build with dim=0 (popxl_addons/layers/linear_gq.py:99-109) without ever
// writing the fp16 weight to memory.  HBM-bound on the packed weight: 0.5 + 4/gs bytes per
// weight element.
#include "gq_common.h"

namespace gq {
namespace {

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

// ---------------------------------------------------------------------------------------
// MFMA path.  v_mfma_f32_16x16x32_f16 computes D[16x16] += A[16x32] * B[32x16]; here A holds
// 16 weight rows (n), B holds the (zero padded) batch as 16 columns (m).  Lane l supplies
// row/column l%16 and the 8 contraction indices of k-chunk l/16, so the 8 codes of one packed
// 32-bit word are exactly one lane's A operand.  The contraction index is a dummy: codes are
// expanded in the order (0,4,1,5,2,6,3,7) of their memory positions, and x is permuted the
// same way, which saves re-pairing the weights.
//
// A wave owns 16 rows and walks K in chunks of 512 (four 16-byte loads per lane); the waves of
// a workgroup take interleaved chunks of the same 16 rows and their partial sums meet in LDS.
// ---------------------------------------------------------------------------------------

// 8 codes of `w` -> 8 fp16 weights, order (0,4,1,5,2,6,3,7).  The nibble is or-ed into the
// mantissa of 1024.0 (ulp 1) or, for nibbles sitting at bits 7:4, read as 1024 + 16*code; both
// are brought back to the exact code with one packed op, then scaled with a packed fma.
__device__ __forceinline__ half8_t dequant_word(uint32_t w, half2_t s2, half2_t b2) {
  const half2_t kNeg1024 = {(half_t)-1024.0f, (half_t)-1024.0f};
  const half2_t kSixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  const half2_t kNeg64 = {(half_t)-64.0f, (half_t)-64.0f};
  const uint32_t hi = w >> 8;
  const half2_t c0 = __builtin_elementwise_fma(as_half2((hi & 0x00F000F0u) | 0x64006400u), kSixteenth, kNeg64);
  const half2_t c1 = as_half2((hi & 0x000F000Fu) | 0x64006400u) + kNeg1024;
  const half2_t c2 = __builtin_elementwise_fma(as_half2((w & 0x00F000F0u) | 0x64006400u), kSixteenth, kNeg64);
  const half2_t c3 = as_half2((w & 0x000F000Fu) | 0x64006400u) + kNeg1024;
  const half2_t w0 = __builtin_elementwise_fma(c0, s2, b2);
  const half2_t w1 = __builtin_elementwise_fma(c1, s2, b2);
  const half2_t w2 = __builtin_elementwise_fma(c2, s2, b2);
  const half2_t w3 = __builtin_elementwise_fma(c3, s2, b2);
  half8_t r;
  r[0] = w0[0]; r[1] = w0[1]; r[2] = w1[0]; r[3] = w1[1];
  r[4] = w2[0]; r[5] = w2[1]; r[6] = w3[0]; r[7] = w3[1];
  return r;
}

// 8 consecutive fp16 of x -> order (0,4,1,5,2,6,3,7)
__device__ __forceinline__ half8_t permute_x(uint4_t q) {
  uint4_t p;
  p.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);
  p.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);
  p.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);
  p.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);
  return __builtin_bit_cast(half8_t, p);
}

template <int NWAVES>
__global__ __launch_bounds__(NWAVES * 64) void gemv_mfma_kernel(
    const half_t *__restrict__ x, int m_rows, const uint4_t *__restrict__ packed, const half_t *__restrict__ scale,
    const half_t *__restrict__ bias, const half_t *__restrict__ out_bias, half_t *__restrict__ y, int n_out, int k_in,
    int gs_shift) {
  __shared__ float4_t partial[NWAVES][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int row = min((int)blockIdx.x * 16 + r, n_out - 1);
  const int n_slots = k_in >> 7;  // 128 contraction indices = 4 lanes x 16 bytes per row
  const int groups_per_row = k_in >> gs_shift;
  const uint4_t *wrow = packed + (int64_t)row * (k_in >> 5);
  const half_t *srow = scale + (int64_t)row * groups_per_row;
  const half_t *brow = bias + (int64_t)row * groups_per_row;
  const bool has_x = r < m_rows;
  const half_t *xrow = x + (int64_t)(has_x ? r : 0) * k_in;

  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int c = wave; c * 4 < n_slots; c += NWAVES) {
    uint4_t wq[4], xq[4][4];
    half_t sc[4], bi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int slot = c * 4 + j;
      const bool valid = slot < n_slots;
      const int k0 = slot * 128 + kc * 32;
      wq[j] = uint4_t{0u, 0u, 0u, 0u};
      sc[j] = (half_t)0.f;
      bi[j] = (half_t)0.f;
      if (valid) {
        wq[j] = __builtin_nontemporal_load(wrow + slot * 4 + kc);
        sc[j] = srow[k0 >> gs_shift];
        bi[j] = brow[k0 >> gs_shift];
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        xq[j][s] = uint4_t{0u, 0u, 0u, 0u};
        if (valid && has_x) xq[j][s] = *reinterpret_cast<const uint4_t *>(xrow + k0 + s * 8);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const half2_t s2 = {sc[j], sc[j]}, b2 = {bi[j], bi[j]};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const half8_t a = dequant_word(wq[j][s], s2, b2);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, permute_x(xq[j][s]), acc, 0, 0, 0);
      }
    }
  }
  partial[wave][lane] = acc;
  __syncthreads();
  if (wave == 0) {
    float4_t sum = partial[0][lane];
#pragma unroll
    for (int w = 1; w < NWAVES; ++w) sum += partial[w][lane];
    // lane holds D[n = 4*kc + i][m = r]
    if (r < m_rows) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = (int)blockIdx.x * 16 + 4 * kc + i;
        if (n < n_out) {
          float v = sum[i];
          if (out_bias) v += (float)out_bias[n];
          y[(int64_t)r * n_out + n] = (half_t)v;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Generic path: any group_size % 4 == 0, any alignment.  One wave per output row; the weight is
// rebuilt exactly as the standalone decompress does (two fp16 roundings) and accumulated in fp32.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gemv_generic_kernel(const half_t *__restrict__ x, int m_rows,
                                                           const uint16_t *__restrict__ packed,
                                                           const half_t *__restrict__ scale,
                                                           const half_t *__restrict__ bias,
                                                           const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                           int n_out, int k_in, int group_size) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_out) return;
  const int words = k_in >> 2, groups_per_row = k_in / group_size;
  float acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = 0.f;
  for (int wi = lane; wi < words; wi += 64) {
    const uint32_t w = packed[(int64_t)row * words + wi];
    const int g = (wi * 4) / group_size;
    const half_t s = scale[(int64_t)row * groups_per_row + g], b = bias[(int64_t)row * groups_per_row + g];
    float wv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const half_t code = (half_t)(float)((w >> (12 - 4 * j)) & 15u);
      const half_t prod = code * s;
      wv[j] = (float)(half_t)(prod + b);
    }
#pragma unroll
    for (int m = 0; m < 16; ++m)
      if (m < m_rows) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[m] += (float)x[(int64_t)m * k_in + wi * 4 + j] * wv[j];
      }
  }
#pragma unroll
  for (int m = 0; m < 16; ++m) {
    if (m < m_rows) {
      float v = acc[m];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
      if (lane == 0) {
        if (out_bias) v += (float)out_bias[row];
        y[(int64_t)m * n_out + row] = (half_t)v;
      }
    }
  }
}

}  // namespace

int launch_gemv(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, hipStream_t stream) {
  const int variant = option_gemv_variant();
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  const bool fast_ok = pow2 && group_size >= 32 && k_in % 128 == 0 && k_in > 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)packed % 16) == 0;
  if (fast_ok && variant != 1) {
    const int gs_shift = __builtin_ctzll((unsigned long long)group_size);
    const unsigned blocks = (unsigned)((n_out + 15) / 16);
    gemv_mfma_kernel<8><<<dim3(blocks), dim3(512), 0, stream>>>(
        reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const uint4_t *>(packed),
        reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
        reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, gs_shift);
    return check_launch("gemv_mfma_kernel");
  }
  const unsigned blocks = (unsigned)((n_out + 3) / 4);
  gemv_generic_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(
      reinterpret_cast<const half_t *>(x), (int)m_rows, packed, reinterpret_cast<const half_t *>(scale),
      reinterpret_cast<const half_t *>(bias), reinterpret_cast<const half_t *>(out_bias),
      reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, (int)group_size);
  return check_launch("gemv_generic_kernel");
}

// Any m_rows through the generic kernel, 16 batch rows per launch (fallback of the GEMM entry).
int launch_gemv_generic_rows(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                             const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                             int64_t k_in, int64_t group_size, hipStream_t stream) {
  const unsigned blocks = (unsigned)((n_out + 3) / 4);
  for (int64_t m0 = 0; m0 < m_rows; m0 += 16) {
    const int m = (int)(m_rows - m0 < 16 ? m_rows - m0 : 16);
    gemv_generic_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(
        reinterpret_cast<const half_t *>(x) + m0 * k_in, m, packed, reinterpret_cast<const half_t *>(scale),
        reinterpret_cast<const half_t *>(bias), reinterpret_cast<const half_t *>(out_bias),
        reinterpret_cast<half_t *>(y) + m0 * n_out, (int)n_out, (int)k_in, (int)group_size);
  }
  return check_launch("gemv_generic_kernel");
}

}  // namespace gq
