// Device-side 4-bit group-quantization compress (fp16 input) for gfx950.
//
// Produces the same packed / scale / bias bits as group_quantize_compress_numpy on a float16
// array (popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:178-196):
//   hi = max(group), lo = min(group)                       (:186-187)
//   scale = f16(f16(hi - lo) / 15), bias = lo              (:189-190)
//   code  = rint_half_even(f16(f16(x - lo) / scale))       (:192)
//   word  = c0 << 12 | c1 << 8 | c2 << 4 | c3               (:193-195)
// Every fp16 operation is rounded on its own: sums/differences are native fp16 ops, quotients
// are correctly rounded fp32 divisions rounded again to fp16 (24 >= 2*11+2 bits makes the double
// rounding exact).  Compiled with -ffp-contract=off.  HBM-bound: 2 B read, 0.5 + 4/gs B written
// per element.
#include "gq_common.h"

namespace gq {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ bool nonfinite_bits(uint32_t h) { return (h & 0x7c00u) == 0x7c00u; }

// f16(diff / scale), correctly rounded, from a reciprocal shared by the group: one Newton step on
// the fp32 product.  Why that is enough: the residual e = diff - scale * t is exact (an fma of
// 11-bit by 24-bit operands whose result cancels down to a few bits), so t2 = t + e * r lies
// within one fp32 ulp of the true quotient, while a quotient of two 11-bit significands is at
// least 2^-22 (relative, in [1, 2)) away from every fp16 rounding boundary -- four fp32 ulps.  No
// boundary can lie between t2 and the quotient, so rounding t2 rounds the quotient.
__device__ __forceinline__ half_t divide(half_t diff, float scale_f32, float recip) {
  const float d = (float)diff;
  const float t = d * recip;
  const float e = __builtin_fmaf(-scale_f32, t, d);
  return (half_t)__builtin_fmaf(e, recip, t);
}

__device__ __forceinline__ uint32_t quantize(half_t v, half_t lo, float scale_f32, float recip) {
  const half_t diff = v - lo;
  const half_t quot = divide(diff, scale_f32, recip);
  int c = (int)__builtin_rintf((float)quot);
  c = c < 0 ? 0 : (c > 15 ? 15 : c);  // no effect wherever the reference is well defined
  return (uint32_t)c;
}

// LANES lanes share one group; each lane holds 8 consecutive elements (one 16-byte load) and
// writes the two uint16 words made from them as one 32-bit store.  group_size = 8 * LANES.
template <int LANES>
__global__ __launch_bounds__(kThreads) void compress_kernel(const uint4_t *__restrict__ t, uint32_t *__restrict__ packed,
                                                            half_t *__restrict__ scale, half_t *__restrict__ bias,
                                                            int32_t *__restrict__ flag, int64_t n_items) {
  const int64_t item = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const bool live = item < n_items;
  uint4_t q = {0u, 0u, 0u, 0u};
  if (live) q = __builtin_nontemporal_load(t + item);
  half_t v[8];
  bool bad = false;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const uint32_t w = q[d];
    bad |= nonfinite_bits(w) | nonfinite_bits(w >> 16);
    const half2_t h = __builtin_bit_cast(half2_t, w);
    v[2 * d] = h[0];
    v[2 * d + 1] = h[1];
  }
  half_t hi = v[0], lo = v[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) {
    hi = v[e] > hi ? v[e] : hi;
    lo = v[e] < lo ? v[e] : lo;
  }
  // the whole wave executes the shuffles; items of one group are LANES consecutive lanes
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) {
    const half_t ohi = (half_t)__shfl_xor((float)hi, off, 64), olo = (half_t)__shfl_xor((float)lo, off, 64);
    hi = ohi > hi ? ohi : hi;
    lo = olo < lo ? olo : lo;
  }
  const half_t range = hi - lo;
  const half_t sc = (half_t)((float)range / 15.0f);
  // scale 0 (a constant group, or a range too small for fp16): every code is 0; dividing by 1 gives
  // that without a branch, because every difference is then below 2^-20
  const float sc32 = (float)sc == 0.f ? 1.0f : (float)sc;
  const float recip = __builtin_amdgcn_rcpf(sc32);
  uint32_t c[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) c[e] = quantize(v[e], lo, sc32, recip);
  const uint32_t w0 = (c[0] << 12) | (c[1] << 8) | (c[2] << 4) | c[3];
  const uint32_t w1 = (c[4] << 12) | (c[5] << 8) | (c[6] << 4) | c[7];
  if (live) {
    packed[item] = w0 | (w1 << 16);
    if ((item & (LANES - 1)) == 0) {
      scale[item / LANES] = sc;
      bias[item / LANES] = lo;
    }
    if (bad && flag) *flag = 1;
  }
}

// Any group_size % 4 == 0: one lane per group.
__global__ __launch_bounds__(kThreads) void compress_generic_kernel(const half_t *__restrict__ t,
                                                                    uint16_t *__restrict__ packed,
                                                                    half_t *__restrict__ scale, half_t *__restrict__ bias,
                                                                    int32_t *__restrict__ flag, int64_t n_groups_total,
                                                                    int group_size) {
  const int64_t g = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (g >= n_groups_total) return;
  const half_t *src = t + g * group_size;
  half_t hi = src[0], lo = src[0];
  bool bad = false;
  for (int e = 0; e < group_size; ++e) {
    const half_t v = src[e];
    bad |= nonfinite_bits(__builtin_bit_cast(uint16_t, v));
    hi = v > hi ? v : hi;
    lo = v < lo ? v : lo;
  }
  const half_t range = hi - lo;
  const half_t sc = (half_t)((float)range / 15.0f);
  scale[g] = sc;
  bias[g] = lo;
  const float sc32 = (float)sc == 0.f ? 1.0f : (float)sc;
  const float recip = __builtin_amdgcn_rcpf(sc32);
  for (int i = 0; i < group_size / 4; ++i) {
    uint32_t w = 0;
    for (int j = 0; j < 4; ++j) w = (w << 4) | quantize(src[4 * i + j], lo, sc32, recip);
    packed[g * (group_size / 4) + i] = (uint16_t)w;
  }
  if (bad && flag) *flag = 1;
}

}  // namespace

int launch_compress(const uint16_t *t, uint16_t *packed, uint16_t *scale, uint16_t *bias, int32_t *flag,
                    int64_t rows, int64_t n_groups, int64_t group_size, hipStream_t stream) {
  const int64_t groups_total = rows * n_groups;
  const int lanes = (int)(group_size / 8);
  const bool fast = group_size % 8 == 0 && (lanes & (lanes - 1)) == 0 && lanes <= 64 && ((uintptr_t)t % 16) == 0 &&
                    ((uintptr_t)packed % 4) == 0;
  if (fast) {
    const int64_t n_items = groups_total * lanes;
    const int64_t blocks = (n_items + kThreads - 1) / kThreads;
    if (blocks >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "gq_compress_f16: tensor too large");
    const dim3 grid((unsigned)blocks), block(kThreads);
    const uint4_t *src = reinterpret_cast<const uint4_t *>(t);
    uint32_t *dst = reinterpret_cast<uint32_t *>(packed);
    half_t *s = reinterpret_cast<half_t *>(scale), *b = reinterpret_cast<half_t *>(bias);
    switch (lanes) {
      case 1: compress_kernel<1><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 2: compress_kernel<2><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 4: compress_kernel<4><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 8: compress_kernel<8><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 16: compress_kernel<16><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 32: compress_kernel<32><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      default: compress_kernel<64><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
    }
    return check_launch("compress_kernel");
  }
  const int64_t blocks = (groups_total + kThreads - 1) / kThreads;
  if (blocks >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "gq_compress_f16: tensor too large");
  compress_generic_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
      reinterpret_cast<const half_t *>(t), packed, reinterpret_cast<half_t *>(scale),
      reinterpret_cast<half_t *>(bias), flag, groups_total, (int)group_size);
  return check_launch("compress_generic_kernel");
}

}  // namespace gq
