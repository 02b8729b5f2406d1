// Device-side 4-bit group-quantization compress (fp16 or fp32 input) for gfx950.
//
// Produces the same packed / scale / bias bits as group_quantize_compress_numpy on a float16
// array (popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:178-196):
//   hi = max(group), lo = min(group)                       (:186-187)
//   scale = f16(f16(hi - lo) / 15), bias = lo              (:189-190)
//   code  = rint_half_even(f16(f16(x - lo) / scale))       (:192)
//   word  = c0 << 12 | c1 << 8 | c2 << 4 | c3               (:193-195)
// Every fp16 operation is rounded on its own: sums/differences are native fp16 ops, quotients
// are correctly rounded fp32 divisions rounded again to fp16 (24 >= 2*11+2 bits makes the double
// rounding exact), or products with a correctly rounded reciprocal where that is proved equal.
// Compiled with -ffp-contract=off.  HBM-bound: 2 B read, 0.5 + 4/gs B written per element.
#include "gq_common.h"

namespace gq {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ bool nonfinite_bits(uint32_t h) { return (h & 0x7c00u) == 0x7c00u; }

// f16(diff / scale) from the reciprocal of the scale, shared by the group: ONE fp32 product, rounded
// again to fp16.  Why that is enough: the reciprocal is the correctly rounded one (an IEEE division,
// once per group), so the product lies within 1.5 fp32 ulps of the true quotient (half an ulp of the
// reciprocal, scaled by a quotient below 2, and half an ulp of the product), while a quotient of two
// 11-bit significands D/S in [1, 2) is at least 1/(S 2^11) > 2^-22 -- two fp32 ulps -- away from
// every fp16 rounding boundary M/2^11, M odd (|D 2^11 - M S| is a nonzero integer).  No boundary
// can lie between the product and the quotient, so rounding the product rounds the quotient.  (Where
// the quotient is subnormal in fp16 the boundaries are closer; every such quotient gives code 0.)
__device__ __forceinline__ half_t divide(half_t diff, float recip) {
  // the product as a mixed-precision fma that reads diff as fp16 and writes fp16
  return (half_t)__builtin_fmaf((float)diff, recip, 0.f);
}

__device__ __forceinline__ uint32_t quantize(half_t v, half_t lo, float recip) {
  const half_t diff = v - lo;
  const half_t quot = divide(diff, recip);
  int c = (int)__builtin_rintf((float)quot);
  c = c < 0 ? 0 : (c > 15 ? 15 : c);  // no effect wherever the reference is well defined
  return (uint32_t)c;
}

// LANES lanes share one group; each lane holds 8 (or 16) consecutive elements (one or two 16-byte
// loads) and writes the uint16 words made from them as one 32-bit (64-bit) store.
// The work is done two elements per instruction wherever a packed fp16 form exists (the roundings
// are those of the scalar forms).  What bounds the kernel is neither that arithmetic (a third fewer
// instructions changed nothing) nor the loads in flight (more of them per thread made it slower):
// without its stores of packed words the same kernel runs at 93 % of the HBM peak, with them at 69 %.
typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));

// packed minimum / maximum as single instructions (the generic builtins first quieten their
// operands with two more)
__device__ __forceinline__ half2_t pk_min(half2_t a, half2_t b) {
  half2_t r;
  asm("v_pk_min_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ half2_t pk_max(half2_t a, half2_t b) {
  half2_t r;
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// V: 16-byte vectors per lane (1: 8 elements, group_size = 8 LANES; 2: 16 elements, group_size =
// 16 LANES -- half the lanes per group: one shuffle round less, and the scale, reciprocal and
// store of the group's statistics amortised over twice the elements)
template <int LANES, int V>
__device__ __forceinline__ void compress_item(const uint4_t (&q)[V], int64_t item, bool live, uint32_t *__restrict__ packed,
                                              half_t *__restrict__ scale, half_t *__restrict__ bias,
                                              int32_t *__restrict__ flag) {
  half2_t h[4 * V];
  half2_t poison = {(half_t)0.f, (half_t)0.f};  // sum of 0 * x: NaN once an Inf or NaN has been seen
  const half2_t zero_pair = {(half_t)0.f, (half_t)0.f};
#pragma unroll
  for (int v = 0; v < V; ++v) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t w = q[v][d];  // (a bit cast straight from a vector element reads element 0)
      h[4 * v + d] = __builtin_bit_cast(half2_t, w);
      poison = __builtin_elementwise_fma(h[4 * v + d], zero_pair, poison);
    }
  }
  half2_t mx = pk_max(pk_max(h[0], h[1]), pk_max(h[2], h[3]));
  half2_t mn = pk_min(pk_min(h[0], h[1]), pk_min(h[2], h[3]));
  if (V == 2) {
    mx = pk_max(mx, pk_max(pk_max(h[4], h[5]), pk_max(h[6], h[7])));
    mn = pk_min(mn, pk_min(pk_min(h[4], h[5]), pk_min(h[6], h[7])));
  }
  // (min, max) of the group travel through the shuffles as one register; the whole wave executes
  // them, items of one group are LANES consecutive lanes
  half2_t p = {mn[0] < mn[1] ? mn[0] : mn[1], mx[0] > mx[1] ? mx[0] : mx[1]};
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) {
    const half2_t o = __builtin_bit_cast(half2_t, __shfl_xor(__builtin_bit_cast(int, p), off, 64));
    const half2_t lo2 = pk_min(p, o), hi2 = pk_max(p, o);
    p = half2_t{lo2[0], hi2[1]};
  }
  const half_t lo = p[0], hi = p[1];
  const half_t range = hi - lo;
  const half_t sc = (half_t)((float)range / 15.0f);
  // scale 0 (a constant group, or a range too small for fp16): every code is 0; dividing by 1 gives
  // that without a branch, because every difference is then below 2^-20
  const float sc32 = (float)sc == 0.f ? 1.0f : (float)sc;
  const float recip = 1.0f / sc32;  // (correctly rounded: the compiler's IEEE division)
  const half2_t lo_pair = {lo, lo}, ceiling = {(half_t)1039.0f, (half_t)1039.0f}, magic = {(half_t)1024.0f, (half_t)1024.0f};
  // Each step for all pairs before the next step for any: an instruction that reads what the one
  // before it wrote with a half-word selection costs a wait state on this hardware, and the
  // compiler's own order (one pair at a time) put one in front of three instructions in five.
  half2_t diff[4 * V], quot[4 * V];
#pragma unroll
  for (int d = 0; d < 4 * V; ++d) diff[d] = h[d] - lo_pair;
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 0; d < 4 * V; ++d) quot[d][0] = divide(diff[d][0], recip);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 0; d < 4 * V; ++d) quot[d][1] = divide(diff[d][1], recip);
  __builtin_amdgcn_sched_barrier(0);
  // quot + 1024 rounds to an integer, ties to even (the ulp of fp16 at 1024 is 1): that is
  // 1024 + rint(quot) = 0x6400 + code as a bit pattern.  Codes above 15 are clipped (no effect
  // wherever the reference is well defined; a NaN becomes 15).
#pragma unroll
  for (int d = 0; d < 4 * V; ++d) quot[d] = quot[d] + magic;
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 0; d < 4 * V; ++d) quot[d] = pk_min(quot[d], ceiling);
  // A uint16 word is 4096 c0 + 256 c1 + 16 c2 + c3: two dot products of 16-bit pairs, the second
  // starting from the first; the 0x6400 of the four patterns is taken out where the sum starts
  // (modulo 2^32, and the result is below 2^16).
  const ushort2_t hi_weights = {4096, 256}, lo_weights = {16, 1};
  const uint32_t start = 0u - 0x6400u * (4096u + 256u + 16u + 1u);
  uint32_t word[V];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    uint32_t w16[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t part = __builtin_amdgcn_udot2(__builtin_bit_cast(ushort2_t, quot[4 * v + 2 * i + 1]), lo_weights, start, false);
      w16[i] = __builtin_amdgcn_udot2(__builtin_bit_cast(ushort2_t, quot[4 * v + 2 * i]), hi_weights, part, false);
    }
    word[v] = __builtin_amdgcn_perm(w16[1], w16[0], 0x05040100u);  // the low halves of both, side by side
  }
  if (live) {
    // (streaming stores: nothing reads the result soon; 0.4 us of 31 on 4096 x 16384)
    if (V == 1) {
      __builtin_nontemporal_store(word[0], packed + item);
    } else {
      __builtin_nontemporal_store(uint2_t{word[0], word[V - 1]}, reinterpret_cast<uint2_t *>(packed + item * 2));
    }
    if (flag && (poison[0] != poison[0] || poison[1] != poison[1])) *flag = 1;
  }
  // (Collecting the statistics of four groups in one lane for 8-byte stores was measured: the
  // shuffles cost what the wider stores save.)
  if (LANES == 1) {
    if (live) {
      scale[item] = sc;
      bias[item] = lo;
    }
  } else if (live && (item & (LANES - 1)) < 2) {
    // the first lane of a group stores its scale, the second its bias: one store instruction for
    // both arrays (0.15 us of 31 against one lane storing both)
    half_t *const dst = (item & 1) ? bias : scale;
    dst[item / LANES] = (item & 1) ? lo : sc;
  }
}

template <int LANES, int V>
__global__ __launch_bounds__(kThreads) void compress_kernel(const uint4_t *__restrict__ t, uint32_t *__restrict__ packed,
                                                            half_t *__restrict__ scale, half_t *__restrict__ bias,
                                                            int32_t *__restrict__ flag, int64_t n_items) {
  // One item per thread and as many workgroups as that takes.  (Measured on 4096 x 16384: several
  // items per thread with all their loads issued first, 34 to 38 us, and a fixed grid of 1024 to
  // 8192 workgroups that loads an item ahead, 34 to 37 us, against 31 us.)
  const int64_t item = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const bool live = item < n_items;
  uint4_t q[V];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    q[v] = uint4_t{0u, 0u, 0u, 0u};
    if (live) q[v] = __builtin_nontemporal_load(t + item * V + v);
  }
  compress_item<LANES, V>(q, item, live, packed, scale, bias, flag);
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
  const float recip = 1.0f / sc32;  // (correctly rounded: the compiler's IEEE division)
  for (int i = 0; i < group_size / 4; ++i) {
    uint32_t w = 0;
    for (int j = 0; j < 4; ++j) w = (w << 4) | quantize(src[4 * i + j], lo, recip);
    packed[g * (group_size / 4) + i] = (uint16_t)w;
  }
  if (bad && flag) *flag = 1;
}

// ---------------------------------------------------------------------------------------
// fp32 input (what LinearGQ.torch_mapping feeds the packer: nn.Linear weights, linear_gq.py:130).
// The reference promotes to fp32 there (group_quantize_decompress.py:186-192): max / min are taken
// in fp32 and cast to fp16, the scale is fp16 arithmetic, and (x - lo) / scale is an fp32
// subtraction and a correctly rounded fp32 division.  HBM-bound: 4 B read per element.
// LANES lanes share a group, 8 elements (two 16-byte loads) per lane; LANES == 0: one lane per
// group, any group_size % 4 == 0.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t quantize_f32(float v, float lo, float sc) {
  const float quot = (v - lo) / sc;  // both rounded to fp32 (contraction is off; the division is IEEE)
  int c = (int)__builtin_rintf(quot);
  c = c < 0 ? 0 : (c > 15 ? 15 : c);  // no effect wherever the reference is well defined
  return (uint32_t)c;
}

template <int LANES>
__global__ __launch_bounds__(kThreads) void compress_f32_kernel(const float4_t *__restrict__ t, uint32_t *__restrict__ packed,
                                                                half_t *__restrict__ scale, half_t *__restrict__ bias,
                                                                int32_t *__restrict__ flag, int64_t n_items) {
  const int64_t item = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const bool live = item < n_items;
  float v[8];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    float4_t f = {0.f, 0.f, 0.f, 0.f};
    if (live) f = __builtin_nontemporal_load(t + item * 2 + q);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[4 * q + e] = f[e];
  }
  float mx = v[0], mn = v[0];
  bool bad = false;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    bad |= (__builtin_bit_cast(uint32_t, v[e]) & 0x7f800000u) == 0x7f800000u;
    mx = v[e] > mx ? v[e] : mx;
    mn = v[e] < mn ? v[e] : mn;
  }
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) {
    const float omx = __shfl_xor(mx, off, 64), omn = __shfl_xor(mn, off, 64);
    mx = omx > mx ? omx : mx;
    mn = omn < mn ? omn : mn;
  }
  const half_t hi = (half_t)mx, lo = (half_t)mn;
  const half_t range = hi - lo;
  const half_t sc = (half_t)((float)range / 15.0f);
  const float lo32 = (float)lo;
  // scale 0 (constant group): every code is 0; an infinite divisor gives that without a branch
  const float sc32 = (float)sc == 0.f ? __builtin_inff() : (float)sc;
  uint32_t w[2];
#pragma unroll
  for (int q = 0; q < 2; ++q)
    w[q] = (quantize_f32(v[4 * q], lo32, sc32) << 12) | (quantize_f32(v[4 * q + 1], lo32, sc32) << 8) |
           (quantize_f32(v[4 * q + 2], lo32, sc32) << 4) | quantize_f32(v[4 * q + 3], lo32, sc32);
  if (live) {
    packed[item] = w[0] | (w[1] << 16);
    if ((item & (LANES - 1)) == 0) {
      scale[item / LANES] = sc;
      bias[item / LANES] = lo;
    }
    if (flag && bad) *flag = 1;
  }
}

__global__ __launch_bounds__(kThreads) void compress_f32_generic_kernel(const float *__restrict__ t,
                                                                        uint16_t *__restrict__ packed,
                                                                        half_t *__restrict__ scale,
                                                                        half_t *__restrict__ bias, int32_t *__restrict__ flag,
                                                                        int64_t n_groups_total, int group_size) {
  const int64_t g = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (g >= n_groups_total) return;
  const float *src = t + g * group_size;
  float mx = src[0], mn = src[0];
  bool bad = false;
  for (int e = 0; e < group_size; ++e) {
    const float v = src[e];
    bad |= (__builtin_bit_cast(uint32_t, v) & 0x7f800000u) == 0x7f800000u;
    mx = v > mx ? v : mx;
    mn = v < mn ? v : mn;
  }
  const half_t hi = (half_t)mx, lo = (half_t)mn;
  const half_t range = hi - lo;
  const half_t sc = (half_t)((float)range / 15.0f);
  scale[g] = sc;
  bias[g] = lo;
  const float lo32 = (float)lo;
  const float sc32 = (float)sc == 0.f ? __builtin_inff() : (float)sc;
  for (int i = 0; i < group_size / 4; ++i) {
    uint32_t w = 0;
    for (int j = 0; j < 4; ++j) w = (w << 4) | quantize_f32(src[4 * i + j], lo32, sc32);
    packed[g * (group_size / 4) + i] = (uint16_t)w;
  }
  if (bad && flag) *flag = 1;
}

}  // namespace

int launch_compress(const uint16_t *t, uint16_t *packed, uint16_t *scale, uint16_t *bias, int32_t *flag,
                    int64_t rows, int64_t n_groups, int64_t group_size, hipStream_t stream) {
  const int64_t groups_total = rows * n_groups;
  // 16 elements per lane where the group allows it, else 8
  const int per_lane = group_size % 16 == 0 && ((uintptr_t)packed % 8) == 0 ? 16 : 8;
  const int lanes = (int)(group_size / per_lane);
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
#define GQ_COMPRESS(L)                                                                                  \
  do {                                                                                                  \
    if (per_lane == 16) compress_kernel<L, 2><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); \
    else compress_kernel<L, 1><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items);              \
  } while (0)
    switch (lanes) {
      case 1: GQ_COMPRESS(1); break;
      case 2: GQ_COMPRESS(2); break;
      case 4: GQ_COMPRESS(4); break;
      case 8: GQ_COMPRESS(8); break;
      case 16: GQ_COMPRESS(16); break;
      case 32: GQ_COMPRESS(32); break;
      default: GQ_COMPRESS(64); break;
    }
#undef GQ_COMPRESS
    return check_launch("compress_kernel");
  }
  const int64_t blocks = (groups_total + kThreads - 1) / kThreads;
  if (blocks >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "gq_compress_f16: tensor too large");
  compress_generic_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
      reinterpret_cast<const half_t *>(t), packed, reinterpret_cast<half_t *>(scale),
      reinterpret_cast<half_t *>(bias), flag, groups_total, (int)group_size);
  return check_launch("compress_generic_kernel");
}

int launch_compress_f32(const float *t, uint16_t *packed, uint16_t *scale, uint16_t *bias, int32_t *flag, int64_t rows,
                        int64_t n_groups, int64_t group_size, hipStream_t stream) {
  const int64_t groups_total = rows * n_groups;
  const int lanes = (int)(group_size / 8);
  const bool fast = group_size % 8 == 0 && (lanes & (lanes - 1)) == 0 && lanes <= 64 && ((uintptr_t)t % 16) == 0 &&
                    ((uintptr_t)packed % 4) == 0;
  half_t *s = reinterpret_cast<half_t *>(scale), *b = reinterpret_cast<half_t *>(bias);
  if (fast) {
    const int64_t n_items = groups_total * lanes;
    const int64_t blocks = (n_items + kThreads - 1) / kThreads;
    if (blocks >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "gq_compress_f32: tensor too large");
    const dim3 grid((unsigned)blocks), block(kThreads);
    const float4_t *src = reinterpret_cast<const float4_t *>(t);
    uint32_t *dst = reinterpret_cast<uint32_t *>(packed);
    switch (lanes) {
      case 1: compress_f32_kernel<1><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 2: compress_f32_kernel<2><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 4: compress_f32_kernel<4><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 8: compress_f32_kernel<8><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 16: compress_f32_kernel<16><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      case 32: compress_f32_kernel<32><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
      default: compress_f32_kernel<64><<<grid, block, 0, stream>>>(src, dst, s, b, flag, n_items); break;
    }
    return check_launch("compress_f32_kernel");
  }
  const int64_t blocks = (groups_total + kThreads - 1) / kThreads;
  if (blocks >= (int64_t)1 << 31) return fail(GQ_ERR_UNSUPPORTED, "gq_compress_f32: tensor too large");
  compress_f32_generic_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(t, packed, s, b, flag, groups_total,
                                                                                     (int)group_size);
  return check_launch("compress_f32_generic_kernel");
}

}  // namespace gq
