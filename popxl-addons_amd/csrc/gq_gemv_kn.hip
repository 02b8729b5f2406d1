// Fused int4 dequant + GEMV for weights grouped along the OUTPUT features -- the layout of LinearGQ
// with dim = -1 or 1, the constructor default of the reference
// (popxl_addons/layers/linear_gq.py:26, 59-62, 99-101) -- on a derived copy of the weight that is
// made once at load time, for decode batches (1 <= m_rows <= 16) on gfx950.
//
//   W[k][n] = code[k][n] * scale[k][g] + bias[k][g],  g = n / 64
//   y[m][n] = sum_k x[m][k] W[k][n]
//           = sum_k (x[m][k] scale[k][g]) code[k][n]  +  sum_k x[m][k] bias[k][g]
//
// In the reference layout a packed word holds 8 consecutive outputs of ONE input feature, so no lane
// can hold a run of the contraction index.  The algebra above moves the scale from the weight to the
// activation: per group g of 64 outputs there is an activation vector xs_g[m][k] = x[m][k] scale[k][g],
// the codes go to the MFMA raw, and the bias term is a dot product per (group, batch row).  What is
// left is to have the codes of an output contiguous along k: the KN STREAMING LAYOUT, written by
// gq_gemv_kn_prepack_f16 -- the same 0.5625 bytes per weight, every load 1 KiB contiguous:
//
//   unit (g, c) = 64 outputs x 512 input features = 18432 bytes, units ordered g-major
//     [0, 16384)       four row blocks j of 16 outputs (n = 64 g + 16 j + r), 4 KiB each: load s (1 KiB),
//                      lane (r, kc) = 16 kc + r, 32-bit word w holds the codes of output n at input features
//                      512 c + 128 s + 32 kc + 8 w + e, e = 0..7, code e in nibble (3,7,2,6,1,5,0,4)[e]:
//                      the order in which the 5-instruction expansion (raw_codes) hands them to the MFMA
//     [16384, 17408)   scale[512 c + i][g], i = 0..511 (binary16)
//     [17408, 18432)   bias[512 c + i][g]
//
// v_mfma_f32_16x16x32_f16: A = raw codes of 16 outputs (64 + code or 1024 + code, exact), B = xs of up to
// 16 batch rows.  The offsets come out through per-lane sums: sum_k off_k xs[m][k] is taken from the
// very values that went into the MFMA (the rounded binary16 products), so it cancels exactly.
#include <algorithm>

#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {

constexpr int kKnUnitBytes = 18432;
constexpr int kKnWaves = 8;

// 8 codes of a word of the kn streaming layout as fp16, in the order of their input features:
// (64 + c, 64 + c, 1024 + c, 1024 + c) twice.  5 VALU instructions: the masks and magic numbers come
// in vector registers that the compiler cannot see through, which makes it select v_and_or_b32.
// (Plain C, not inline assembly: a VALU write to a register that an MFMA in flight still reads or is
// going to write needs wait states, and the compiler's hazard recogniser does not look into assembly
// -- with the results wrong now and then, whenever the register allocator re-used such a register.)
__device__ __forceinline__ half8_t kn_raw_codes(uint32_t w, uint32_t mask_lo, uint32_t mask_hi, uint32_t magic_lo,
                                                uint32_t magic_hi) {
  const uint32_t hi = w >> 8;
  uint4_t v;
  v.x = (hi & mask_hi) | magic_hi;  // nibbles 3, 7: features 0, 1
  v.y = (hi & mask_lo) | magic_lo;  // nibbles 2, 6: features 2, 3
  v.z = (w & mask_hi) | magic_hi;   // nibbles 1, 5: features 4, 5
  v.w = (w & mask_lo) | magic_lo;   // nibbles 0, 4: features 6, 7
  return __builtin_bit_cast(half8_t, v);
}

// Sums of N values per lane over the 64 lanes of a wave: each exchange halves the values a lane
// keeps (the lane with the exchanged bit clear keeps the lower half), then the lanes that hold the
// same value add up.  Afterwards lane l holds the sum of value l / (64 / N) in v[0].
template <int N, int WIDTH = 32>
__device__ __forceinline__ void wave_sums(float (&v)[N], int lane) {
  if constexpr (N > 1) {
    const bool upper = (lane & WIDTH) != 0;
    float kept[N / 2];
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
      const float send = upper ? v[i] : v[i + N / 2];
      const float keep = upper ? v[i + N / 2] : v[i];
      kept[i] = keep + __shfl_xor(send, WIDTH, 64);
    }
    wave_sums<N / 2, WIDTH / 2>(kept, lane);
    v[0] = kept[0];
  } else {
#pragma unroll
    for (int width = WIDTH; width > 0; width >>= 1) v[0] += __shfl_xor(v[0], width, 64);
  }
}

constexpr int knp_region_bytes(int r, int xm) { return (xm > r ? xm : r) * 1024; }
constexpr int knp_lds_bytes(int r, int xm) { return kKnWaves * knp_region_bytes(r, xm) + kKnWaves * 16 * 4; }

// One launch = one GEMV.  A workgroup of 8 waves owns R of the four row blocks of a group of 64
// outputs; its waves take the units of that group in turn (chunks of 512 input features) and their
// partial sums meet in LDS.  Per chunk a wave
//   * issues every load: R x 4 KiB of codes (16 bytes per lane and load), 1 KiB each of the group's
//     scales and biases (lane l: features 8 l .. 8 l + 7 of the chunk), and the same 8 features of x
//     for each of up to XM batch rows;
//   * multiplies x by the scales (packed binary16, one rounding), leaves the products in its LDS
//     stage (row m, 16-byte piece l at l ^ m: the sixteen rows that the lanes of a slice read are
//     spread over the banks) and adds to its per-lane sums  sum x bias - sum off xs;
//   * runs 16 R MFMAs: B operand of step (s, w) = piece 16 s + 4 kc + w of batch row (lane % 16).
// XM: 1, 4, 8 or 16 >= m_rows.
template <int R, int XM>
__global__ __launch_bounds__(kKnWaves * 64) void gemv_knp_kernel(const half_t *__restrict__ x, int m_rows,
                                                                const char *__restrict__ blob,
                                                                const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                                int n_out, int k_in, int act, int ldx) {
  constexpr int kRegion = knp_region_bytes(R, XM);
  constexpr int kPerGroup = 4 / R;  // workgroups that share a group of 64 outputs
  extern __shared__ __attribute__((aligned(16))) char knp_lds[];
  char(*const region)[kRegion] = reinterpret_cast<char(*)[kRegion]>(knp_lds);
  float(*const corr)[16] = reinterpret_cast<float(*)[16]>(knp_lds + kKnWaves * kRegion);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int n_chunks = k_in >> 9;

  // Workgroups go to the eight XCDs (each with an L2 of its own) in turn: the workgroups that share
  // a group's scales and biases get the same XCD.
  int wg = blockIdx.x;
  if (kPerGroup > 1) {
    const int span = 8 * kPerGroup, full = (int)gridDim.x / span * span;
    if (wg < full) {
      const int base = wg / span * span, t = wg - base;  // t = 8 * slot + xcd
      wg = base + (t & 7) * kPerGroup + (t >> 3);
    }
  }
  const int group = wg / kPerGroup, j0 = (wg % kPerGroup) * R;
  const char *const gbase = blob + (int64_t)group * n_chunks * kKnUnitBytes + lane * 16;

  uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x00F000F0u, kMagicLo = 0x64006400u, kMagicHi = 0x54005400u;
  asm volatile("" : "+v"(kMaskLo), "+v"(kMaskHi), "+v"(kMagicLo), "+v"(kMagicHi));
  const half2_t kNeg64 = {(half_t)-64.f, (half_t)-64.f}, kNeg1024 = {(half_t)-1024.f, (half_t)-1024.f};

  float4_t acc[R];
#pragma unroll
  for (int i = 0; i < R; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
  float cbias[XM], coff[XM];  // this lane's share of  sum_k x bias  and of  - sum_k off xs  per batch row
#pragma unroll
  for (int m = 0; m < XM; ++m) cbias[m] = coff[m] = 0.f;

  char *const stage = region[wave];
  const int x_row = r < m_rows ? r : 0;  // (columns past the batch are never stored: they may hold any row)
  // (batch rows past m_rows: the last row again -- no branches in the loop; their products are never read)
  const char *const x_lane = reinterpret_cast<const char *>(x) + lane * 16;

  struct Chunk {  // what a wave loads of one chunk
    uint4_t sv, bv, xq[XM], wq[4][R];
  };
  // What the scaled activations need first, then the codes in the order of their use: loads land in
  // the order issued.
  auto issue = [&](Chunk &k, int c) {
    const char *const u = gbase + (int64_t)c * kKnUnitBytes;
    k.sv = *reinterpret_cast<const uint4_t *>(u + 16384);
    k.bv = *reinterpret_cast<const uint4_t *>(u + 17408);
#pragma unroll
    for (int m = 0; m < XM; ++m)
      k.xq[m] = *reinterpret_cast<const uint4_t *>(x_lane + ((int64_t)min(m, m_rows - 1) * ldx + c * 512) * 2);  // (rows of x: ldx elements apart)
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int i = 0; i < R; ++i)  // (read once, whole cache lines: marked so, 3 - 7 % faster on every shape and batch)
        k.wq[s][i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(u + (j0 + i) * 4096 + s * 1024));
  };
  // The empty assembly statements pin the order: every load in front of the first of them is issued
  // before it (left to itself the compiler moves loads down to their first use, between the MFMAs,
  // or an instruction that needs the first load up between the loads: either way a memory latency
  // is waited out with most of the chunk not yet requested), and a loaded value is only touched
  // behind its own statement, i.e. when the loads in front of it have landed.
  auto work = [&](Chunk &k) {
    asm volatile("" : "+v"(k.sv), "+v"(k.bv) : : "memory");
    // ---- x times scale into the stage; the sums that take out the offsets and bring in the bias
    // (two sums per batch row and dot products of all rows in turn: no long chains of dependent instructions)
#pragma unroll
    for (int m = 0; m < XM; ++m) asm volatile("" : "+v"(k.xq[m]));
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int m = 0; m < XM; ++m) {
        const half2_t xv = as_half2(k.xq[m][t]);
        const half2_t p = xv * as_half2(k.sv[t]);  // (one rounding: the value the MFMA multiplies)
        k.xq[m][t] = __builtin_bit_cast(uint32_t, p);
        cbias[m] = __builtin_amdgcn_fdot2(xv, as_half2(k.bv[t]), cbias[m], false);
        coff[m] = __builtin_amdgcn_fdot2(p, (t & 1) ? kNeg1024 : kNeg64, coff[m], false);
      }
    }
#pragma unroll
    for (int m = 0; m < XM; ++m) *reinterpret_cast<uint4_t *>(stage + m * 1024 + ((lane ^ m) & 63) * 16) = k.xq[m];
    // ---- expand and multiply
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int i = 0; i < R; ++i) asm volatile("" : "+v"(k.wq[s][i]));
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const half8_t b = *reinterpret_cast<const half8_t *>(stage + x_row * 1024 + ((s * 16 + kc * 4 + w) ^ x_row) * 16);
#pragma unroll
        for (int i = 0; i < R; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kn_raw_codes(k.wq[s][i][w], kMaskLo, kMaskHi, kMagicLo, kMagicHi), b,
                                                          acc[i], 0, 0, 0);
        // (four row blocks and many batch rows: the expanded codes of later steps would not fit the registers)
        if (R * XM >= 32) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // (Requesting a wave's next chunk before it works on the current one -- two chunks' worth of
  // registers -- was measured and is slower: 16384 -> 4096 at one batch row 10.0 against 9.7 us, at eight
  // rows, where the registers no longer suffice, 17.6 against 14.7 us.  The other waves of the
  // compute unit keep the memory system busy while one of them computes.)
  for (int c = wave; c < n_chunks; c += kKnWaves) {
    Chunk a;
    issue(a, c);
    work(a);
  }
  float cacc[XM];
#pragma unroll
  for (int m = 0; m < XM; ++m) cacc[m] = cbias[m] + coff[m];
  // ---- the wave's sums: the per-lane corrections over its 64 lanes, then everything into LDS
  wave_sums<XM>(cacc, lane);
  if (lane < 16) corr[wave][lane] = 0.f;
  if ((lane & (64 / XM - 1)) == 0) corr[wave][lane / (64 / XM)] = cacc[0];  // (same wave: the LDS stores stay in order)
#pragma unroll
  for (int i = 0; i < R; ++i) *reinterpret_cast<float4_t *>(region[wave] + (i * 64 + lane) * 16) = acc[i];
  __syncthreads();
  // lane holds D[n = 4 * kc + e][m = r] of row block i
  for (int t = threadIdx.x; t < R * 64; t += kKnWaves * 64) {
    const int i = t >> 6, l = t & 63;
    const int m = l & 15;
    float4_t sum = *reinterpret_cast<const float4_t *>(region[0] + (i * 64 + l) * 16);
    float extra = corr[0][m];
#pragma unroll
    for (int w = 1; w < kKnWaves; ++w) {
      sum += *reinterpret_cast<const float4_t *>(region[w] + (i * 64 + l) * 16);
      extra += corr[w][m];
    }
    if (m < m_rows) {
      const int n0 = (group * 4 + j0 + i) * 16 + 4 * (l >> 4);
      half4_t out;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = sum[e] + extra;
        if (out_bias) v += (float)out_bias[n0 + e];
        out[e] = (half_t)apply_activation(v, act);
      }
      *reinterpret_cast<half4_t *>(y + (int64_t)m * n_out + n0) = out;  // (n_out % 64 == 0: 8-byte aligned)
    }
  }
}

// The kn streaming layout from the three variables of the layer: one thread per 16 bytes of the blob.
__global__ __launch_bounds__(256) void kn_prepack_kernel(const uint16_t *__restrict__ packed, const uint16_t *__restrict__ scale,
                                                         const uint16_t *__restrict__ bias, uint4_t *__restrict__ blob,
                                                         int n_out, int k_in, int64_t pieces) {
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= pieces) return;
  constexpr int kPieces = kKnUnitBytes / 16;  // 1152
  const int64_t unit = p / kPieces;
  const int q = (int)(p % kPieces), chunks = k_in >> 9;
  const int group = (int)(unit / chunks), c = (int)(unit % chunks);
  const int n_groups = n_out >> 6;
  uint4_t v;
  if (q < 1024) {
    const int j = q >> 8, s = (q >> 6) & 3, lane = q & 63;
    const int n = 64 * group + 16 * j + (lane & 15);
    const int shift = 12 - 4 * (n & 3);
    const uint16_t *src = packed + (n >> 2);
    const int64_t row_words = n_out >> 2;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int k0 = 512 * c + 128 * s + 32 * (lane >> 4) + 8 * w;
      uint32_t word = 0;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t code = (src[(int64_t)(k0 + e) * row_words] >> shift) & 15u;
        const int nibble = (e & 1) * 4 + 3 - (e >> 1);  // (3, 7, 2, 6, 1, 5, 0, 4)[e]
        word |= code << (4 * nibble);
      }
      v[w] = word;
    }
  } else {
    const uint16_t *src = q < 1088 ? scale : bias;
    const int i0 = ((q - 1024) & 63) * 8;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t lo = src[(int64_t)(512 * c + i0 + 2 * w) * n_groups + group];
      const uint32_t hi = src[(int64_t)(512 * c + i0 + 2 * w + 1) * n_groups + group];
      v[w] = lo | (hi << 16);
    }
  }
  blob[p] = v;
}

}  // namespace

bool gemv_kn_prepack_shape_ok(int64_t n_out, int64_t k_in, int64_t group_size) {
  return group_size == 64 && n_out > 0 && n_out % 64 == 0 && k_in > 0 && k_in % 512 == 0 && n_out <= (1 << 22) && k_in <= (1 << 24);
}

int64_t gemv_kn_prepacked_bytes(int64_t n_out, int64_t k_in) { return (n_out / 64) * (k_in / 512) * (int64_t)kKnUnitBytes; }

int launch_gemv_kn_prepack(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob, int64_t n_out,
                           int64_t k_in, hipStream_t stream) {
  const int64_t pieces = gemv_kn_prepacked_bytes(n_out, k_in) / 16;
  const int64_t blocks = (pieces + 255) / 256;
  if (blocks > 0x7fffffff) return fail(GQ_ERR_UNSUPPORTED, "gq_gemv_kn_prepack_f16: weight too large");
  kn_prepack_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(packed, scale, bias, reinterpret_cast<uint4_t *>(blob),
                                                                     (int)n_out, (int)k_in, pieces);
  return check_launch("kn_prepack_kernel");
}

// One GEMV on a weight in the kn streaming layout (m_rows <= 16; the caller has checked the shape).  ldx: elements
// from a row of x to the next (0: k_in; a multiple of 8).
int launch_gemv_knp(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                    int64_t k_in, int act, hipStream_t stream, int64_t ldx) {
  const int64_t groups = n_out / 64;
  // Row blocks per wave (1, 2 or 4: they share the scaled activations): the choice that moves the
  // fewest bytes per busy compute unit -- the codes once, scales, biases and x once per workgroup
  // (out of L2: counted half), divided by the share of the compute units' turns the workgroups fill.
  int r = 1;
  double best = 0;
  for (int cand = 4; cand >= 1; cand >>= 1) {
    const int64_t wgs = groups * (4 / cand);
    const double fill = (double)wgs / (double)((wgs + 255) / 256 * 256);
    const double bytes = (double)n_out * k_in * 0.5 + 0.5 * (double)wgs * k_in * (4.0 + 2.0 * m_rows);
    if (best == 0 || bytes / fill < best) best = bytes / fill, r = cand;
  }
  if (m_rows > 8 && r == 4) r = 2;  // (four row blocks and sixteen batch rows do not fit the registers)
  // Two to four batch rows with four row blocks take more than 128 vector registers, so one workgroup per
  // compute unit instead of two: on wide weights (256 workgroups or more) two row blocks, two workgroups
  // per compute unit measure faster (28672x4096 at batch 4: 15.9 against 17.4 us), on narrower ones not.
  if (m_rows > 1 && m_rows <= 4 && r == 4 && groups >= 256) r = 2;
  const unsigned blocks = (unsigned)(groups * (4 / r));
#define GQ_KNP_LAUNCH(R, XM)                                                                                    \
  do {                                                                                                        \
    constexpr int lds_bytes = knp_lds_bytes(R, XM);                                                           \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                    \
    if (lds_bytes > 64 * 1024) { /* beyond the default limit of a launch */                                   \
      constexpr int kMaxDevices = 64;                                                                         \
      static bool configured[kMaxDevices] = {false};                                                          \
      int dev = 0;                                                                                            \
      if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return GQ_ERR_NO_DEVICE;         \
      if (!configured[dev]) {                                                                                 \
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_knp_kernel<R, XM>),      \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);      \
        if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));            \
        configured[dev] = true;                                                                               \
      }                                                                                                       \
    }                                                                                                         \
    gemv_knp_kernel<R, XM><<<dim3(blocks), dim3(kKnWaves * 64), lds_bytes, stream>>>(                         \
        reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const char *>(blob),               \
        reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, act,  \
        (int)(ldx ? ldx : k_in));                                                                             \
  } while (0)
#define GQ_KNP_BY_R(XM)                            \
  do {                                             \
    if (r == 4) GQ_KNP_LAUNCH(4, XM);              \
    else if (r == 2) GQ_KNP_LAUNCH(2, XM);         \
    else GQ_KNP_LAUNCH(1, XM);                     \
  } while (0)
#define GQ_KNP_BY_R2(XM)                           \
  do {                                             \
    if (r == 2) GQ_KNP_LAUNCH(2, XM);              \
    else GQ_KNP_LAUNCH(1, XM);                     \
  } while (0)
  if (m_rows == 1) GQ_KNP_BY_R(1);
  else if (m_rows <= 4) GQ_KNP_BY_R(4);
  else if (m_rows <= 8) GQ_KNP_BY_R(8);
  else GQ_KNP_BY_R2(16);
#undef GQ_KNP_BY_R2
#undef GQ_KNP_BY_R
#undef GQ_KNP_LAUNCH
  return check_launch("gemv_knp_kernel");
}

}  // namespace gq
