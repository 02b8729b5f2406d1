// Fused int4 dequant + GEMV for one or two batch rows, weights grouped along the INPUT features
// (LinearGQ.build with dim=0, popxl_addons/layers/linear_gq.py:99-109), group 64, k_in % 512 == 0:
// scale and bias are applied to GROUP SUMS, not to weights.
//
//   y[m][n] = sum_g scale[n][g] ( sum_{k in g} (off_k + c[n][k]) x[m][k]  -  sum_{k in g} off_k x[m][k] )
//           + sum_g bias[n][g]    sum_{k in g} x[m][k]
//
// The codes go to the MFMA raw -- the nibble or-ed into the mantissa of 64.0 or 1024.0 (exact: 64 + c
// or 1024 + c), five VALU instructions per eight weights instead of thirteen -- as the B operand of
// v_mfma_f32_16x16x32_f16; the A operand holds x with its sixteen rows used as (group, batch row)
// combinations: row i = 2 g + m is x[m] on the 64 input features of group g of the chunk and zero
// elsewhere.  One accumulator per chunk of 512 features (8 groups x 2 batch rows) thus separates the
// groups, and lane (n, kc) -- weight row n, accumulator rows 4 kc + e -- finds in its four registers
// the sums of ITS weight row for groups 2 kc, 2 kc + 1 and both batch rows: the groups whose scales
// and biases are one dword of the row's.  The two sums of x per (group, batch row) are taken once
// per chunk (v_dot2_f32_f16, fp32) and shared by the row blocks of the wave.
//
// Work decomposition as in gq_gemv.hip: a workgroup of 8 waves owns R row blocks of 16 weight rows,
// its waves take chunks of 512 input features in turn, and their partial sums meet in LDS.  The
// weight comes as the three variables or as their streaming-layout copy (BLOB; gq_gemv_stream.hip:
// every load of codes 1 KiB contiguous and read once).
#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {

constexpr int kSumsWaves = 8;
constexpr int kSumsItemBytes = 4608;    // streaming layout: 4 KiB of codes, 16 x 16 B of scales, of biases
constexpr int kSumsRegionBytes = 2560;  // per wave: 2 KiB of x (two batch rows of a chunk), 128 B of group sums, spare
constexpr int kSumsLdsBytes = kSumsWaves * kSumsRegionBytes + 1024;  // + 1 KiB of zeros for the A rows without data

// XM: 1 or 2 >= m_rows.
template <int R, int XM, bool BLOB>
__global__ __launch_bounds__(kSumsWaves * 64) void gemv_sums_kernel(const half_t *__restrict__ x, int m_rows,
                                                                   const uint4_t *__restrict__ packed,
                                                                   const half_t *__restrict__ scale,
                                                                   const half_t *__restrict__ bias,
                                                                   const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                                   int n_out, int k_in, int act, int ldx) {
  extern __shared__ __attribute__((aligned(16))) char sums_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int n_chunks = k_in >> 9;
  char *const stage = sums_lds + wave * kSumsRegionBytes;                      // x of the chunk: row m at m KiB
  float *const sums = reinterpret_cast<float *>(stage + 2048);                // [group 0..7][batch row 0..1][sum x, sum off x]
  char *const zeros = sums_lds + kSumsWaves * kSumsRegionBytes;
  for (int i = threadIdx.x; i < 256; i += kSumsWaves * 64) reinterpret_cast<uint32_t *>(zeros)[i] = 0u;
  __syncthreads();

  // ---- where this lane's loads start
  const uint4_t *wrow[R];
  const uint32_t *srow[R], *brow[R];  // the dword with the scales (biases) of groups 2 kc, 2 kc + 1 of chunk 0
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if constexpr (BLOB) {
      const int rb = min((int)blockIdx.x * R + i, ((n_out + 15) >> 4) - 1);  // (the copy pads the last row block)
      const char *const items = reinterpret_cast<const char *>(packed) + (int64_t)rb * n_chunks * kSumsItemBytes;
      wrow[i] = reinterpret_cast<const uint4_t *>(items) + lane;
      srow[i] = reinterpret_cast<const uint32_t *>(items + 4096 + r * 16) + kc;
      brow[i] = reinterpret_cast<const uint32_t *>(items + 4352 + r * 16) + kc;
    } else {
      const int row = min(((int)blockIdx.x * R + i) * 16 + r, n_out - 1);
      wrow[i] = packed + (int64_t)row * (k_in >> 5) + kc;
      srow[i] = reinterpret_cast<const uint32_t *>(scale + (int64_t)row * (k_in >> 6)) + kc;
      brow[i] = reinterpret_cast<const uint32_t *>(bias + (int64_t)row * (k_in >> 6)) + kc;
    }
  }
  // ---- the A operand: this lane supplies row i = r (group r / 2 of the chunk, batch row r % 2) on the eight
  // features 32 kc + 8 s .. of slot j; it has data in the one slot whose group that is, zeros elsewhere
  const int a_m = r & 1, a_group = r >> 1;
  const bool a_live = a_m < m_rows && (a_group & 1) == (kc >> 1);
  const int a_slot = a_group >> 1;
  const char *a_piece[4];  // by step s, without the slot's 256 bytes: piece 16 j + 4 kc + s of row a_m lies at piece ^ a_m
#pragma unroll
  for (int s = 0; s < 4; ++s) a_piece[s] = stage + a_m * 1024 + ((kc * 4 + s) ^ a_m) * 16;

  uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x00F000F0u, kMagicLo = 0x64006400u, kMagicHi = 0x54005400u;
  asm volatile("" : "+v"(kMaskLo), "+v"(kMaskHi), "+v"(kMagicLo), "+v"(kMagicHi));
  const half2_t kOnes = {(half_t)1.f, (half_t)1.f}, kOffsets = {(half_t)64.f, (half_t)1024.f};

  float4_t tot[R];
#pragma unroll
  for (int i = 0; i < R; ++i) tot[i] = float4_t{0.f, 0.f, 0.f, 0.f};

  const char *const x_lane = reinterpret_cast<const char *>(x) + lane * 16;
  for (int c = wave; c < n_chunks; c += kSumsWaves) {
    // ---- every load of the chunk first: x (lane l: features 8 l .. 8 l + 7 of each batch row), the scale and
    // bias dwords, then the codes in the order of their use
    uint4_t xq[XM], wq[R][4];
    uint32_t sdw[R], bdw[R];
#pragma unroll
    for (int m = 0; m < XM; ++m)
      xq[m] = *reinterpret_cast<const uint4_t *>(x_lane + ((int64_t)min(m, m_rows - 1) * ldx + c * 512) * 2);  // (rows of x: ldx elements apart)
#pragma unroll
    for (int i = 0; i < R; ++i) {
      sdw[i] = *(srow[i] + (BLOB ? c * (kSumsItemBytes / 4) : c * 4));
      bdw[i] = *(brow[i] + (BLOB ? c * (kSumsItemBytes / 4) : c * 4));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < R; ++i)
        wq[i][j] = BLOB ? __builtin_nontemporal_load(wrow[i] + c * (kSumsItemBytes / 16) + j * 64) : *(wrow[i] + (c * 4 + j) * 4);
    // (the empty assembly statements pin the order: all loads are issued before anything waits for one)
#pragma unroll
    for (int m = 0; m < XM; ++m) asm volatile("" : "+v"(xq[m]) : : "memory");
#pragma unroll
    for (int i = 0; i < R; ++i) asm volatile("" : "+v"(sdw[i]), "+v"(bdw[i]));
    // ---- x into the stage in the order of the codes; the group's sums of x and of off x (8 lanes per group)
#pragma unroll
    for (int m = 0; m < XM; ++m) {
      float sx = 0.f, sw = 0.f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        sx = __builtin_amdgcn_fdot2(as_half2(xq[m][t]), kOnes, sx, false);
        sw = __builtin_amdgcn_fdot2(as_half2(xq[m][t]), kOffsets, sw, false);  // (even features: 64, odd: 1024)
      }
#pragma unroll
      for (int width = 1; width < 8; width <<= 1) {
        sx += __shfl_xor(sx, width, 64);
        sw += __shfl_xor(sw, width, 64);
      }
      if ((lane & 7) == 0) *reinterpret_cast<float2 *>(sums + ((lane >> 3) * 2 + m) * 2) = float2{sx, sw};
      *reinterpret_cast<half8_t *>(stage + m * 1024 + ((lane ^ m) & 63) * 16) = permute_x(xq[m]);
    }
    if (XM == 1) {  // (the second batch row does not exist: its sums are never used, but must be finite)
      if ((lane & 7) == 0) *reinterpret_cast<float2 *>(sums + ((lane >> 3) * 2 + 1) * 2) = float2{0.f, 0.f};
    }
    // ---- expand and multiply: one accumulator per row block for the whole chunk
    float4_t acc[R];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int i = 0; i < R; ++i) asm volatile("" : "+v"(wq[i][j]));
      const bool here = a_live && a_slot == j;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const half8_t a = *reinterpret_cast<const half8_t *>((here ? a_piece[s] : zeros) + j * 256);
#pragma unroll
        for (int i = 0; i < R; ++i) {
          const half8_t b = sums_raw_codes(wq[i][j][s], kMaskLo, kMaskHi, kMagicLo, kMagicHi);
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, (j == 0 && s == 0) ? float4_t{0.f, 0.f, 0.f, 0.f} : acc[i], 0, 0, 0);
        }
      }
    }
    // ---- group sums to results: register e is accumulator row 4 kc + e = (group 2 kc + e / 2, batch row e % 2)
    const float4_t g0 = *reinterpret_cast<const float4_t *>(sums + kc * 8);      // group 2 kc: (sx, sw) of rows 0, 1
    const float4_t g1 = *reinterpret_cast<const float4_t *>(sums + kc * 8 + 4);  // group 2 kc + 1
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const half2_t s2 = as_half2(sdw[i]), b2 = as_half2(bdw[i]);
      const float s_lo = (float)s2[0], s_hi = (float)s2[1], b_lo = (float)b2[0], b_hi = (float)b2[1];
      tot[i][0] += s_lo * (acc[i][0] - g0[1]) + b_lo * g0[0];
      tot[i][1] += s_lo * (acc[i][1] - g0[3]) + b_lo * g0[2];
      tot[i][2] += s_hi * (acc[i][2] - g1[1]) + b_hi * g1[0];
      tot[i][3] += s_hi * (acc[i][3] - g1[3]) + b_hi * g1[2];
    }
  }
  // ---- the wave's sums: registers e and e + 2 are the same batch row; the four lanes kc of a weight row add up
  float2 part[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    float p0 = tot[i][0] + tot[i][2], p1 = tot[i][1] + tot[i][3];
    p0 += __shfl_xor(p0, 16, 64);
    p1 += __shfl_xor(p1, 16, 64);
    p0 += __shfl_xor(p0, 32, 64);
    p1 += __shfl_xor(p1, 32, 64);
    part[i] = float2{p0, p1};
  }
  __syncthreads();  // (every wave has left its chunk loop: the stages may be overwritten)
  float2 *const meet = reinterpret_cast<float2 *>(sums_lds);  // [wave][row block][weight row]
  if (kc == 0) {
#pragma unroll
    for (int i = 0; i < R; ++i) meet[(wave * R + i) * 16 + r] = part[i];
  }
  __syncthreads();
  for (int t = threadIdx.x; t < R * 16; t += kSumsWaves * 64) {
    float2 sum = meet[t];
#pragma unroll
    for (int w = 1; w < kSumsWaves; ++w) {
      const float2 v = meet[w * R * 16 + t];
      sum.x += v.x;
      sum.y += v.y;
    }
    const int n = ((int)blockIdx.x * R + (t >> 4)) * 16 + (t & 15);
    if (n < n_out) {
      const float ob = out_bias ? (float)out_bias[n] : 0.f;
      y[n] = (half_t)apply_activation(sum.x + ob, act);
      if (m_rows > 1) y[(int64_t)n_out + n] = (half_t)apply_activation(sum.y + ob, act);
    }
  }
}

}  // namespace

// One or two batch rows on group 64, k_in % 512 == 0, everything 16-byte aligned (the caller has checked);
// `blob`: NULL (the three variables are read) or the weight's streaming-layout copy.
int launch_gemv_sums(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                     const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in, int act,
                     hipStream_t stream, int64_t ldx) {
  const int64_t row_blocks = (n_out + 15) / 16;
  // Row blocks per wave (1, 2 or 4; they share the x operands): the fewest bytes per busy compute unit -- the weights
  // once, x once per workgroup (out of L2: counted half), divided by the share of the compute units' turns that the
  // workgroups fill.  With one or two row blocks a wave takes at most 116 registers and two workgroups share a compute
  // unit (512 places a turn), with four 178 and one (256 places, and 8 % more time for the same bytes: 16384 x 4096 at
  // one row 8.9 us against 8.2 us with two row blocks, 28672 x 4096 15.7 against 13.8 us).
  int r = 1;
  double best = 0;
  for (int cand = 4; cand >= 1; cand >>= 1) {
    const int64_t wgs = (row_blocks + cand - 1) / cand, places = cand == 4 ? 256 : 512;
    const double fill = wgs <= places ? (wgs < 256 ? (double)wgs / 256.0 : 1.0)
                                      : (double)wgs / (double)((wgs + places - 1) / places * places);
    const double bytes = (double)n_out * k_in * 0.5625 + 0.5 * (double)wgs * m_rows * k_in * 2.0;
    const double cost = bytes / fill * (cand == 4 ? 1.08 : 1.0);
    if (best == 0 || cost < best) best = cost, r = cand;
  }
  const unsigned blocks = (unsigned)((row_blocks + r - 1) / r);
  const uint4_t *const weight = reinterpret_cast<const uint4_t *>(blob ? blob : packed);
#define GQ_SUMS_LAUNCH(R, XM, BLOB)                                                                                   \
  gemv_sums_kernel<R, XM, BLOB><<<dim3(blocks), dim3(kSumsWaves * 64), kSumsLdsBytes, stream>>>(                      \
      reinterpret_cast<const half_t *>(x), (int)m_rows, weight, reinterpret_cast<const half_t *>(scale),              \
      reinterpret_cast<const half_t *>(bias), reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), \
      (int)n_out, (int)k_in, act, (int)(ldx ? ldx : k_in))
#define GQ_SUMS_BY_R(XM, BLOB)                   \
  do {                                           \
    if (r == 4) GQ_SUMS_LAUNCH(4, XM, BLOB);     \
    else if (r == 2) GQ_SUMS_LAUNCH(2, XM, BLOB); \
    else GQ_SUMS_LAUNCH(1, XM, BLOB);            \
  } while (0)
  if (blob && m_rows == 1) GQ_SUMS_BY_R(1, true);
  else if (blob) GQ_SUMS_BY_R(2, true);
  else if (m_rows == 1) GQ_SUMS_BY_R(1, false);
  else GQ_SUMS_BY_R(2, false);
#undef GQ_SUMS_BY_R
#undef GQ_SUMS_LAUNCH
  return check_launch("gemv_sums_kernel");
}

}  // namespace gq
