// Fused int4 dequant + GEMV (decode-sized batches, 1 <= m_rows <= 16) for gfx950.
//
// y[m][n] = sum_k x[m][k] * W[n][k] (+ out_bias[n]) with W[n][k] = code * scale[n][k/gs] + bias[n][k/gs]
// -- LinearGQ.build with dim=0 (popxl_addons/layers/linear_gq.py:99-109) without ever
// writing the fp16 weight to memory.  HBM-bound on the packed weight: 0.5 + 4/gs bytes per
// weight element.
#include <algorithm>

#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {


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

// One chunk = 512 contraction indices = four 16-byte loads per lane and row block ("slots" of
// 128 indices: lane (r, kc) takes bytes [64 * slot + 16 * kc, +16) of its row's chunk).
// R     row blocks of 16 rows handled by one wave with the same x fragments (x is loaded and
//       permuted once per chunk, then reused R times).
// GS    64 or 128: scale/bias of a chunk are fetched as one 16/8-byte load per row and the lane's
//       value is picked with a byte permute; 0: any power-of-two group >= 32, 2-byte loads.
// FULL  k_in is a multiple of 512 (no slot predication).
// XM    1, 4, 8 or 16 >= m_rows: the 1 KiB of x that a chunk needs of a batch row is fetched by ONE load
//       instruction of the whole wave, ahead of the weight loads, and handed to the row's four lanes
//       through LDS.  (Those four lanes fetching their sixteen 16-byte pieces themselves -- sixteen
//       load instructions per chunk with 4 m_rows lanes active -- cost 0.8 us of 5.9 at one batch row
//       and 1.9 us of 7.1 at eight on 4096 x 4096.)
constexpr int gemv_region_bytes(int r, int xm) { return (xm > r ? xm : r) * 1024; }

// BLOB  `packed` is the weight in the streaming layout of gq_gemv_prepack_f16 (scale and bias are not read;
//       GS == 64 and FULL): item (row block, chunk) = 4 KiB of codes as [slot][kc][r] 16-byte pieces -- each of
//       the four loads of a chunk is 1 KiB contiguous, read once -- then the rows' 16 bytes of scales, of biases.
constexpr int kStreamItemBytes = 4608;

template <int NWAVES, int R, int GS, bool FULL, int XM, bool BLOB = false>
__global__ __launch_bounds__(NWAVES * 64) void gemv_mfma_kernel(
    const half_t *__restrict__ x, int m_rows, const uint4_t *__restrict__ packed, const half_t *__restrict__ scale,
    const half_t *__restrict__ bias, const half_t *__restrict__ out_bias, half_t *__restrict__ y, int n_out, int k_in,
    int gs_shift, int act, int ldx) {
  // per wave: the x chunk of up to XM batch rows while the wave walks K, its partial sums at the end
  constexpr int kRegion = gemv_region_bytes(R, XM);
  extern __shared__ __attribute__((aligned(16))) char region_base[];
  char(*const region)[kRegion] = reinterpret_cast<char(*)[kRegion]>(region_base);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int n_slots = k_in >> 7;
  const int n_chunks = (n_slots + 3) >> 2;
  const int groups_per_row = k_in >> gs_shift;
  const uint4_t *wrow[R];
  const half_t *srow[R], *brow[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = min(((int)blockIdx.x * R + i) * 16 + r, n_out - 1);
    if constexpr (BLOB) {
      static_assert(GS == 64 && FULL, "the streaming layout has groups of 64 and whole chunks");
      const int rb = min((int)blockIdx.x * R + i, ((n_out + 15) >> 4) - 1);  // (the copy pads the last row block)
      const char *const items = reinterpret_cast<const char *>(packed) + (int64_t)rb * n_chunks * kStreamItemBytes;
      wrow[i] = reinterpret_cast<const uint4_t *>(items) + lane;
      srow[i] = reinterpret_cast<const half_t *>(items + 4096 + r * 16);
      brow[i] = reinterpret_cast<const half_t *>(items + 4352 + r * 16);
      continue;
    }
    wrow[i] = packed + (int64_t)row * (k_in >> 5) + kc;
    srow[i] = scale + (int64_t)row * groups_per_row;
    brow[i] = bias + (int64_t)row * groups_per_row;
  }
  // byte selector that broadcasts the low or the high half of a 32-bit word (GS == 64: the lane's
  // group within a slot is kc / 2)
  const uint32_t half_sel = (kc & 2) ? 0x07060706u : 0x05040504u;

  float4_t acc[R];
#pragma unroll
  for (int i = 0; i < R; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};

  // staged x: 16-byte piece p of batch row m lies at piece p ^ m of the row's KiB, so that the sixteen
  // rows read by the lanes of one slice are spread over the banks (measured on 4096 x 4096: no
  // bank-conflict cycles at one batch row, 2.5 per LDS instruction at eight -- 2 % of the waves' cycles)
  char *const stage = region[wave];
  const int x_row = r < m_rows ? r : 0;  // (columns past the batch are never stored: they may hold any row)
  for (int c = wave; c < n_chunks; c += NWAVES) {
    uint4_t xq[XM];
    {
#pragma unroll
      for (int m = 0; m < XM; ++m) {
        xq[m] = uint4_t{0u, 0u, 0u, 0u};
        if (m < m_rows && (FULL || c * 512 + lane * 8 < k_in))  // (k_in is a multiple of 128: a piece is whole or absent)
          xq[m] = *reinterpret_cast<const uint4_t *>(x + (int64_t)m * ldx + c * 512 + lane * 8);  // (rows of x: ldx elements apart)
      }
    }
    uint4_t wq[R][4];
    uint32_t s2[R][4], b2[R][4];  // (scale, scale) and (bias, bias) as packed fp16 pairs
    // ---- issue every load of the chunk
#pragma unroll
    for (int i = 0; i < R; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int slot = c * 4 + j;
        if (BLOB)
          wq[i][j] = __builtin_nontemporal_load(wrow[i] + c * (kStreamItemBytes / 16) + j * 64);
        else if (FULL || slot < n_slots)
          // (ordinary loads: marked read-once they were 1 - 8 % slower on every shape and batch but
          // 4096 x 4096, where it makes no difference: 12288 x 4096 at 8 rows 12.5 against 11.3 us --
          // a lane's 16 bytes are part of a line that the other slots' loads complete)
          wq[i][j] = *(wrow[i] + slot * 4);
        else
          wq[i][j] = uint4_t{0u, 0u, 0u, 0u};
      }
      if constexpr (GS == 64) {
        // A last chunk of fewer than four slots: the 16 bytes END with the row (the launcher sees to it
        // that there is a whole chunk in front), and the dword of slot j is found `back` places later.
        // The dwords that then stand for the absent slots belong to earlier groups of the row: finite
        // numbers, multiplied by codes and x that are zero.
        const int back = (!FULL && c == n_chunks - 1) ? 4 - (n_slots - c * 4) : 0;
        uint4_t sv = *reinterpret_cast<const uint4_t *>(srow[i] + (BLOB ? c * (kStreamItemBytes / 2) : c * 8 - back * 2));
        uint4_t bv = *reinterpret_cast<const uint4_t *>(brow[i] + (BLOB ? c * (kStreamItemBytes / 2) : c * 8 - back * 2));
        if (!FULL) {
          if (back & 1) sv = uint4_t{sv.y, sv.z, sv.w, sv.x}, bv = uint4_t{bv.y, bv.z, bv.w, bv.x};
          if (back & 2) sv = uint4_t{sv.z, sv.w, sv.x, sv.y}, bv = uint4_t{bv.z, bv.w, bv.x, bv.y};
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s2[i][j] = __builtin_amdgcn_perm(sv[j], sv[j], half_sel);
          b2[i][j] = __builtin_amdgcn_perm(bv[j], bv[j], half_sel);
        }
      } else if constexpr (GS == 128) {
        const uint2_t sv = *reinterpret_cast<const uint2_t *>(srow[i] + c * 4);
        const uint2_t bv = *reinterpret_cast<const uint2_t *>(brow[i] + c * 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t sel = (j & 1) ? 0x07060706u : 0x05040504u;
          s2[i][j] = __builtin_amdgcn_perm(sv[j >> 1], sv[j >> 1], sel);
          b2[i][j] = __builtin_amdgcn_perm(bv[j >> 1], bv[j >> 1], sel);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int slot = c * 4 + j;
          uint32_t sv = 0, bv = 0;
          if (FULL || slot < n_slots) {
            const int g = (slot * 128 + kc * 32) >> gs_shift;
            sv = __builtin_bit_cast(uint16_t, srow[i][g]);
            bv = __builtin_bit_cast(uint16_t, brow[i][g]);
          }
          s2[i][j] = sv | (sv << 16);
          b2[i][j] = bv | (bv << 16);
        }
      }
    }
    half8_t xp[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (j == 0 && s == 0) {
#pragma unroll
          for (int m = 0; m < XM; ++m)
            if (m < m_rows) *reinterpret_cast<uint4_t *>(stage + m * 1024 + ((lane ^ m) & 63) * 16) = xq[m];
        }
        const uint4_t q = *reinterpret_cast<const uint4_t *>(stage + x_row * 1024 + ((j * 16 + kc * 4 + s) ^ x_row) * 16);
        xp[j][s] = permute_x(q);
      }
    }
    // ---- expand and multiply
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const half8_t a = dequant_word(wq[i][j][s], as_half2(s2[i][j]), as_half2(b2[i][j]));
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, xp[j][s], acc[i], 0, 0, 0);
        }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) *reinterpret_cast<float4_t *>(region[wave] + (i * 64 + lane) * 16) = acc[i];
  __syncthreads();
  // lane holds D[n = 4 * kc + e][m = r] of row block i
  for (int t = threadIdx.x; t < R * 64; t += NWAVES * 64) {
    const int i = t >> 6, l = t & 63;
    float4_t sum = *reinterpret_cast<const float4_t *>(region[0] + (i * 64 + l) * 16);
#pragma unroll
    for (int w = 1; w < NWAVES; ++w) sum += *reinterpret_cast<const float4_t *>(region[w] + (i * 64 + l) * 16);
    const int m = l & 15;
    if (m < m_rows) {
      const int n0 = ((int)blockIdx.x * R + i) * 16 + 4 * (l >> 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = n0 + e;
        if (n < n_out) {
          float v = sum[e];
          if (out_bias) v += (float)out_bias[n];
          y[(int64_t)m * n_out + n] = (half_t)apply_activation(v, act);
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
                                                           int n_out, int k_in, int group_size, int act, int ldx) {
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
        for (int j = 0; j < 4; ++j) acc[m] += (float)x[(int64_t)m * ldx + wi * 4 + j] * wv[j];
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
        y[(int64_t)m * n_out + row] = (half_t)apply_activation(v, act);
      }
    }
  }
}

}  // namespace

// `blob`: NULL, or the same weight in the streaming layout of gq_gemv_prepack_f16 (then group_size is 64 and
// k_in % 512 == 0); with x and the blob 16-byte aligned the kernels read it and packed, scale, bias may be NULL.
int launch_gemv(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, int act, hipStream_t stream, const void *blob, int64_t ldx) {
  if (ldx == 0) ldx = k_in;  // rows of x: ldx elements apart (a multiple of 8 where x must be 16-byte aligned)
  const bool x_aligned = ((uintptr_t)x % 16) == 0 && ldx % 8 == 0;  // every row of x on a 16-byte boundary
  if (blob && (group_size != 64 || k_in % 512 != 0 || k_in <= 0 || !x_aligned || ((uintptr_t)blob % 16) != 0)) {
    if (!packed || !scale || !bias)
      return fail(GQ_ERR_UNSUPPORTED, "a weight in the streaming layout needs group_size 64, k_in %% 512 == 0 and 16-byte aligned x");
    blob = nullptr;  // (the variables serve)
  }
  // One or two batch rows on group 64 and whole chunks: the kernel that applies scale and bias to group sums
  // (five vector instructions per eight weights instead of thirteen; on the large weights of the next rule it
  // measured 14.1 / 11.1 / 11.9 us at one row on 28672 / 20480 / 24576 x 4096 against 15.4 / 12.6 / 14.2 us).
  if (m_rows <= 2 && group_size == 64 && k_in > 0 && k_in % 512 == 0 && x_aligned &&
      (blob || (((uintptr_t)packed % 16) == 0 && ((uintptr_t)scale % 4) == 0 && ((uintptr_t)bias % 4) == 0)))
    return launch_gemv_sums(x, m_rows, packed, scale, bias, blob, out_bias, y, n_out, k_in, act, stream, ldx);
  // Three to eight rows on a weight whose rows alone fill the compute units (k_in <= 4096): the kernel whose waves
  // share the rows' x
  if (group_size == 64 && x_aligned &&
      (blob || (((uintptr_t)packed % 16) == 0 && ((uintptr_t)scale % 16) == 0 && ((uintptr_t)bias % 16) == 0)) &&
      gemv_rows_fits(m_rows, n_out, k_in))
    return launch_gemv_rows(x, m_rows, packed, scale, bias, blob, out_bias, y, n_out, k_in, act, stream, ldx);
  // Weights of 72 Mi elements or more with rows shorter than 8192 features go through the persistent
  // kernel at batches up to 4, as a sequence of one: its pipelined rings beat the one-shot kernel below
  // there (measured at one row: 20480x4096 15.1 -> 13.2 us, 24576x4096 19.7 -> 14.6 us, 32768x4096
  // 22.6 -> 17.9 us; 16384x4096 is a tie at one row, 11.6 us, and the one-shot kernel wins at four rows,
  // 11.6 against 12.9 us).  With longer rows a wave of the one-shot kernel has several chunks to
  // overlap and wins (4096x16384 at one row: 12.0 against 14.5 us; 8192x8192: 13.3 against 14.1).
  const bool large = n_out * k_in >= ((int64_t)72 << 20) && k_in < 8192;
  if (large && m_rows <= 4 && ldx == k_in) {  // (a sequence entry's x is contiguous)
    const int rc = blob ? launch_gemv_streamed(x, m_rows, static_cast<const uint16_t *>(blob), nullptr, nullptr, out_bias, y, n_out,
                                               k_in, group_size, act, stream)
                        : launch_gemv_streamed(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, act, stream);
    if (rc != GQ_ERR_UNSUPPORTED) return rc;
  }
  if (blob) {  // (shape and alignment were checked above: the streaming-layout instantiations of the one-shot kernel)
    packed = static_cast<const uint16_t *>(blob);
    scale = bias = nullptr;
  }
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  const bool fast_ok = pow2 && group_size >= 32 && k_in % 128 == 0 && k_in > 0 && x_aligned &&
                       ((uintptr_t)packed % 16) == 0;
  if (fast_ok) {
    const int gs_shift = __builtin_ctzll((unsigned long long)group_size);
    const int64_t row_blocks = (n_out + 15) / 16;
    const bool full = k_in % 512 == 0;
    // rows per wave: reuse the permuted x fragments as often as the row count allows while still
    // filling 256 compute units
    // Row blocks per wave (1, 2 or 4; they re-use the x fragments): the choice that moves the fewest
    // bytes per busy compute unit -- the weights once, x once per workgroup (out of L2: counted half),
    // divided by the share of the compute units' turns that the workgroups fill (192 workgroups
    // leave a quarter of the 256 compute units idle).  Measured on 12288 x 4096 at one row: 9.7 us with
    // one row block per wave (768 workgroups), 12.5 us with two (384), 11.2 us with four (192).
    int r = 1;
    double best = 0;
    for (int cand = 4; cand >= 1; cand >>= 1) {
      const int64_t wgs = (row_blocks + cand - 1) / cand;
      const double fill = (double)wgs / (double)((wgs + 255) / 256 * 256);
      const double bytes = (double)n_out * k_in * 0.5625 + 0.5 * (double)wgs * m_rows * k_in * 2.0;
      if (best == 0 || bytes / fill < best) best = bytes / fill, r = cand;
    }
    // the GS == 64 / 128 instantiations fetch a chunk's scales and biases as one 16 / 8-byte load per
    // row: that needs the arrays aligned accordingly; otherwise the 2-byte loads of GS == 0 serve
    const uintptr_t sb_align = (uintptr_t)scale | (uintptr_t)bias;
    // (group 64 with a partial last chunk, e.g. k_in = 11008: the rows of scale / bias are then only
    // 4-byte aligned, which the 16-byte loads take, and the last load reaches back into the chunk before)
    const int gs_mode = blob ? 64 : (group_size == 64 && (full || k_in > 512) && sb_align % 16 == 0)
                            ? 64
                            : ((group_size == 128 && full && sb_align % 8 == 0) ? 128 : 0);
    const unsigned blocks = (unsigned)((row_blocks + r - 1) / r);
#define GQ_GEMV_ARGS                                                                                      \
  reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const uint4_t *>(packed),            \
      reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),                    \
      reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, gs_shift, act, (int)ldx
#define GQ_GEMV_LAUNCH(NW, R, GS, FULL, XM, BLOB)                                                            \
  do {                                                                                                    \
    constexpr int lds_bytes = NW * gemv_region_bytes(R, XM);                                              \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                \
    if (lds_bytes > 64 * 1024) { /* beyond the default limit of a launch */                               \
      constexpr int kMaxDevices = 64;                                                                     \
      static bool configured[kMaxDevices] = {false};                                                      \
      int dev = 0;                                                                                        \
      if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return GQ_ERR_NO_DEVICE;     \
      if (!configured[dev]) {                                                                             \
        const hipError_t e = hipFuncSetAttribute(                                                         \
            reinterpret_cast<const void *>(gemv_mfma_kernel<NW, R, GS, FULL, XM, BLOB>),                       \
            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);                                       \
        if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));        \
        configured[dev] = true;                                                                           \
      }                                                                                                   \
    }                                                                                                     \
    gemv_mfma_kernel<NW, R, GS, FULL, XM, BLOB><<<dim3(blocks), dim3(NW * 64), lds_bytes, stream>>>(GQ_GEMV_ARGS); \
  } while (0)
#define GQ_GEMV_BY_R(NW, GS, FULL, XM, BLOB)                      \
  do {                                                            \
    if (r == 4) GQ_GEMV_LAUNCH(NW, 4, GS, FULL, XM, BLOB);        \
    else if (r == 2) GQ_GEMV_LAUNCH(NW, 2, GS, FULL, XM, BLOB);   \
    else GQ_GEMV_LAUNCH(NW, 1, GS, FULL, XM, BLOB);               \
  } while (0)
    // x through LDS, one load instruction per batch row and chunk (the rows of x are 16-byte aligned:
    // k_in % 128 == 0), on eight waves whatever the length of the rows (measured on 4096 x 16384:
    // 16 waves are no faster with x staged; without, eight rows took 20.1 us against 14.7 us)
#define GQ_GEMV_BY_M(GS, FULL, BLOB)                              \
  do {                                                            \
    if (m_rows == 1) GQ_GEMV_BY_R(8, GS, FULL, 1, BLOB);          \
    else if (m_rows <= 4) GQ_GEMV_BY_R(8, GS, FULL, 4, BLOB);     \
    else if (m_rows <= 8) GQ_GEMV_BY_R(8, GS, FULL, 8, BLOB);     \
    else GQ_GEMV_BY_R(8, GS, FULL, 16, BLOB);                     \
  } while (0)
    if (blob) GQ_GEMV_BY_M(64, true, true);
    else if (gs_mode == 64 && full) GQ_GEMV_BY_M(64, true, false);
    else if (gs_mode == 64) GQ_GEMV_BY_M(64, false, false);
    else if (gs_mode == 128) GQ_GEMV_BY_M(128, true, false);
    else if (full) GQ_GEMV_BY_M(0, true, false);
    else GQ_GEMV_BY_M(0, false, false);  // (a last chunk of 128, 256 or 384 features, e.g. k_in = 11008)
#undef GQ_GEMV_BY_M
#undef GQ_GEMV_BY_R
#undef GQ_GEMV_LAUNCH
#undef GQ_GEMV_ARGS
    return check_launch("gemv_mfma_kernel");
  }
  const unsigned blocks = (unsigned)((n_out + 3) / 4);
  gemv_generic_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(
      reinterpret_cast<const half_t *>(x), (int)m_rows, packed, reinterpret_cast<const half_t *>(scale),
      reinterpret_cast<const half_t *>(bias), reinterpret_cast<const half_t *>(out_bias),
      reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, (int)group_size, act, (int)ldx);
  return check_launch("gemv_generic_kernel");
}

// Passes of 16 rows against the GEMM kernel, from times measured on the three layer shapes of the 6B
// stack (us): a pass takes 4.7 + 0.124 per Mi weights (6.8 on 4096 x 4096, 13.0 on 16384 x 4096; a
// third more with rows of 8192 features or longer: 17.5 on 4096 x 16384); the GEMM kernel's 128 x 64
// tiles take 8 per 1024 input features and round of 256 tiles (31 / 34 / 112 on the same shapes,
// whatever the batch up to 128; its own estimate is asked).  Measured: 4096 x 4096 at 32 rows 13.3 against 31.8, 4096 x 16384 at 64
// rows 69.7 against 117.1, 16384 x 4096 at 32 rows 25.4 against 34.1 (and 38.0 against 35.2 at 48 rows).
bool launch_gemv_passes(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                        const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                        int64_t group_size, int act, bool gemm_may_split, hipStream_t stream, int *rc, const void *blob) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  const bool fast_ok = pow2 && group_size >= 32 && k_in % 128 == 0 && k_in > 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)packed % 16) == 0;
  if (!fast_ok || m_rows <= 16 || m_rows > 128) return false;
  const int64_t passes = (m_rows + 15) / 16;
  const double weights_mi = (double)n_out * (double)k_in / 1048576.0;
  const double t_pass = 4.7 + 0.124 * weights_mi * (k_in >= 8192 ? 1.35 : 1.0);
  // (the GEMM kernel: what its own choice of tile -- and, with a workspace, of workgroups per tile -- expects)
  const bool pipelined = (k_in / group_size) % 2 == 0 && k_in % 64 == 0;
  const double t_gemm = pipelined ? gemm_expected_us(m_rows, n_out, k_in, gemm_may_split) : 1e30;
  if ((double)passes * t_pass >= t_gemm) return false;
  for (int64_t m0 = 0; m0 < m_rows; m0 += 16) {
    const int64_t m = m_rows - m0 < 16 ? m_rows - m0 : 16;
    *rc = launch_gemv(x + m0 * k_in, m, packed, scale, bias, out_bias, y + m0 * n_out, n_out, k_in, group_size, act, stream, blob);
    if (*rc != GQ_OK) return true;
  }
  return true;
}

// Any m_rows through the generic kernel, 16 batch rows per launch (fallback of the GEMM entry).
int launch_gemv_generic_rows(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                             const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                             int64_t k_in, int64_t group_size, int act, hipStream_t stream) {
  const unsigned blocks = (unsigned)((n_out + 3) / 4);
  for (int64_t m0 = 0; m0 < m_rows; m0 += 16) {
    const int m = (int)(m_rows - m0 < 16 ? m_rows - m0 : 16);
    gemv_generic_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(
        reinterpret_cast<const half_t *>(x) + m0 * k_in, m, packed, reinterpret_cast<const half_t *>(scale),
        reinterpret_cast<const half_t *>(bias), reinterpret_cast<const half_t *>(out_bias),
        reinterpret_cast<half_t *>(y) + m0 * n_out, (int)n_out, (int)k_in, (int)group_size, act, (int)k_in);
  }
  return check_launch("gemv_generic_kernel");
}

}  // namespace gq
