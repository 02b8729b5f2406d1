// Fused int4 dequant + GEMV for three to eight batch rows, weights grouped along the INPUT features
// (LinearGQ.build with dim=0, popxl_addons/layers/linear_gq.py:99-109), group 64, k_in % 512 == 0:
// the waves of a workgroup share the batch rows' x.
//
// With several batch rows the work that belongs to x -- per chunk of 512 input features and batch row a load,
// a permutation into the order of the codes, two sums per group of 64 -- is as much as the work on a row
// block's codes.  A kernel whose waves divide K between them (gq_gemv.hip, gq_gemv_sums.hip) repeats it for
// every row block or two: measured on 28672 x 4096 at eight rows, 23.6 us of which 7.5 us were x.  Here a
// workgroup's eight waves own DIFFERENT row blocks over ALL of K (at most 8 chunks: k_in <= 4096): together
// they prepare the x of every chunk once, in LDS, meet at one barrier, and then each wave runs over the chunks
// on its own and stores its rows' results itself.  That pays where the groups of 8 row blocks alone fill the
// compute units (28672 x 4096: 224 workgroups; 14.4 against 16.8 us at four rows, 16.7 against 19.9 us at
// eight).  Dividing K over workgroups for weights with fewer or longer rows (fp32 partial sums through a
// workspace, the last workgroup to arrive adding them in a fixed order) was built and measured: the exchange
// costs what the shared x saves (16384 x 4096 at four rows 11.4 against 11.9 us, at eight 12.8 against 11.6;
// 4096 x 20480 16.2 against 14.9 and 18.0 against 15.3), so those stay with the other kernels.
//
// Arithmetic as in gq_gemv_sums.hip: the raw codes (64 + c or 1024 + c) are the B operand of
// v_mfma_f32_16x16x32_f16; the sixteen rows of the A operand are (group, batch row) combinations, 4 x 4 or
// 2 x 8, row i = MB ga + m being x[m] on the 64 features of group ga of the accumulator and zero
// elsewhere; a chunk takes MB / 2 accumulators (a slot of 128 features feeds the accumulator of its two
// groups: sixteen MFMAs per chunk and row block whatever MB); scale and bias are applied to the group sums:
//   y[m][n] = sum_g scale[n][g] ( sum_{k in g} (off_k + c[n][k]) x[m][k]  -  sum_{k in g} off_k x[m][k] )
//           + sum_g bias[n][g]    sum_{k in g} x[m][k]
// Lane (n, kc) holds in the four registers of accumulator a the sums of ONE group, 16 a / MB + 4 kc / MB of
// the chunk, for batch rows (4 kc) % MB + e, and picks that group's scale and bias out of the row's 16 bytes.
#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {

constexpr int kRowsWaves = 8;
constexpr int kRowsItemBytes = 4608;  // streaming layout: 4 KiB of codes, 16 x 16 B of scales, of biases
constexpr int kRowsMaxChunks = 8;     // chunks of K (their x sits in LDS together)
// per chunk: the batch rows' x (1 KiB each), then 8 bytes of sums per (group, batch row)
constexpr int rows_chunk_bytes(int xm) { return xm * 1024 + 512; }
constexpr int rows_lds_bytes(int xm, int chunks) { return chunks * rows_chunk_bytes(xm) + 1024; }  // + 1 KiB of zeros for the A rows without data

// XM: 4 or 8 >= m_rows.  R: row blocks per wave (1 in every launch: with two, 28672 x 4096 has 112 workgroups and
// took 19.2 against 14.8 us at four rows).  Grid: groups of 8 R row blocks; k_in <= 4096.
template <int R, int XM, bool BLOB>
__global__ __launch_bounds__(kRowsWaves * 64) void gemv_rows_kernel(const half_t *__restrict__ x, int m_rows,
                                                                   const uint4_t *__restrict__ packed,
                                                                   const half_t *__restrict__ scale,
                                                                   const half_t *__restrict__ bias,
                                                                   const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                                   int n_out, int k_in, int act, int ldx) {
  static_assert(XM == 4 || XM == 8, "batch rows of an accumulator");
  constexpr int MB = XM;      // batch rows of an accumulator (16 / MB groups)
  constexpr int NA = MB / 2;  // accumulators per chunk
  constexpr int SA = 4 / NA;  // slots of 128 features (two groups) per accumulator
  constexpr int kChunk = rows_chunk_bytes(XM);
  extern __shared__ __attribute__((aligned(16))) char rows_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int n_chunks = k_in >> 9;
  char *const zeros = rows_lds + n_chunks * kChunk;
  for (int i = threadIdx.x; i < 256; i += kRowsWaves * 64) reinterpret_cast<uint32_t *>(zeros)[i] = 0u;

  // ---- the x of all chunks: (chunk, batch row) pairs in turn over the waves.  Lane l holds features
  // 8 l .. 8 l + 7 of the row's chunk: into the stage in the order of the codes, and the group's sums of x
  // and of off x (8 lanes per group) beside it.
  {
    const half2_t kOnes = {(half_t)1.f, (half_t)1.f}, kOffsets = {(half_t)64.f, (half_t)1024.f};
    for (int p = wave; p < n_chunks * XM; p += kRowsWaves) {
      const int cl = p / XM, m = p % XM;
      const uint4_t xq = *reinterpret_cast<const uint4_t *>(reinterpret_cast<const char *>(x) + lane * 16 +
                                                            ((int64_t)min(m, m_rows - 1) * ldx + cl * 512) * 2);  // (rows of x: ldx elements apart)
      float sx = 0.f, sw = 0.f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        sx = __builtin_amdgcn_fdot2(as_half2(xq[t]), kOnes, sx, false);
        sw = __builtin_amdgcn_fdot2(as_half2(xq[t]), kOffsets, sw, false);  // (even features: 64, odd: 1024)
      }
#pragma unroll
      for (int width = 1; width < 8; width <<= 1) {
        sx += __shfl_xor(sx, width, 64);
        sw += __shfl_xor(sw, width, 64);
      }
      char *const stage = rows_lds + cl * kChunk;
      if ((lane & 7) == 0) *reinterpret_cast<float2 *>(stage + XM * 1024 + ((lane >> 3) * MB + m) * 8) = float2{sx, sw};
      *reinterpret_cast<half8_t *>(stage + m * 1024 + ((lane ^ m) & 63) * 16) = permute_x(xq);
    }
  }

  // ---- where this lane's loads start
  const uint4_t *wrow[R];
  const char *srow[R], *brow[R];  // the 16 bytes of scales (biases) of the row's groups of chunk 0
  constexpr int kChunkStride = BLOB ? kRowsItemBytes : 16;  // from a chunk's scales to the next chunk's
  const int rb0 = ((int)blockIdx.x * kRowsWaves + wave) * R;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if constexpr (BLOB) {
      const int rb = min(rb0 + i, ((n_out + 15) >> 4) - 1);  // (a wave without rows reads the last row block's)
      const char *const items = reinterpret_cast<const char *>(packed) + (int64_t)rb * n_chunks * kRowsItemBytes;
      wrow[i] = reinterpret_cast<const uint4_t *>(items) + lane;
      srow[i] = items + 4096 + r * 16;
      brow[i] = items + 4352 + r * 16;
    } else {
      const int row = min((rb0 + i) * 16 + r, n_out - 1);
      wrow[i] = packed + (int64_t)row * (k_in >> 5) + kc;
      srow[i] = reinterpret_cast<const char *>(scale + (int64_t)row * (k_in >> 6));
      brow[i] = reinterpret_cast<const char *>(bias + (int64_t)row * (k_in >> 6));
    }
  }
  // ---- the A operand: this lane supplies row i = r (group r / MB of its accumulator, batch row r % MB) on the
  // eight features 32 kc + 8 s .. of slot j; it has data in the one slot of each accumulator whose group that
  // is, zeros elsewhere
  const int a_m = r % MB, a_group = r / MB;
  const bool a_live = a_m < m_rows && (a_group & 1) == (kc >> 1);
  const int a_slot = a_group >> 1;  // within the accumulator's SA slots
  int a_piece[4];                   // by step s, without the slot's 256 bytes: piece 16 j + 4 kc + s of row a_m lies at piece ^ a_m
#pragma unroll
  for (int s = 0; s < 4; ++s) a_piece[s] = a_m * 1024 + ((kc * 4 + s) ^ a_m) * 16;
  // where this lane's group of accumulator a has its scale in the row's 16 bytes: half 4 a + kc (MB == 4) or
  // 2 a + kc / 2 (MB == 8) -- the dword's upper half for odd ones
  const uint32_t half_shift = (MB == 4 ? (kc & 1) : (kc >> 1)) * 16;
  const bool odd_dword = MB == 4 && (kc >> 1) != 0;

  uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x00F000F0u, kMagicLo = 0x64006400u, kMagicHi = 0x54005400u;
  asm volatile("" : "+v"(kMaskLo), "+v"(kMaskHi), "+v"(kMagicLo), "+v"(kMagicHi));

  float4_t tot[R];
#pragma unroll
  for (int i = 0; i < R; ++i) tot[i] = float4_t{0.f, 0.f, 0.f, 0.f};

  __syncthreads();  // the x of every chunk is in LDS: from here on a wave meets nobody

  for (int c = 0; c < n_chunks; ++c) {
    // ---- every load of the chunk first: the scales and biases, then the codes in the order of their use
    uint4_t wq[R][4], sqw[R], bqw[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      sqw[i] = *reinterpret_cast<const uint4_t *>(srow[i] + c * kChunkStride);
      bqw[i] = *reinterpret_cast<const uint4_t *>(brow[i] + c * kChunkStride);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < R; ++i)
        wq[i][j] = BLOB ? __builtin_nontemporal_load(wrow[i] + c * (kRowsItemBytes / 16) + j * 64) : *(wrow[i] + (c * 4 + j) * 4);
    // (the empty assembly statements pin the order: all loads are issued before anything waits for one)
#pragma unroll
    for (int i = 0; i < R; ++i) asm volatile("" : "+v"(sqw[i]), "+v"(bqw[i]) : : "memory");
    const char *const stage = rows_lds + c * kChunk;
    const float *const sums = reinterpret_cast<const float *>(stage + XM * 1024);
    // ---- expand and multiply: NA accumulators per row block for the whole chunk
    float4_t acc[R][NA];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int i = 0; i < R; ++i) asm volatile("" : "+v"(wq[i][j]));
      const bool here = a_live && a_slot == j % SA;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const half8_t a = *reinterpret_cast<const half8_t *>((here ? stage + a_piece[s] : zeros) + j * 256);
#pragma unroll
        for (int i = 0; i < R; ++i) {
          const half8_t b = sums_raw_codes(wq[i][j][s], kMaskLo, kMaskHi, kMagicLo, kMagicHi);
          acc[i][j / SA] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
              a, b, (j % SA == 0 && s == 0) ? float4_t{0.f, 0.f, 0.f, 0.f} : acc[i][j / SA], 0, 0, 0);
        }
      }
    }
    // ---- group sums to results: register e of accumulator a is its row 4 kc + e, entry 16 a + 4 kc + e of the sums
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      const float4_t g0 = *reinterpret_cast<const float4_t *>(sums + (a * 16 + kc * 4) * 2);      // (sx, sw) of rows 4 kc, 4 kc + 1
      const float4_t g1 = *reinterpret_cast<const float4_t *>(sums + (a * 16 + kc * 4) * 2 + 4);  // of rows 4 kc + 2, 4 kc + 3
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const uint32_t sd = MB == 4 ? (odd_dword ? sqw[i][2 * a + 1] : sqw[i][2 * a]) : sqw[i][a];
        const uint32_t bd = MB == 4 ? (odd_dword ? bqw[i][2 * a + 1] : bqw[i][2 * a]) : bqw[i][a];
        const float sc = (float)as_half2(sd >> half_shift)[0], bi = (float)as_half2(bd >> half_shift)[0];
        tot[i][0] += sc * (acc[i][a][0] - g0[1]) + bi * g0[0];
        tot[i][1] += sc * (acc[i][a][1] - g0[3]) + bi * g0[2];
        tot[i][2] += sc * (acc[i][a][2] - g1[1]) + bi * g1[0];
        tot[i][3] += sc * (acc[i][a][3] - g1[3]) + bi * g1[2];
      }
    }
  }

  // ---- the wave's sums.  MB == 4: register e is batch row e and the four lanes kc of a weight row add up;
  // MB == 8: lanes kc and kc + 2 add up, lane kc < 2 then holds batch rows 4 kc + e.
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float p = tot[i][e];
      if (MB == 4) p += __shfl_xor(p, 16, 64);
      p += __shfl_xor(p, 32, 64);
      tot[i][e] = p;
    }
  const bool holder = kc < (MB == 8 ? 2 : 1);
  const int m_first = MB == 8 ? kc * 4 : 0;

  if (holder) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int n = (rb0 + i) * 16 + r;
      if (n < n_out) {
        const float ob = out_bias ? (float)out_bias[n] : 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (m_first + e < m_rows) y[(int64_t)(m_first + e) * n_out + n] = (half_t)apply_activation(tot[i][e] + ob, act);
      }
    }
  }
}

}  // namespace

// Whether the kernel takes the shape (three to eight rows, group 64; alignment is the caller's to check): all of K
// fits the LDS, and the groups of 8 row blocks alone give most of the 256 compute units a workgroup.  Measured at
// four / eight rows against the kernels that serve otherwise (this kernel's time / theirs): 16384 x 4096, 128
// workgroups, 1.32 / 1.51; 24576 x 4096, 192 workgroups, 0.93 / 0.99; 28672 x 4096, 224, 0.86 / 0.92 (14.3 / 16.9 us);
// 32768 x 4096 0.85 / 0.91; 49152 x 4096 0.90 / 0.90; 65536 x 2048 0.72 / 0.69; 32768 x 1024 0.58 / 0.63.
bool gemv_rows_fits(int64_t m_rows, int64_t n_out, int64_t k_in) {
  if (m_rows < 3 || m_rows > 8 || k_in < 512 || k_in % 512 != 0 || k_in / 512 > kRowsMaxChunks) return false;
  const int64_t groups = ((n_out + 15) / 16 + kRowsWaves - 1) / kRowsWaves;
  return groups >= 208;
}

// Three to eight batch rows on group 64, x, packed (or blob), scale and bias 16-byte aligned, a shape that
// gemv_rows_fits (the caller has checked).  `blob`: NULL (the three variables are read) or the weight's
// streaming-layout copy.
int launch_gemv_rows(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                     const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in, int act,
                     hipStream_t stream, int64_t ldx) {
  const int xm = m_rows <= 4 ? 4 : 8;
  const unsigned groups = (unsigned)(((n_out + 15) / 16 + kRowsWaves - 1) / kRowsWaves);
  const uint4_t *const weight = reinterpret_cast<const uint4_t *>(blob ? blob : packed);
  const int lds_bytes = rows_lds_bytes(xm, (int)(k_in / 512));
#define GQ_ROWS_LAUNCH(XM, BLOB)                                                                                      \
  do {                                                                                                                \
    static_assert(rows_lds_bytes(XM, kRowsMaxChunks) <= 160 * 1024, "LDS budget");                                    \
    if (rows_lds_bytes(XM, kRowsMaxChunks) > 64 * 1024) { /* beyond the default limit of a launch */                  \
      constexpr int kMaxDevices = 64;                                                                                 \
      static bool configured[kMaxDevices] = {false};                                                                  \
      int dev = 0;                                                                                                    \
      if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return GQ_ERR_NO_DEVICE;                 \
      if (!configured[dev]) {                                                                                         \
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_rows_kernel<1, XM, BLOB>),       \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize,                          \
                                                 rows_lds_bytes(XM, kRowsMaxChunks));                                 \
        if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));                    \
        configured[dev] = true;                                                                                       \
      }                                                                                                               \
    }                                                                                                                 \
    gemv_rows_kernel<1, XM, BLOB><<<dim3(groups), dim3(kRowsWaves * 64), lds_bytes, stream>>>(                        \
        reinterpret_cast<const half_t *>(x), (int)m_rows, weight, reinterpret_cast<const half_t *>(scale),            \
        reinterpret_cast<const half_t *>(bias), reinterpret_cast<const half_t *>(out_bias),                           \
        reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, act, (int)(ldx ? ldx : k_in));                          \
  } while (0)
  if (blob && xm == 4) GQ_ROWS_LAUNCH(4, true);
  else if (blob) GQ_ROWS_LAUNCH(8, true);
  else if (xm == 4) GQ_ROWS_LAUNCH(4, false);
  else GQ_ROWS_LAUNCH(8, false);
#undef GQ_ROWS_LAUNCH
  return check_launch("gemv_rows_kernel");
}

}  // namespace gq
