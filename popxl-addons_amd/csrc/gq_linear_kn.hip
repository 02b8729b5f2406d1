// Fused int4 dequant + matmul for weights grouped along the OUTPUT features, for gfx950:
// the layout of LinearGQ with dim = -1 or 1, the constructor default of the reference
// (popxl_addons/layers/linear_gq.py:26, 59-62, 99-101).
//
//   packed [k_in, n_out / gs, gs / 4] uint16, scale / bias [k_in, n_out / gs]
//   W[k][n] = code * scale[k][n / gs] + bias[k][n / gs],   y[m][n] = sum_k x[m][k] * W[k][n] (+ out_bias[n])
//
// A packed word holds 8 consecutive OUTPUT features of one input feature k: along the contraction
// the codes of one output are a weight row (n_out / 2 bytes) apart.  The MFMA wants every lane to
// hold a run of the contraction index, which this layout cannot give without a transposition, so:
//
//  * decode batches (m_rows <= 16), HBM-bound on the packed weight: the MFMA contracts over 4 input
//    features and the 8 codes of a word at once, with a ONE-HOT B operand that routes code p of a
//    word to output column p -- see gemv_kn_kernel.  The contraction is split over the waves of a
//    workgroup (LDS) and over workgroups (fp32 partial sums in a scratch buffer; the last
//    workgroup to arrive at an output strip adds them up in a fixed order).
//  * prefill batches: the weight tile is expanded into LDS transposed (gemm_kn_tile_kernel).
#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {

// ---------------------------------------------------------------------------------------
// Decode kernel.  v_mfma_f32_16x16x32_f16: D[i][c] += sum_{kc, p} A[i][(kc, p)] * B[(kc, p)][c],
// lane (i = lane % 16, kc = lane / 16) supplies A[i][(kc, 0..7)] and B[(kc, 0..7)][c = lane % 16].
//   A: lane (i, kc) loads 8 bytes = 2 words = 16 outputs of input feature k0 + kc, at outputs
//      n_strip + 16 i ..; word t of the lane is the A operand of MFMA t (dequantised, 8 fp16 in the
//      pair order (0,4,1,5,2,6,3,7) of their positions in the word).
//   B: column c = (p', mm): position p' of a word, batch row mm of the pair the MFMA serves.
//      B[(kc, p)][c] = x[mm][k0 + kc] if p == p' else 0 -- one non-zero half per lane.
//   D_t[i][(p', mm)] = sum_kc W[k0 + kc][n_strip + 16 i + 8 t + order(p')] * x[mm][k0 + kc].
// One MFMA thus does 4 x 128 x 2 useful multiply-adds of its 8192: the matrix pipe has the room
// (HBM delivers ~12 bytes per clock to a compute unit; 64 lanes x 8 bytes feed 2 MFMAs per batch
// pair), and the weights go from memory to the MFMA without a shuffle or an LDS round trip.
// A workgroup covers a strip of 256 outputs (128 contiguous bytes per weight row, four rows per
// load instruction) and a slab of input features; its NW waves take every NW-th block of 4 input
// features.  Narrow strips keep the cross-workgroup reduction small: one workgroup per compute
// unit means (256 / strips) slabs, each leaving 2 KiB per batch-row pair for the strip's last
// workgroup to add up.
// ---------------------------------------------------------------------------------------
constexpr int kStrip = 256;       // outputs per workgroup
constexpr int kMaxStrips = 4096;  // arrival counters at the start of the scratch buffer (16 KiB)

// device-coherent 16-byte accesses (sc1: written through to, and read from, the level of the memory
// system that every compute unit sees): the partial sums of one workgroup are read by another
// workgroup of the same launch
__device__ __forceinline__ void store_coherent(float4_t *p, float4_t v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
template <int N>
__device__ __forceinline__ void load_coherent(const float4_t *p, int64_t stride, float4_t (&v)[N]) {
#pragma unroll
  for (int j = 0; j < N; ++j) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[j]) : "v"(p + j * stride) : "memory");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int j = 0; j < N; ++j) asm volatile("" : "+v"(v[j]));  // (uses of v stay below the wait)
}

// MP: batch-row pairs (m_rows <= 2 MP); NW: waves.  Scratch: one arrival counter per strip (zero
// before and after every launch) and partial[split][strip][pair][t][lane] (a float4 each: the
// accumulators as the lanes hold them).
template <int MP, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_kn_kernel(const half_t *__restrict__ x, int m_rows,
                                                          const char *__restrict__ packed, const half_t *__restrict__ scale,
                                                          const half_t *__restrict__ bias, const half_t *__restrict__ out_bias,
                                                          half_t *__restrict__ y, int n_out, int k_in, int gs_shift, int act,
                                                          int slab, float4_t *__restrict__ partial,
                                                          unsigned *__restrict__ counters) {
  __shared__ float4_t red[NW][2][64];
  __shared__ unsigned arrived;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, kc = lane >> 4;
  const int strip = blockIdx.x, n_strips = gridDim.x, split = blockIdx.y, n_splits = gridDim.y;
  const int n_groups = n_out >> gs_shift;
  const int64_t row_bytes = n_out >> 1;
  // this lane's 16 outputs; lanes past n_out re-read the last 8 bytes of the row (results dropped)
  const int n_lane = strip * kStrip + 16 * i;
  const int n_load = min(n_lane, n_out - 16);
  const int g_lane = n_load >> gs_shift;
  const int k_begin = split * slab, k_end = min(k_in, k_begin + slab);

  // B operand masks: column c = 2 p' + mm keeps x at position p' of the half8
  const int c = lane & 15, p_sel = c >> 1, mm = c & 1;
  uint32_t mask[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) mask[r] = (p_sel >> 1) == r ? ((p_sel & 1) ? 0xFFFF0000u : 0x0000FFFFu) : 0u;

  float4_t acc[MP][2];
#pragma unroll
  for (int mp = 0; mp < MP; ++mp)
#pragma unroll
    for (int t = 0; t < 2; ++t) acc[mp][t] = float4_t{0.f, 0.f, 0.f, 0.f};

  // U blocks of 4 input features per iteration, every load of them issued before the first use:
  // a wave keeps U x 512 bytes of weights in flight
  constexpr int U = MP <= 2 ? 8 : (MP <= 4 ? 4 : 2);
  for (int kb = k_begin + 4 * wave; kb < k_end; kb += 4 * NW * U) {
    uint2_t wq[U];
    uint32_t sv[U], bv[U], xv[U][MP];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = kb + 4 * NW * u + kc;
      const bool live = k < k_end;
      const int kk = live ? k : k_end - 1;  // (past the slab: any valid row, multiplied by x = 0)
      wq[u] = __builtin_nontemporal_load(reinterpret_cast<const uint2_t *>(packed + kk * row_bytes + (n_load >> 1)));
      sv[u] = __builtin_bit_cast(uint16_t, scale[(int64_t)kk * n_groups + g_lane]);
      bv[u] = __builtin_bit_cast(uint16_t, bias[(int64_t)kk * n_groups + g_lane]);
#pragma unroll
      for (int mp = 0; mp < MP; ++mp) {
        const int m = 2 * mp + mm;
        xv[u][mp] = (live && m < m_rows) ? (uint32_t)__builtin_bit_cast(uint16_t, x[(int64_t)m * k_in + k]) : 0u;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const half2_t s2 = as_half2(sv[u] | (sv[u] << 16)), b2 = as_half2(bv[u] | (bv[u] << 16));
      half8_t a[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) a[t] = dequant_word(wq[u][t], s2, b2);
#pragma unroll
      for (int mp = 0; mp < MP; ++mp) {
        const uint32_t xx = xv[u][mp] | (xv[u][mp] << 16);
        uint4_t bq;
#pragma unroll
        for (int r = 0; r < 4; ++r) bq[r] = xx & mask[r];
        const half8_t b = __builtin_bit_cast(half8_t, bq);
#pragma unroll
        for (int t = 0; t < 2; ++t) acc[mp][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t], b, acc[mp][t], 0, 0, 0);
      }
    }
  }

  // lane (c, rg) of accumulator (mp, t) holds, in element e, row i = 4 rg + e: the output
  // n = strip + 16 i + 8 t + order(p'), batch row m = 2 mp + mm.  The waves' sums meet in LDS, one
  // batch-row pair at a time; threads 0..127 then own one float4 (t, lane) each.
  const bool direct = n_splits == 1;
  const int ot = (threadIdx.x >> 6) & 1, ol = threadIdx.x & 63;
  auto finish = [&](int mp, float4_t sum) {  // sum + out_bias -> activation -> y
    const int cc = ol & 15, rg = ol >> 4;
    const int m = 2 * mp + (cc & 1);
    if (m >= m_rows) return;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // position p' = cc / 2 of a word holds its element p' / 2 + 4 (p' % 2)
      const int n = strip * kStrip + 16 * (4 * rg + e) + 8 * ot + (cc >> 2) + 4 * ((cc >> 1) & 1);
      if (n >= n_out) continue;
      float v = sum[e];
      if (out_bias) v += (float)out_bias[n];
      y[(int64_t)m * n_out + n] = (half_t)apply_activation(v, act);
    }
  };
  float4_t *mine = partial + (((int64_t)split * n_strips + strip) * MP) * 128 + threadIdx.x;
#pragma unroll
  for (int mp = 0; mp < MP; ++mp) {
    if (mp > 0) __syncthreads();
#pragma unroll
    for (int t = 0; t < 2; ++t) red[wave][t][lane] = acc[mp][t];
    __syncthreads();
    if (threadIdx.x < 128) {
      float4_t sum = red[0][ot][ol];
#pragma unroll
      for (int w = 1; w < NW; ++w) sum += red[w][ot][ol];
      if (direct) finish(mp, sum);
      else store_coherent(mine + mp * 128, sum);
    }
  }
  if (direct) return;
  // the workgroup's partial sums are in memory before it counts itself in
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned before = __hip_atomic_fetch_add(counters + strip, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    arrived = before;
    if (before == (unsigned)n_splits - 1)  // the last one: leave the counter at zero for the next launch
      __hip_atomic_store(counters + strip, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (arrived != (unsigned)n_splits - 1 || threadIdx.x >= 128) return;
  // last workgroup of the strip: add the slabs in order (the same result whoever arrives last),
  // eight loads in flight at a time
  const int64_t stride = (int64_t)n_strips * MP * 128;  // float4 between consecutive slabs
  const float4_t *first = partial + ((int64_t)strip * MP) * 128 + threadIdx.x;
#pragma unroll
  for (int mp = 0; mp < MP; ++mp) {
    float4_t sum = {0.f, 0.f, 0.f, 0.f};
    int s = 0;
    for (; s + 8 <= n_splits; s += 8) {
      float4_t v[8];
      load_coherent<8>(first + mp * 128 + s * stride, stride, v);
#pragma unroll
      for (int j = 0; j < 8; ++j) sum += v[j];
    }
    for (; s < n_splits; ++s) {
      float4_t v[1];
      load_coherent<1>(first + mp * 128 + s * stride, stride, v);
      sum += v[0];
    }
    finish(mp, sum);
  }
}

// Any group_size % 4 == 0, any n_out % 4 == 0: one thread per output, up to 16 batch rows per launch;
// the weight is rebuilt with the two fp16 roundings of the standalone decompress.
__global__ __launch_bounds__(256) void linear_kn_generic_kernel(const half_t *__restrict__ x, int m_rows,
                                                                const uint16_t *__restrict__ packed,
                                                                const half_t *__restrict__ scale,
                                                                const half_t *__restrict__ bias,
                                                                const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                                int n_out, int k_in, int group_size, int act) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= n_out) return;
  const int words = n_out >> 2, n_groups = n_out / group_size;
  const int shift = 12 - 4 * (n & 3), g = n / group_size;
  float acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = 0.f;
  for (int k = 0; k < k_in; ++k) {
    const uint32_t w = packed[(int64_t)k * words + (n >> 2)];
    const half_t code = (half_t)(float)((w >> shift) & 15u);
    const half_t prod = code * scale[(int64_t)k * n_groups + g];
    const float wv = (float)(half_t)(prod + bias[(int64_t)k * n_groups + g]);
#pragma unroll
    for (int m = 0; m < 16; ++m)
      if (m < m_rows) acc[m] += (float)x[(int64_t)m * k_in + k] * wv;
  }
#pragma unroll
  for (int m = 0; m < 16; ++m)
    if (m < m_rows) {
      float v = acc[m];
      if (out_bias) v += (float)out_bias[n];
      y[(int64_t)m * n_out + n] = (half_t)apply_activation(v, act);
    }
}

// ---------------------------------------------------------------------------------------
// Prefill kernel.  Workgroup = 4 waves (2 x 2), tile 128 (m) x 128 (n) x 64 (k), as the tile kernel
// of the other layout, except for how the weight tile reaches LDS: thread (input feature kr = tid
// % 64, quarter q = tid / 64) loads the 16 bytes = 32 outputs n0 + 32 q .. of feature k0 + kr,
// expands them and stores them TRANSPOSED, Bs[n][kr]; the 64 lanes of a wave write 128 contiguous
// bytes of one Bs row per instruction.
// ---------------------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 64, LDK = BK + 8;

__device__ __forceinline__ uint32_t as_u32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

// gridDim.z > 1: the workgroups of a tile divide K into slabs of `slab` input features; their fp32
// accumulators meet in `partial` ([slab][tile][element][thread], a float4 per element quarter) and the
// last one to arrive at the tile (arrival counters as in the decode kernel: zero before and after)
// adds them in the order of the slabs and stores y.
__global__ __launch_bounds__(256) void gemm_kn_tile_kernel(const half_t *__restrict__ x, int m_rows,
                                                           const char *__restrict__ packed, const half_t *__restrict__ scale,
                                                           const half_t *__restrict__ bias,
                                                           const half_t *__restrict__ out_bias, half_t *__restrict__ y,
                                                           int n_out, int k_in, int gs_shift, int act, int slab,
                                                           float4_t *__restrict__ partial, unsigned *__restrict__ counters) {
  __shared__ __attribute__((aligned(16))) half_t As[BM][LDK];
  __shared__ __attribute__((aligned(16))) half_t Bs[BN][LDK];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int n_groups = n_out >> gs_shift;
  const int64_t row_bytes = n_out >> 1;

  const int a_col = (tid & 7) * 8, a_row = tid >> 3;
  const half_t *a_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) a_src[i] = x + (int64_t)min(m0 + a_row + 32 * i, m_rows - 1) * k_in + a_col;
  const int kr = tid & 63, q = tid >> 6;
  const int n_load = min(n0 + 32 * q, n_out - 32);  // columns past n_out re-read the last 32 (never stored to y)
  const int g = n_load >> gs_shift;
  const char *b_src = packed + (n_load >> 1);

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
    b_reg = *reinterpret_cast<const uint4_t *>(b_src + (int64_t)(k0 + kr) * row_bytes);
    s_reg = scale[(int64_t)(k0 + kr) * n_groups + g];
    z_reg = bias[(int64_t)(k0 + kr) * n_groups + g];
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4_t *>(&As[a_row + 32 * i][a_col]) = a_reg[i];
    const half2_t s2 = {s_reg, s_reg}, z2 = {z_reg, z_reg};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      // pair order (0,4) (1,5) (2,6) (3,7) of the word's eight outputs
      const half8_t v = dequant_word(b_reg[w], s2, z2);
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        Bs[32 * q + 8 * w + p][kr] = v[2 * p];
        Bs[32 * q + 8 * w + p + 4][kr] = v[2 * p + 1];
      }
    }
  };

  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
  const int k_begin = (int)blockIdx.z * slab, k_end = min(k_in, k_begin + slab);
  load_tile(k_begin);
  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    __syncthreads();
    store_tile();
    __syncthreads();
    if (k0 + BK < k_end) load_tile(k0 + BK);
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

  if (gridDim.z > 1) {
    __shared__ unsigned tile_arrived;
    const int n_splits = gridDim.z, tile = blockIdx.y * gridDim.x + blockIdx.x, n_tiles = gridDim.x * gridDim.y;
    float4_t *mine = partial + ((int64_t)blockIdx.z * n_tiles + tile) * (16 * 256) + tid;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          store_coherent(mine + ((i * 2 + j) * 4 + q4) * 256,
                         float4_t{acc[i][j][4 * q4], acc[i][j][4 * q4 + 1], acc[i][j][4 * q4 + 2], acc[i][j][4 * q4 + 3]});
    // the workgroup's partial sums are in memory before it counts itself in
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      const unsigned before = __hip_atomic_fetch_add(counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      tile_arrived = before;
      if (before == (unsigned)n_splits - 1)  // the last one: leave the counter at zero for the next launch
        __hip_atomic_store(counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (tile_arrived != (unsigned)n_splits - 1) return;
    // the slabs in order (the same result whoever arrives last), a slab's sixteen loads in flight at a time
    const float4_t *first = partial + (int64_t)tile * (16 * 256) + tid;
    const int64_t stride = (int64_t)n_tiles * (16 * 256);  // float4 between consecutive slabs
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int sp = 0; sp < n_splits; ++sp) {
      float4_t v[16];
      load_coherent<16>(first + sp * stride, 256, v);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] += v[(i * 2 + j) * 4 + (e >> 2)][e & 3];
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
        if (m < m_rows) y[(int64_t)m * n_out + n] = (half_t)apply_activation(acc[i][j][e] + ob, act);
      }
    }
}

// waves of the decode kernel for a batch (the 16 accumulator registers per batch-row pair of the
// largest batches leave room for 8 waves' worth of registers only)
int kn_waves(int64_t m_rows) { return m_rows <= 8 ? 16 : 8; }
int kn_pairs(int64_t m_rows) { return m_rows <= 2 ? 1 : (m_rows <= 4 ? 2 : (m_rows <= 8 ? 4 : 8)); }

// K slabs of the decode kernel: one workgroup per compute unit (256), slabs a multiple of the input
// features that the waves take per round, at least two rounds per wave
int kn_splits(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t *slab_out) {
  const int64_t round = 4 * kn_waves(m_rows);
  const int64_t strips = (n_out + kStrip - 1) / kStrip;
  int64_t splits = (256 + strips - 1) / strips;
  const int64_t max_splits = (k_in + 2 * round - 1) / (2 * round);
  if (splits > max_splits) splits = max_splits;
  if (splits < 1) splits = 1;
  int64_t slab = (k_in + splits - 1) / splits;
  slab = (slab + round - 1) / round * round;
  splits = (k_in + slab - 1) / slab;
  *slab_out = slab;
  return (int)splits;
}

bool kn_fast_shape(const uint16_t *x, const uint16_t *packed, int64_t n_out, int64_t k_in, int64_t group_size) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  return pow2 && group_size >= 32 && n_out % 32 == 0 && n_out >= 32 && n_out <= (int64_t)kMaxStrips * kStrip &&
         k_in > 0 && ((uintptr_t)packed % 16) == 0 && ((uintptr_t)x % 2) == 0;
}

}  // namespace

// K slabs of the prefill kernel: enough workgroups for the 256 compute units where the tiles alone are
// few (a weight with 4096 outputs has 32 per 128 rows), slabs of at least 512 input features, at most 16
int kn_prefill_splits(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t *slab_out) {
  const int64_t tiles = ((n_out + BN - 1) / BN) * ((m_rows + BM - 1) / BM);
  int64_t splits = tiles >= 192 ? 1 : (256 + tiles - 1) / tiles;
  if (splits > 16) splits = 16;
  if (splits > k_in / 512) splits = k_in / 512;
  if (splits < 1 || tiles > kMaxStrips) splits = 1;
  int64_t slab = (k_in + splits - 1) / splits;
  slab = (slab + BK - 1) / BK * BK;
  *slab_out = slab;
  return (int)((k_in + slab - 1) / slab);
}

bool kn_prefill_shape(int64_t n_out, int64_t k_in, int64_t group_size) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  return pow2 && group_size >= 32 && n_out % 32 == 0 && n_out >= 32 && n_out <= (int64_t)kMaxStrips * kStrip && k_in % BK == 0;
}

// Batches of 17 to 128 rows as passes of the decode kernel over 16 rows each, against the prefill
// kernel, whose 128 x 128 tiles are mostly empty there.  From measured times (us): a pass of 16 rows
// 18 + 0.37 per Mi weights (23.9 on 4096 -> 4096, 41.8 on 4096 -> 16384, 41.3 on 16384 -> 4096), fewer
// rows in the last pass less; the prefill kernel 1.4 per 64 input features of a slab and round of 256
// workgroups, plus 10 for the partial sums where K is divided (measured with the workspace for that:
// 25 - 28 / 61 - 63 / 61 - 64 on the same shapes, whatever the batch up to 128; undivided 84 / 103 / 370).
// With K divided the prefill kernel wins nearly everywhere; the passes remain for weights whose slabs
// cannot be short enough (few input features, many outputs).
bool kn_passes_faster(int64_t m_rows, int64_t n_out, int64_t k_in) {
  if (m_rows <= 16 || m_rows > 128) return false;
  const double t16 = 18.0 + 0.37 * (double)n_out * (double)k_in / 1048576.0;
  const int64_t rest = m_rows % 16;
  const double last = rest == 0 ? 0.0 : (rest <= 2 ? 0.45 : (rest <= 4 ? 0.55 : (rest <= 8 ? 0.7 : 1.0)));
  const double t_passes = ((double)(m_rows / 16) + last) * t16;
  // (with K divided over workgroups: a slab's steps, and some 10 us for the partial sums to meet)
  int64_t slab = 0;
  const int splits = kn_prefill_splits(m_rows, n_out, k_in, &slab);
  const int64_t tiles = (n_out + BN - 1) / BN * splits;  // (one row of tiles up to 128 rows)
  const double t_prefill = 1.4 * (double)slab / 64.0 * (double)((tiles + 255) / 256) + (splits > 1 ? 10.0 : 0.0);
  return t_passes < t_prefill;
}

// Scratch bytes the decode kernel needs for this problem (0: none): the arrival counters (a fixed
// 16 KiB at the start, so that calls of any shape find them at the same place), then 2 KiB of
// fp32 partial sums per (K slab, strip, batch-row pair).
int64_t linear_kn_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size) {
  if (m_rows > 16 && kn_passes_faster(m_rows, n_out, k_in)) m_rows = 16;  // passes of the decode kernel over 16 rows
  if (m_rows > 16) {
    // the prefill kernel with K divided over workgroups: counters, then 64 KiB of partial sums per (slab, tile)
    if (!kn_prefill_shape(n_out, k_in, group_size)) return 0;
    int64_t slab = 0;
    const int splits = kn_prefill_splits(m_rows, n_out, k_in, &slab);
    if (splits == 1) return 0;
    const int64_t tiles = ((n_out + BN - 1) / BN) * ((m_rows + BM - 1) / BM);
    return (int64_t)kMaxStrips * 4 + splits * tiles * 65536;
  }
  if (m_rows < 1 || m_rows > 16 || k_in < 1) return 0;
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  if (!pow2 || group_size < 32 || n_out % 32 != 0 || n_out < 32 || n_out > (int64_t)kMaxStrips * kStrip) return 0;
  int64_t slab = 0;
  const int splits = kn_splits(m_rows, n_out, k_in, &slab);
  if (splits == 1) return 0;
  const int64_t strips = (n_out + kStrip - 1) / kStrip;
  return (int64_t)kMaxStrips * 4 + splits * strips * kn_pairs(m_rows) * 2048;
}

// `workspace`: linear_kn_workspace_bytes() bytes of device memory whose first 16 KiB (the counters)
// are zero; the kernel leaves them zero.
int launch_linear_kn(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                     const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                     int64_t group_size, int act, void *workspace, hipStream_t stream) {
  const half_t *xh = reinterpret_cast<const half_t *>(x), *sh = reinterpret_cast<const half_t *>(scale),
               *bh = reinterpret_cast<const half_t *>(bias), *oh = reinterpret_cast<const half_t *>(out_bias);
  half_t *yh = reinterpret_cast<half_t *>(y);
  const bool fast = kn_fast_shape(x, packed, n_out, k_in, group_size);
  const int gs_shift = fast ? __builtin_ctzll((unsigned long long)group_size) : 0;
  if (fast && m_rows > 16 && kn_passes_faster(m_rows, n_out, k_in) &&
      (workspace || linear_kn_workspace_bytes(16, n_out, k_in, group_size) == 0)) {
    for (int64_t m0 = 0; m0 < m_rows; m0 += 16) {
      const int64_t m = m_rows - m0 < 16 ? m_rows - m0 : 16;
      const int rc = launch_linear_kn(x + m0 * k_in, m, packed, scale, bias, out_bias, y + m0 * n_out, n_out, k_in, group_size,
                                      act, workspace, stream);
      if (rc != GQ_OK) return rc;
    }
    return GQ_OK;
  }
  if (fast && m_rows <= 16) {
    int64_t slab = 0;
    const int splits = kn_splits(m_rows, n_out, k_in, &slab);
    const int64_t strips = (n_out + kStrip - 1) / kStrip;
    unsigned *counters = static_cast<unsigned *>(workspace);
    float4_t *partial = reinterpret_cast<float4_t *>(counters + kMaxStrips);
    const dim3 grid((unsigned)strips, (unsigned)splits);
#define GQ_KN(MP, NW)                                                                                                       \
  gemv_kn_kernel<MP, NW><<<grid, dim3(NW * 64), 0, stream>>>(xh, (int)m_rows, reinterpret_cast<const char *>(packed), sh, bh, \
                                                             oh, yh, (int)n_out, (int)k_in, gs_shift, act, (int)slab, partial, \
                                                             counters)
    if (m_rows <= 2) GQ_KN(1, 16);
    else if (m_rows <= 4) GQ_KN(2, 16);
    else if (m_rows <= 8) GQ_KN(4, 16);
    else GQ_KN(8, 8);
#undef GQ_KN
    return check_launch("gemv_kn_kernel");
  }
  if (fast && k_in % BK == 0 && ((uintptr_t)x % 16) == 0) {
    const dim3 grid((unsigned)((n_out + BN - 1) / BN), (unsigned)((m_rows + BM - 1) / BM));
    if (grid.y > 65535) return fail(GQ_ERR_UNSUPPORTED, "gq_linear_kn: m_rows=%lld too large", (long long)m_rows);
    // K divided over workgroups where the tiles are few and the caller brought the workspace for it
    int64_t slab = k_in;
    int splits = workspace ? kn_prefill_splits(m_rows, n_out, k_in, &slab) : 1;
    if (splits == 1) slab = k_in;
    unsigned *counters = static_cast<unsigned *>(workspace);
    float4_t *partial = workspace ? reinterpret_cast<float4_t *>(counters + kMaxStrips) : nullptr;
    const dim3 grid3(grid.x, grid.y, (unsigned)splits);
    gemm_kn_tile_kernel<<<grid3, dim3(256), 0, stream>>>(xh, (int)m_rows, reinterpret_cast<const char *>(packed), sh, bh, oh,
                                                         yh, (int)n_out, (int)k_in, gs_shift, act, (int)slab, partial, counters);
    return check_launch("gemm_kn_tile_kernel");
  }
  const unsigned blocks = (unsigned)((n_out + 255) / 256);
  for (int64_t m0 = 0; m0 < m_rows; m0 += 16) {
    const int m = (int)(m_rows - m0 < 16 ? m_rows - m0 : 16);
    linear_kn_generic_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(xh + m0 * k_in, m, packed, sh, bh, oh, yh + m0 * n_out,
                                                                     (int)n_out, (int)k_in, (int)group_size, act);
  }
  return check_launch("linear_kn_generic_kernel");
}

// ---------------------------------------------------------------------------------------
// The same computation for callers that cannot hand over (or allocate) a workspace: the scratch
// buffer is a device array of this library, one copy per GPU, held until the process ends.  Its
// arrival counters are zero when the code object is loaded and every call leaves them zero; the
// partial sums need no clearing (every word that is read was written by the same call).
// Calls on one GPU share the array: calls that overlap (different streams) race.
// ---------------------------------------------------------------------------------------
constexpr int64_t kScratchBytes = (int64_t)kMaxStrips * 4 + GQ_LINEAR_KN_NOALLOC_PARTIAL_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

int launch_linear_kn_noalloc(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                             const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                             int64_t group_size, int act, hipStream_t stream) {
  int64_t need = linear_kn_workspace_bytes(m_rows, n_out, k_in, group_size);
  if (need > kScratchBytes && m_rows > 16) need = 0;  // (no passes of the decode kernel then: the prefill kernel needs no scratch)
  if (need > kScratchBytes)
    return fail(GQ_ERR_UNSUPPORTED,
                "gq_linear_kn_act_noalloc_f16: m_rows=%lld n_out=%lld k_in=%lld needs %lld bytes of scratch, the built-in "
                "buffer holds %lld; use gq_linear_kn_act_f16 with a workspace",
                (long long)m_rows, (long long)n_out, (long long)k_in, (long long)need, (long long)kScratchBytes);
  void *ptr = nullptr;
  if (need > 0) {
    // the array's name is a host-side stand-in: its device address is looked up once per GPU, with
    // that GPU current (every GPU has its own copy at its own address)
    constexpr int kMaxDevices = 64;
    static void *scratch_ptr[kMaxDevices] = {nullptr};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(GQ_ERR_UNSUPPORTED, "device index %d", dev);
    static SharedBlockGuard guard = {};
    const int claimed = claim_shared_block(guard, dev, stream, "gq_linear_kn_act_noalloc_f16");
    if (claimed != GQ_OK) return claimed;
    if (!scratch_ptr[dev]) {
      void *p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !p) return fail(e == hipSuccess ? GQ_ERR_NO_DEVICE : (int)e, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
      scratch_ptr[dev] = p;
    }
    ptr = scratch_ptr[dev];
  }
  return launch_linear_kn(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, act, ptr, stream);
}

}  // namespace gq
