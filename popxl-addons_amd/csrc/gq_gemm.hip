// Fused int4 dequant + GEMM (prefill-sized batches) on fp16 MFMA for gfx950.
//
// y[m][n] = sum_k x[m][k] * W[n][k] (+ out_bias[n]),  W[n][k] = code * scale[n][k/gs] + bias[n][k/gs]
// -- LinearGQ.build with dim=0 (popxl_addons/layers/linear_gq.py:99-109); the fp16 weight only
// ever exists in LDS/registers.  Bound by the fp16 dense MFMA rate for m_rows >= 512.
#include "gq_common.h"

namespace gq {

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
                                                        int n_out, int k_in, int gs_shift, int act) {
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
        if (m < m_rows) y[(int64_t)m * n_out + n] = (half_t)apply_activation(acc[i][j][e] + ob, act);
      }
    }
}


// (w & mask) | magic in one VALU op; mask and magic live in VGPRs.
__device__ __forceinline__ uint32_t and_or(uint32_t w, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "v"(mask), "v"(magic));
  return r;
}

// codes (2p, 2p+1) of a word sit in one byte: byte 1, 0, 3, 2 for p = 0..3, high nibble first.
// The byte is copied to byte 0 and byte 2 of a register; masking 0x000F00F0 leaves code 2p at
// bits 7:4 of the low half (read as 1024 + 16 c) and code 2p+1 at bits 3:0 of the high half
// (1024 + c); one packed fma with (1/16, 1) and (-64, -1024) makes both exact.
__device__ __forceinline__ half8_t dequant_word_natural(uint32_t w, half2_t s2, half2_t b2) {
  const half2_t kMul = {(half_t)0.0625f, (half_t)1.0f};
  const half2_t kAdd = {(half_t)-64.0f, (half_t)-1024.0f};
  const uint32_t kMask = 0x000F00F0u, kMagic = 0x64006400u;
  const uint32_t t0 = __builtin_amdgcn_perm(0u, w, 0x0c010c01u);
  const uint32_t t1 = __builtin_amdgcn_perm(0u, w, 0x0c000c00u);
  const uint32_t t2 = __builtin_amdgcn_perm(0u, w, 0x0c030c03u);
  const uint32_t t3 = __builtin_amdgcn_perm(0u, w, 0x0c020c02u);
  const half2_t c0 = __builtin_elementwise_fma(as_half2(and_or(t0, kMask, kMagic)), kMul, kAdd);
  const half2_t c1 = __builtin_elementwise_fma(as_half2(and_or(t1, kMask, kMagic)), kMul, kAdd);
  const half2_t c2 = __builtin_elementwise_fma(as_half2(and_or(t2, kMask, kMagic)), kMul, kAdd);
  const half2_t c3 = __builtin_elementwise_fma(as_half2(and_or(t3, kMask, kMagic)), kMul, kAdd);
  const half2_t w0 = __builtin_elementwise_fma(c0, s2, b2);
  const half2_t w1 = __builtin_elementwise_fma(c1, s2, b2);
  const half2_t w2 = __builtin_elementwise_fma(c2, s2, b2);
  const half2_t w3 = __builtin_elementwise_fma(c3, s2, b2);
  return __builtin_shufflevector(__builtin_shufflevector(w0, w1, 0, 1, 2, 3),
                                 __builtin_shufflevector(w2, w3, 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
}

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt = bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// s_waitcnt lgkmcnt(n) that also "touches" a register tuple, so that instructions consuming the
// tuple cannot be scheduled above the wait
template <int N>
__device__ __forceinline__ void wait_lds(uint4_t &a) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a) : "n"(N));
}

// ---------------------------------------------------------------------------------------
// Pipelined kernel for large batches.
//
// Workgroup = WM x WN waves; a wave owns FM x FN accumulators of 32 x 32 (v_mfma_f32_32x32x16_f16),
// i.e. a (32 FM) x (32 FN) sub-tile; K advances 64 at a time ("tile").
//
// Data flow.  Everything that comes from global memory goes straight into LDS with
// global_load_lds_* (no VGPR staging), two tiles ahead, and is read back with ds_read instructions
// issued from inline assembly and waited for explicitly.  The compiler therefore never sees a
// register with a load in flight: its own wait insertion is conservative across the loop back edge
// and cannot tell ring stages apart, and would drain the whole prefetch queue (vmcnt(0)) once per
// iteration.
//   x tile  : XS-stage ring shared by the workgroup.  A row is 8 chunks of 16 bytes; chunk c of row
//             r sits at chunk slot c ^ ((r >> 1) & 7), so the 16-byte fragment reads of 16
//             consecutive rows cover all 64 LDS banks once (measured: zero bank conflicts).  The
//             swizzle is applied by choosing each lane's source address.
//   weights : 3-stage ring private to each wave.  Lane (n, h) owns the 16 bytes = 32 codes of row n
//             that start at index 32 h of the tile; lanes with h == 0 also fetch the dword holding
//             the row's scale and the one holding its bias.  One 32-bit word per MFMA step is
//             expanded into the B operand in memory order: per pair of codes one byte permute, one
//             and-or into the mantissa of 1024.0, one packed fma that recovers the exact codes,
//             one packed fma with (scale, bias) -- 16 VALU instructions per 8 weights.
//   MFMA step s of a tile contracts indices {32 h + 8 s + i}: lane (m, h) of the A operand reads
//   chunk 4 h + s of its row.
//
// Schedule of a tile (4 MFMA steps):
//   * steps 0..2 are FM groups of {FN MFMAs, one A-fragment read for the next step, one
//     direct-to-LDS load of the tile two ahead, a slice of the next step's dequantisation}, fenced
//     with sched_barrier so the compiler keeps the interleaving.  Loads are never issued as a
//     burst: eight waves issuing a whole tile at once block each other behind the 64 B/clk
//     address path of the compute unit for ~1000 cycles.
//   * before step 3 comes the only workgroup barrier of the tile: every wave has waited for its
//     own LDS reads of this tile and for its own loads of the next one, so after the barrier the
//     next tile is readable and this tile's x stage may be overwritten.  The next tile's weights,
//     first A fragments and first B operand are fetched and built under the MFMAs of step 3.
// ---------------------------------------------------------------------------------------
constexpr int kWStages = 3;

// KS: groups of WM x WN waves that split the contraction between them (group g takes the g-th
// part of the K tiles, with an x ring of its own) and add their accumulators through LDS at the
// end.  For small batches, where a workgroup per compute unit with one wave per SIMD leaves every
// latency of the K step exposed: twice the waves on the same output tile, no more weight expansion.
template <int WM, int WN, int FM, int FN, int XS, int KS = 1>
struct Pipe2Shape {
  static constexpr int NW = WM * WN, TM = 32 * FM, TN = 32 * FN, TILE_M = WM * TM, TILE_N = WN * TN;
  static constexpr int X_STAGE = TILE_M * 128, W_STAGE = FN * 1280;
  static constexpr int X_BYTES = XS * X_STAGE, LDS_BYTES = KS * (X_BYTES + NW * kWStages * W_STAGE);
  static constexpr int A_OPS = TILE_M / 8 / NW;
  static constexpr int OPS = A_OPS + 3 * FN;
  static constexpr int REDUCE_BYTES = (KS - 1) * NW * FM * FN * 16 * 256;  // accumulators of groups 1.. as floats
  static_assert(REDUCE_BYTES <= LDS_BYTES, "the accumulators of the other groups must fit the rings");
};

// The 16 VALU instructions that turn one packed word into a B operand, cut into PIECES slices so
// that they can be spread between MFMAs.  State: t (permuted bytes / raw halves), c (exact codes).
struct DequantState {
  uint32_t t[4];
  half2_t c[4];
  half2_t w[4];
};

template <int PIECES>
__device__ __forceinline__ void dequant_piece(int piece, uint32_t word, half2_t s2, half2_t z2, DequantState &st) {
  const half2_t kMul = {(half_t)0.0625f, (half_t)1.0f};
  const half2_t kAdd = {(half_t)-64.0f, (half_t)-1024.0f};
  const uint32_t kMask = 0x000F00F0u, kMagic = 0x64006400u;
  const uint32_t sel[4] = {0x0c010c01u, 0x0c000c00u, 0x0c030c03u, 0x0c020c02u};
  // operation o of pair p: 0 byte permute, 1 and-or into 1024.0, 2 exact code, 3 scale and bias
#pragma unroll
  for (int op = 0; op < 16; ++op) {
    if (op * PIECES / 16 != piece) continue;
    const int p = op >> 2, o = op & 3;
    if (o == 0) st.t[p] = __builtin_amdgcn_perm(0u, word, sel[p]);
    if (o == 1) st.t[p] = and_or(st.t[p], kMask, kMagic);
    if (o == 2) st.c[p] = __builtin_elementwise_fma(as_half2(st.t[p]), kMul, kAdd);
    if (o == 3) st.w[p] = __builtin_elementwise_fma(st.c[p], s2, z2);
  }
}

__device__ __forceinline__ half8_t dequant_result(const DequantState &st) {
  return __builtin_shufflevector(__builtin_shufflevector(st.w[0], st.w[1], 0, 1, 2, 3),
                                 __builtin_shufflevector(st.w[2], st.w[3], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
}

// The same for a word of the kn streaming layout (gq_gemv_kn.hip: weights grouped along the OUTPUT
// features, the codes of an output contiguous along the input features).  Code e of a word sits in
// nibble (3,7,2,6,1,5,0,4)[e], so the pair (2p, 2p+1) is the same nibble, 3 - p, of the two 16-bit
// halves: a shift brings it to bits 3:0, one and-or puts both codes into the mantissas of 1024.0, one
// packed add makes them exact, and one packed fma applies the pair's OWN scales and biases (every
// input feature has its own in this layout): sq / zq hold (scale[k], scale[k+1]) for the four pairs.
// (One mask and one magic number for all pairs: the 256 x 256 tile has no registers to spare.)
struct KnMasks {
  uint32_t mask, magic;  // in vector registers the compiler cannot see through (v_and_or_b32)
};
// LATE: the four fmas, which need the scales, are the last four operations (the scales are then
// fetched while the first twelve run).
template <int PIECES, bool LATE = false>
__device__ __forceinline__ void dequant_piece_kn(int piece, uint32_t word, uint4_t sq, uint4_t zq, const KnMasks &km,
                                                 DequantState &st) {
  const half2_t kNeg1024 = {(half_t)-1024.0f, (half_t)-1024.0f};
#pragma unroll
  for (int op = 0; op < 16; ++op) {
    if (op * PIECES / 16 != piece) continue;
    const int p = LATE ? (op < 12 ? op / 3 : op - 12) : op >> 2, o = LATE ? (op < 12 ? op % 3 : 3) : op & 3;
    if (o == 0) st.t[p] = p < 3 ? word >> (12 - 4 * p) : word;
    if (o == 1) st.t[p] = (st.t[p] & km.mask) | km.magic;
    if (o == 2) st.c[p] = as_half2(st.t[p]) + kNeg1024;
    if (o == 3) st.w[p] = __builtin_elementwise_fma(st.c[p], as_half2(sq[p]), as_half2(zq[p]));
  }
}

// KN: `packed` is the weight in the kn streaming layout (scale and bias are not read): lane (n, h) of a
// fragment finds the 32 codes of output n at input features 64 T + 32 h .. of K tile T at
//   unit (n / 64, T / 8) + 4096 ((n / 16) % 4) + 1024 ((T / 2) % 4) + 512 (T % 2) + 256 h + 16 (n % 16),
// and the 64 scales (biases) of the tile at unit + 16384 (17408) + 128 (T % 8).  The 128 bytes of each
// take the places in the wave's ring slot that the 32 scale (bias) dwords of the other layout take;
// a lane reads the 16 bytes of its step's eight input features from them (all lanes of a half-wave
// the same: a broadcast), one step ahead of the expansion that uses them.
// BLOB: `packed` is the weight in the streaming layout of the other layout (groups along the input features;
// gq_gemv_stream.hip): the same ring slots and arithmetic as from the three variables, but lane (n, h) finds its
// 16 bytes of K tile T at
//   item (n / 16, T / 8) + 1024 ((T / 2) % 4) + 512 (T % 2) + 256 h + 16 (n % 16)        (items of 4608 bytes),
// and the dword with the row's scales (biases) of groups T and T ^ 1 at item + 4096 (4352) + 16 (n % 16) + 4 ((T % 8) / 2).
template <int WM, int WN, int FM, int FN, int XS, int KS, bool KN = false, bool BLOB = false>
__device__ __forceinline__ void gemm_pipe2_body(
    const half_t *__restrict__ x, int m_rows, const uint4_t *__restrict__ packed, const half_t *__restrict__ scale,
    const half_t *__restrict__ bias, const half_t *__restrict__ out_bias, half_t *__restrict__ y, int n_out, int k_in,
    int gs_shift, int act, float4_t *__restrict__ partial, unsigned *__restrict__ counters) {
  using S = Pipe2Shape<WM, WN, FM, FN, XS, KS>;
  constexpr int NW = S::NW, TM = S::TM, TN = S::TN, TILE_M = S::TILE_M, TILE_N = S::TILE_N;
  // The streaming layouts, one fragment per wave (every shape in use): its scales and biases come with ONE load
  // instruction, the scales through the lower lanes, the biases through the upper ones (their places in the ring
  // slot are adjacent): 1 - 5 % sooner.  (From the variables, where such a load touches 64 lines instead of twice 32,
  // it measured 3 - 5 % slower at 64 - 128 rows and the same elsewhere.)
  constexpr bool kJoint = FN == 1 && (KN || BLOB);
  constexpr int A_OPS = S::A_OPS, OPS = kJoint ? A_OPS + 2 : S::OPS;
  static_assert(TILE_M % (8 * NW) == 0, "x tile must split evenly over the waves");
  extern __shared__ __attribute__((aligned(16))) char lds[];

  // `wave` is the wave's index within its group of NW; the group takes K tiles [tile0, tile0 + n_tiles)
  const int tid = threadIdx.x, lane = tid & 63, kgrp = (tid >> 6) / NW, wave = (tid >> 6) % NW;
  const int wm = wave / WN, wn = wave % WN;
  const int m0 = blockIdx.y * TILE_M, n0 = blockIdx.x * TILE_N;
  const int groups_per_row = k_in >> gs_shift;
  // gridDim.z > 1: the workgroups of an output tile divide K between them as well (see the end)
  const int n_tiles = (k_in >> 6) / (KS * (int)gridDim.z);  // (the launcher checks divisibility)
  const int tile0 = ((int)blockIdx.z * KS + kgrp) * n_tiles;

  const half_t *a_src[A_OPS];
#pragma unroll
  for (int q = 0; q < A_OPS; ++q) {
    const int slot = (q * NW + wave) * 64 + lane;
    const int r = slot >> 3, c = (slot & 7) ^ ((r >> 1) & 7);
    a_src[q] = x + (int64_t)min(m0 + r, m_rows - 1) * k_in + c * 8 + tile0 * 64;
  }
  const int fr = lane & 31, h = lane >> 5;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  char *x_ring = lds + kgrp * S::X_BYTES;
  const uint32_t a_rd_row = lds_base + kgrp * S::X_BYTES + (wm * TM + fr) * 128;
  uint32_t a_rd_chunk[4];
#pragma unroll
  for (int s4 = 0; s4 < 4; ++s4) a_rd_chunk[s4] = ((4 * h + s4) ^ ((lane >> 1) & 7)) * 16;

  const uint4_t *b_src[FN];
  const uint32_t *s_src[FN], *z_src[FN];
  const char *kn_codes[FN], *kn_scales[FN];  // KN: this lane's codes of K tile 0 / the fragment's scales of K tile 0
  constexpr int kKnUnit = 18432, kStreamItem = 4608;
#pragma unroll
  for (int f = 0; f < FN; ++f) {
    const int row = min(n0 + wn * TN + f * 32 + fr, n_out - 1);
    if (KN) {
      const int64_t chunks = k_in >> 9;
      const int group = min((n0 + wn * TN + f * 32) >> 6, (n_out >> 6) - 1);  // (a fragment lies inside one group of 64)
      kn_codes[f] = reinterpret_cast<const char *>(packed) + (int64_t)(row >> 6) * chunks * kKnUnit + ((row >> 4) & 3) * 4096 +
                    h * 256 + (row & 15) * 16;
      kn_scales[f] = reinterpret_cast<const char *>(packed) + (int64_t)group * chunks * kKnUnit + 16384 + (lane & 7) * 16;
      b_src[f] = nullptr;
      s_src[f] = z_src[f] = nullptr;
    } else if (BLOB) {
      // the items of the row's block of 16 (4608 bytes per 512 input features): this lane's 16 bytes of K tile 0,
      // and the row's 16 bytes of scales (8 groups; the biases 256 bytes on) of the first item
      const char *const items = reinterpret_cast<const char *>(packed) + (int64_t)(row >> 4) * (k_in >> 9) * kStreamItem;
      kn_codes[f] = items + h * 256 + (row & 15) * 16;
      kn_scales[f] = items + 4096 + (row & 15) * 16;
      b_src[f] = nullptr;
      s_src[f] = z_src[f] = nullptr;
    } else {
      kn_codes[f] = kn_scales[f] = nullptr;
      b_src[f] = packed + (int64_t)row * (k_in >> 5) + h + tile0 * 2;
      s_src[f] = reinterpret_cast<const uint32_t *>(scale + (int64_t)row * groups_per_row);
      z_src[f] = reinterpret_cast<const uint32_t *>(bias + (int64_t)row * groups_per_row);
    }
  }
  KnMasks km = {0x000F000Fu, 0x64006400u};
  if (KN) asm volatile("" : "+v"(km.mask), "+v"(km.magic));
  char *w_ring = lds + KS * S::X_BYTES + (kgrp * NW + wave) * (kWStages * S::W_STAGE);
  const uint32_t w_rd = lds_base + KS * S::X_BYTES + (kgrp * NW + wave) * (kWStages * S::W_STAGE);

  // Direct-to-LDS load number `op` (0 .. OPS-1) of tile `t_load` into the ring slots of tile number
  // `t_slot`: A_OPS chunks of the x tile, FN packed fragments, FN scale and FN bias dwords.
  // The two lanes (n, 0) and (n, 1) share one dword of scale and of bias (their groups are the
  // same, or the two halves of it): lanes with h == 0 fetch it.
  auto issue_op = [&](int op, int t_load, int t_slot) {
    char *xs = x_ring + (t_slot % XS) * S::X_STAGE;
    char *ws = w_ring + (t_slot % kWStages) * S::W_STAGE;
    const int g = ((tile0 + t_load) * 64 + h * 32) >> gs_shift;
#pragma unroll
    for (int q = 0; q < A_OPS; ++q)
      if (op == q) __builtin_amdgcn_global_load_lds(a_src[q] + t_load * 64, xs + (q * NW + wave) * 1024, 16, 0, 0);
    if (KN) {
      const int T = tile0 + t_load;  // K tile of the whole weight
      const int64_t unit = (int64_t)(T >> 3) * kKnUnit;
#pragma unroll
      for (int f = 0; f < FN; ++f) {
        if (op == A_OPS + f)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(kn_codes[f] + unit + ((T >> 1) & 3) * 1024 + (T & 1) * 512),
                                           ws + f * 1024, 16, 0, 0);
        // (eight lanes fetch the 128 bytes; like the 32 dword loads of the other layout, one instruction each)
        if (kJoint) {  // (sixteen lanes: 128 bytes of scales, 128 bytes of biases)
          if (op == A_OPS + 1 && lane < 16)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(kn_scales[0] + unit + (lane >> 3) * 1024 + (T & 7) * 128),
                                             ws + 1024, 16, 0, 0);
          continue;
        }
        if (op == A_OPS + FN + f && lane < 8)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(kn_scales[f] + unit + (T & 7) * 128),
                                           ws + FN * 1024 + f * 128, 16, 0, 0);
        if (op == A_OPS + 2 * FN + f && lane < 8)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(kn_scales[f] + unit + 1024 + (T & 7) * 128),
                                           ws + FN * 1152 + f * 128, 16, 0, 0);
      }
      return;
    }
    if (BLOB) {
      const int T = tile0 + t_load;  // K tile of the whole weight; its group of 64 is number T % 8 of the item
      const int64_t item = (int64_t)(T >> 3) * kStreamItem;
#pragma unroll
      for (int f = 0; f < FN; ++f) {
        if (op == A_OPS + f)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(kn_codes[f] + item + ((T >> 1) & 3) * 1024 + (T & 1) * 512),
                                           ws + f * 1024, 16, 0, 0);
        if (kJoint) {
          if (op == A_OPS + 1)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(kn_scales[0] + item + h * 256 + ((T & 7) >> 1) * 4),
                                             ws + 1024, 4, 0, 0);
          continue;
        }
        if (op == A_OPS + FN + f && h == 0)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(kn_scales[f] + item + ((T & 7) >> 1) * 4),
                                           ws + FN * 1024 + f * 128, 4, 0, 0);
        if (op == A_OPS + 2 * FN + f && h == 0)
          __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t *>(kn_scales[f] + item + 256 + ((T & 7) >> 1) * 4),
                                           ws + FN * 1152 + f * 128, 4, 0, 0);
      }
      return;
    }
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      if (op == A_OPS + f) __builtin_amdgcn_global_load_lds(b_src[f] + t_load * 2, ws + f * 1024, 16, 0, 0);
      if (op == A_OPS + FN + f && h == 0)
        __builtin_amdgcn_global_load_lds(s_src[f] + (g >> 1), ws + FN * 1024 + f * 128, 4, 0, 0);
      if (op == A_OPS + 2 * FN + f && h == 0)
        __builtin_amdgcn_global_load_lds(z_src[f] + (g >> 1), ws + FN * 1152 + f * 128, 4, 0, 0);
    }
  };
  auto issue_tile = [&](int t_load, int t_slot) {
#pragma unroll
    for (int op = 0; op < OPS; ++op) issue_op(op, t_load, t_slot);
  };
  // packed words, scale and bias dwords of tile t from this wave's ring (3 FN LDS reads)
  auto read_weights = [&](int t, uint4_t (&wq)[FN], uint32_t (&sw)[FN], uint32_t (&zw)[FN]) {
    const uint32_t ws = w_rd + (t % kWStages) * S::W_STAGE;
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      asm volatile("ds_read_b128 %0, %1" : "=v"(wq[f]) : "v"(ws + f * 1024 + lane * 16));
      if (!KN) {
        asm volatile("ds_read_b32 %0, %1" : "=v"(sw[f]) : "v"(ws + FN * 1024 + f * 128 + fr * 4));
        asm volatile("ds_read_b32 %0, %1" : "=v"(zw[f]) : "v"(ws + FN * 1152 + f * 128 + fr * 4));
      }
    }
  };
  // KN: the scales and biases of the eight input features of MFMA step `step` of tile t (this lane's half h)
  auto read_scales = [&](int t, int step, uint4_t (&sq)[FN], uint4_t (&zq)[FN]) {
    const uint32_t ws = w_rd + (t % kWStages) * S::W_STAGE + h * 64 + step * 16;
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      asm volatile("ds_read_b128 %0, %1" : "=v"(sq[f]) : "v"(ws + FN * 1024 + f * 128));
      asm volatile("ds_read_b128 %0, %1" : "=v"(zq[f]) : "v"(ws + FN * 1152 + f * 128));
    }
  };
  auto half_select = [&](int t) -> uint32_t {
    const int g = ((tile0 + t) * 64 + h * 32) >> gs_shift;
    return (g & 1) ? 0x07060706u : 0x05040504u;
  };

  float16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int f = 0; f < FN; ++f)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][f][e] = 0.f;

  // ---- prologue: tiles 0 and 1 in flight, tile 0 consumed up to the B operand of its first step
  issue_tile(0, 0);
  issue_tile(min(1, n_tiles - 1), 1);
  wait_vmcnt<OPS>();
  __builtin_amdgcn_s_barrier();
  uint4_t wq[FN], a[2][FM];
  uint32_t sw[FN] = {}, zw[FN] = {};
  half2_t s2[FN] = {}, z2[FN] = {};
  half8_t b_cur[FN];
  // KN: two sets of (scales, biases) of one MFMA step each: set [q] serves the steps of parity q of a
  // tile (step 0 is expanded under step 3 of the tile before, step s + 1 under step s), and is
  // fetched a step before it is used
  // (Tiles with four or more A fragments per wave have no registers for two sets: ONE set, fetched
  // at the start of the step whose expansion uses it, with the fmas that need it as the last of the
  // sixteen operations and a counted wait in front of them.)
  constexpr bool kOneSet = FM >= 4;
  uint4_t sq[kOneSet ? 1 : 2][FN] = {}, zq[kOneSet ? 1 : 2][FN] = {};
  read_weights(0, wq, sw, zw);
  if (KN) {
    read_scales(0, 0, sq[0], zq[0]);
    if constexpr (!kOneSet) read_scales(0, 1, sq[1], zq[1]);
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[0][i]) : "v"(a_rd_row + a_rd_chunk[0]), "n"(i * 4096));
  if (KN) {
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      if (kOneSet) asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(wq[f]), "+v"(sq[0][f]), "+v"(zq[0][f]) : "n"(FM));
      else asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(wq[f]), "+v"(sq[0][f]), "+v"(zq[0][f]), "+v"(sq[kOneSet ? 0 : 1][f]), "+v"(zq[kOneSet ? 0 : 1][f]) : "n"(FM));
      DequantState st0;
      dequant_piece_kn<1>(0, wq[f][0], sq[0][f], zq[0][f], km, st0);
      b_cur[f] = dequant_result(st0);
    }
  } else {
    const uint32_t sel = half_select(0);
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(wq[f]), "+v"(sw[f]), "+v"(zw[f]) : "n"(FM));
      s2[f] = as_half2(__builtin_amdgcn_perm(sw[f], sw[f], sel));
      z2[f] = as_half2(__builtin_amdgcn_perm(zw[f], zw[f], sel));
      b_cur[f] = dequant_word_natural(wq[f][0], s2[f], z2[f]);
    }
  }

  constexpr int OPS_PER_GROUP = (OPS + 3 * FM - 1) / (3 * FM);  // loads per MFMA group of steps 0..2
  for (int t = 0; t < n_tiles; ++t) {
    const uint32_t xs = a_rd_row + (t % XS) * S::X_STAGE;
    const int t_ahead = min(t + 2, n_tiles - 1);  // past the end: the last tile again, into dead slots
    // ---- steps 0..2: MFMAs of step s4, A fragments and B operand of step s4 + 1
#pragma unroll
    for (int s4 = 0; s4 < 3; ++s4) {
      DequantState st[FN];
      __builtin_amdgcn_sched_barrier(0);
      wait_lds<0>(a[s4 & 1][FM - 1]);  // issued one step ago
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        if (i + 1 < FM) asm volatile("" : "+v"(a[s4 & 1][i]) : "v"(a[s4 & 1][FM - 1]));
#pragma unroll
        for (int f = 0; f < FN; ++f)
          acc[i][f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a[s4 & 1][i]), b_cur[f],
                                                             acc[i][f], 0, 0, 0);
        asm volatile("ds_read_b128 %0, %1 offset:%2"
                     : "=v"(a[(s4 + 1) & 1][i])
                     : "v"(xs + a_rd_chunk[s4 + 1]), "n"(i * 4096));
        // one load of tile t + 2 per MFMA group: a burst of all of them right after the barrier
        // would block every wave behind the 64 B/clk address path of the compute unit
#pragma unroll
        for (int o = 0; o < OPS_PER_GROUP; ++o)
          if ((s4 * FM + i) * OPS_PER_GROUP + o < OPS) issue_op((s4 * FM + i) * OPS_PER_GROUP + o, t_ahead, t + 2);
        // KN: the scales of step s4 + 2 (of this tile: its ring slot is readable) go into the set that
        // step s4's expansion, which is for step s4 + 1, does not use; they have landed by the next
        // step's wait for this step's fragment reads
        if (KN && i == 0) {
          if (kOneSet) read_scales(t, s4 + 1, sq[0], zq[0]);  // (one set: of the step that is expanded now)
          else if (s4 < 2) read_scales(t, s4 + 2, sq[s4 & 1], zq[s4 & 1]);
        }
        if (KN && kOneSet && i == FM - 2) {
          // the fmas come in the last two groups: the set's reads are older than the FM - 2 fragment reads since
#pragma unroll
          for (int f = 0; f < FN; ++f) asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(sq[0][f]), "+v"(zq[0][f]) : "n"(FM - 2));
        }
#pragma unroll
        for (int f = 0; f < FN; ++f) {
          if (KN && kOneSet) dequant_piece_kn<FM, true>(i, wq[f][s4 + 1], sq[0][f], zq[0][f], km, st[f]);
          else if (KN) dequant_piece_kn<FM>(i, wq[f][s4 + 1], sq[(s4 + 1) & 1][f], zq[(s4 + 1) & 1][f], km, st[f]);
          else dequant_piece<FM>(i, wq[f][s4 + 1], s2[f], z2[f], st[f]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // keep this step's fragments allocated until here: a fragment read for the next step that
      // reused the registers of an MFMA still in flight would have to wait for that MFMA
#pragma unroll
      for (int i = 0; i < FM; ++i) asm volatile("" : : "v"(a[s4 & 1][i]));
#pragma unroll
      for (int f = 0; f < FN; ++f) b_cur[f] = dequant_result(st[f]);
    }
    // ---- step 3: the next tile becomes readable; its first A fragments and B operand are fetched
    //      and built under the MFMAs of this step
    __builtin_amdgcn_sched_barrier(0);
    wait_lds<0>(a[1][FM - 1]);     // this wave's last LDS reads of tile t have landed (issued a step ago)
    wait_vmcnt<OPS>();             // own loads of tile t + 1 (older than the OPS of tile t + 2)
    __builtin_amdgcn_s_barrier();  // everybody's: tile t + 1 is readable, the x stage of tile t is dead
    __builtin_amdgcn_sched_barrier(0);
    uint4_t wq_next[FN];
    read_weights(t + 1, wq_next, sw, zw);
    if (KN) {  // (the expansions that used the two sets are done: the last one ran under step 2)
      read_scales(t + 1, 0, sq[0], zq[0]);
      if constexpr (!kOneSet) read_scales(t + 1, 1, sq[1], zq[1]);
    }
    const uint32_t xs_next = a_rd_row + ((t + 1) % XS) * S::X_STAGE;
    const uint32_t sel_next = KN ? 0u : half_select(t + 1);
    DequantState st[FN];
    half2_t s2n[FN] = {}, z2n[FN] = {};
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if (i + 1 < FM) asm volatile("" : "+v"(a[1][i]) : "v"(a[1][FM - 1]));
#pragma unroll
      for (int f = 0; f < FN; ++f)
        acc[i][f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a[1][i]), b_cur[f], acc[i][f],
                                                           0, 0, 0);
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[0][i]) : "v"(xs_next + a_rd_chunk[0]), "n"(i * 4096));
      if (i == 1) {
        // the weight reads are older than the two fragment reads issued since
#pragma unroll
        for (int f = 0; f < FN; ++f) {
          if (KN) {
            asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(wq_next[f]), "+v"(sq[0][f]), "+v"(zq[0][f]));
            if (!kOneSet) asm volatile("" : "+v"(sq[kOneSet ? 0 : 1][f]), "+v"(zq[kOneSet ? 0 : 1][f]));
          } else {
            asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(wq_next[f]), "+v"(sw[f]), "+v"(zw[f]));
            s2n[f] = as_half2(__builtin_amdgcn_perm(sw[f], sw[f], sel_next));
            z2n[f] = as_half2(__builtin_amdgcn_perm(zw[f], zw[f], sel_next));
          }
        }
      }
      if (i >= 2) {
#pragma unroll
        for (int f = 0; f < FN; ++f) {
          if (KN) dequant_piece_kn<(FM > 2 ? FM - 2 : 1)>(i - 2, wq_next[f][0], sq[0][f], zq[0][f], km, st[f]);
          else dequant_piece<(FM > 2 ? FM - 2 : 1)>(i - 2, wq_next[f][0], s2n[f], z2n[f], st[f]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < FM; ++i) asm volatile("" : : "v"(a[1][i]));
    if (FM == 1) {  // (the weight reads are older than the one fragment read issued since)
#pragma unroll
      for (int f = 0; f < FN; ++f) {
        if (KN) {
          asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(wq_next[f]), "+v"(sq[0][f]), "+v"(zq[0][f]));
          if (!kOneSet) asm volatile("" : "+v"(sq[kOneSet ? 0 : 1][f]), "+v"(zq[kOneSet ? 0 : 1][f]));
        } else {
          asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(wq_next[f]), "+v"(sw[f]), "+v"(zw[f]));
          s2n[f] = as_half2(__builtin_amdgcn_perm(sw[f], sw[f], sel_next));
          z2n[f] = as_half2(__builtin_amdgcn_perm(zw[f], zw[f], sel_next));
        }
      }
    }
    if (FM <= 2) {  // no MFMA group left to hide the expansion behind
#pragma unroll
      for (int f = 0; f < FN; ++f) {
        if (KN) dequant_piece_kn<1>(0, wq_next[f][0], sq[0][f], zq[0][f], km, st[f]);
        else dequant_piece<1>(0, wq_next[f][0], s2n[f], z2n[f], st[f]);
      }
    }
#pragma unroll
    for (int f = 0; f < FN; ++f) {
      b_cur[f] = dequant_result(st[f]);
      wq[f] = wq_next[f];
      s2[f] = s2n[f];
      z2[f] = z2n[f];
    }
  }
  wait_vmcnt<0>();  // surplus prefetches past the last tile
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

  if (KS > 1) {
    // the groups' partial sums meet in LDS (over the rings, which nobody reads any more):
    // [group - 1][wave][accumulator][element][lane], group 0 adds them to its own
    float *red = reinterpret_cast<float *>(lds);
    __builtin_amdgcn_s_barrier();
    if (kgrp > 0) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int f = 0; f < FN; ++f)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            red[((((kgrp - 1) * NW + wave) * FM * FN + i * FN + f) * 16 + e) * 64 + lane] = acc[i][f][e];
    }
    __builtin_amdgcn_s_barrier();
    if (kgrp > 0) return;
#pragma unroll
    for (int g = 1; g < KS; ++g)
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int f = 0; f < FN; ++f)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            acc[i][f][e] += red[((((g - 1) * NW + wave) * FM * FN + i * FN + f) * 16 + e) * 64 + lane];
  }

  if (gridDim.z > 1) {
    // K divided over the workgroups of the tile: their accumulators meet in `partial`
    // ([slab][tile][wave][accumulator][quarter][lane], a float4 each); the last workgroup to arrive
    // (arrival counters, zero before and after every launch) adds them in the order of the slabs.
    // (The waves of the other K groups of this workgroup have left: barriers count the live waves.)
    constexpr int kPerWave = FM * FN * 4;  // float4 per lane
    const int n_splits = gridDim.z, tile = blockIdx.y * gridDim.x + blockIdx.x, n_out_tiles = gridDim.x * gridDim.y;
    float4_t *mine = partial + (((int64_t)blockIdx.z * n_out_tiles + tile) * NW + wave) * (kPerWave * 64) + lane;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const float4_t v = {acc[i][f][4 * q4], acc[i][f][4 * q4 + 1], acc[i][f][4 * q4 + 2], acc[i][f][4 * q4 + 3]};
          asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(mine + ((i * FN + f) * 4 + q4) * 64), "v"(v) : "memory");
        }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the partial sums are in memory before the workgroup counts itself in
    __builtin_amdgcn_s_barrier();
    unsigned *arrived = reinterpret_cast<unsigned *>(lds);
    if (tid == 0) {
      const unsigned before = __hip_atomic_fetch_add(counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (before == (unsigned)n_splits - 1)  // the last one: leave the counter at zero for the next launch
        __hip_atomic_store(counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(arrived, before, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __builtin_amdgcn_s_barrier();
    if (__hip_atomic_load(arrived, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != (unsigned)n_splits - 1) return;
    const float4_t *first = partial + ((int64_t)tile * NW + wave) * (kPerWave * 64) + lane;
    const int64_t stride = (int64_t)n_out_tiles * NW * (kPerWave * 64);  // float4 between consecutive slabs
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int f = 0; f < FN; ++f)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][f][e] = 0.f;
    for (int sp = 0; sp < n_splits; ++sp) {
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        float4_t v[FN * 4];
#pragma unroll
        for (int j = 0; j < FN * 4; ++j)
          asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[j]) : "v"(first + sp * stride + (i * FN * 4 + j) * 64) : "memory");
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int j = 0; j < FN * 4; ++j) asm volatile("" : "+v"(v[j]));  // (uses of v stay below the wait)
#pragma unroll
        for (int f = 0; f < FN; ++f)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][f][e] += v[f * 4 + (e >> 2)][e & 3];
      }
    }
  }

  // D[m][n]: lane holds n = lane % 32 and m = 8 * (e / 4) + 4 * (lane / 32) + e % 4
  // (The lane's position is worked out again from the thread index, through a register the compiler
  // cannot see through: kept from the top of the kernel it would occupy registers across the K loop,
  // which the largest tile does not have.)
  int tid_e = tid;
  asm volatile("" : "+v"(tid_e));
  const int wave_e = (tid_e >> 6) % NW, wm_e = wave_e / WN, wn_e = wave_e % WN, fr_e = tid_e & 31, h_e = (tid_e >> 5) & 1;
  const bool interior = m0 + TILE_M <= m_rows && n0 + TILE_N <= n_out;
#pragma unroll
  for (int f = 0; f < FN; ++f) {
    const int n = n0 + wn_e * TN + f * 32 + fr_e;
    const float ob = (out_bias && n < n_out) ? (float)out_bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      half_t *dst = y + (int64_t)(m0 + wm_e * TM + i * 32 + 4 * h_e) * n_out + n;
      if (interior) {
#pragma unroll
        for (int e = 0; e < 16; ++e)
          dst[(int64_t)(8 * (e >> 2) + (e & 3)) * n_out] = (half_t)apply_activation(acc[i][f][e] + ob, act);
      } else if (n < n_out) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm_e * TM + i * 32 + 8 * (e >> 2) + 4 * h_e + (e & 3);
          if (m < m_rows) y[(int64_t)m * n_out + n] = (half_t)apply_activation(acc[i][f][e] + ob, act);
        }
      }
    }
  }
}



}  // namespace

// (external linkage: their address is taken on the host for hipFuncSetAttribute)
// OCC: waves per SIMD the register budget is sized for (2: 256 registers per lane, 1: 512)
// BLOB: `packed` is the weight in the streaming layout of gq_gemv_prepack_f16 (scale and bias are not read)
template <int WM, int WN, int FM, int FN, int XS, int OCC, int KS, bool BLOB>
__global__ __launch_bounds__(KS * WM * WN * 64, OCC) void gemm_pipe2_kernel(const half_t *x, int m_rows, const uint4_t *packed,
                                                                  const half_t *scale, const half_t *bias,
                                                                  const half_t *out_bias, half_t *y, int n_out,
                                                                  int k_in, int gs_shift, int act, float4_t *partial,
                                                                  unsigned *counters) {
  gemm_pipe2_body<WM, WN, FM, FN, XS, KS, false, BLOB>(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, gs_shift, act,
                                                       partial, counters);
}

// the same pipeline on a weight in the kn streaming layout (groups along the output features)
template <int WM, int WN, int FM, int FN, int XS, int OCC, int KS>
__global__ __launch_bounds__(KS * WM * WN * 64, OCC) void gemm_pipe2_kn_kernel(const half_t *x, int m_rows, const uint4_t *blob,
                                                                     const half_t *out_bias, half_t *y, int n_out, int k_in,
                                                                     int act) {
  gemm_pipe2_body<WM, WN, FM, FN, XS, KS, true>(x, m_rows, blob, nullptr, nullptr, out_bias, y, n_out, k_in, 6, act, nullptr,
                                                nullptr);
}

namespace {

constexpr int kGemmCounters = 4096;  // arrival counters at the start of a workspace (16 KiB), one per output tile

template <bool BLOB, int WM, int WN, int FM, int FN, int XS, int OCC, int KS = 1>
int launch_pipe2(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                 const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in, int gs_shift,
                 int act, int z_splits, void *workspace, hipStream_t stream) {
  using S = Pipe2Shape<WM, WN, FM, FN, XS, KS>;
  constexpr int TILE_M = S::TILE_M, TILE_N = S::TILE_N, lds_bytes = S::LDS_BYTES;
  static_assert(lds_bytes <= 160 * 1024, "LDS budget of a gfx950 compute unit");
  auto kern = gemm_pipe2_kernel<WM, WN, FM, FN, XS, OCC, KS, BLOB>;
  // the attribute belongs to the (function, device) pair; same value every time: a benign race
  constexpr int kMaxDevices = 64;
  static bool configured[kMaxDevices] = {false};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(GQ_ERR_NO_DEVICE, "no current device");
  if (!configured[dev]) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute(lds=%d): %s", lds_bytes, hipGetErrorString(e));
    configured[dev] = true;
  }
  const dim3 grid((unsigned)((n_out + TILE_N - 1) / TILE_N), (unsigned)((m_rows + TILE_M - 1) / TILE_M), (unsigned)z_splits);
  if (grid.y > 65535) return fail(GQ_ERR_UNSUPPORTED, "gq_gemm_f16: m_rows=%lld too large", (long long)m_rows);
  unsigned *counters = static_cast<unsigned *>(workspace);
  float4_t *partial = workspace ? reinterpret_cast<float4_t *>(counters + kGemmCounters) : nullptr;
  kern<<<grid, dim3(KS * WM * WN * 64), lds_bytes, stream>>>(
      reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const uint4_t *>(packed),
      reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
      reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, gs_shift, act, partial,
      counters);
  return check_launch("gemm_pipe2_kernel");
}

template <int WM, int WN, int FM, int FN, int XS, int OCC, int KS = 1>
int launch_pipe2_kn(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                    int64_t k_in, int act, hipStream_t stream) {
  using S = Pipe2Shape<WM, WN, FM, FN, XS, KS>;
  constexpr int TILE_M = S::TILE_M, TILE_N = S::TILE_N, lds_bytes = S::LDS_BYTES;
  auto kern = gemm_pipe2_kn_kernel<WM, WN, FM, FN, XS, OCC, KS>;
  constexpr int kMaxDevices = 64;
  static bool configured[kMaxDevices] = {false};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(GQ_ERR_NO_DEVICE, "no current device");
  if (!configured[dev]) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute(lds=%d): %s", lds_bytes, hipGetErrorString(e));
    configured[dev] = true;
  }
  const dim3 grid((unsigned)((n_out + TILE_N - 1) / TILE_N), (unsigned)((m_rows + TILE_M - 1) / TILE_M), 1u);
  if (grid.y > 65535) return fail(GQ_ERR_UNSUPPORTED, "gq_linear_knp_act_f16: m_rows=%lld too large", (long long)m_rows);
  kern<<<grid, dim3(KS * WM * WN * 64), lds_bytes, stream>>>(
      reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const uint4_t *>(blob),
      reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, act);
  return check_launch("gemm_pipe2_kn_kernel");
}

}  // namespace

namespace {

// The tile shape and the number of workgroups that divide K for one output tile.
//
// Five tile shapes.  The larger the tile, the less x and weight traffic per multiply-add, but a
// launch is as slow as its busiest compute unit: expected time = workgroups per compute unit (256 of
// them; a last, partly filled round runs faster: fewer workgroups share memory and clocks) x time
// per workgroup, from measured times per 1024 input features with every compute unit busy:
//   64 x 64    6.3 us  (two groups of four waves of 32 x 32 that split K; needs k_in % 256 == 0)
//   128 x 64   8 us    (16384 x 4096 at 128 rows: 34.5 us)
//   256 x 128  22 us   (16384 x 4096 at 512 rows: 87 us; 16 us with an eighth of the compute units busy)
//   256 x 256  34 us   (16384 x 4096 at 2048 rows: two rounds, 271 us; at 1024 rows one, 140 us)
//   128 x 256  22 us   (eight waves of 128 x 32; 20.7 us for a weight in a streaming layout)
// Fixed thresholds on the batch alone (256 x 128 from 256 rows, 256 x 256 from 1024) left weights
// with 4096 outputs on 16 to 64 workgroups: 4096 x 4096 at 512 rows took 75.6 us, now 36 us.  With each
// shape forced in turn, this choice was the fastest or within 2 % of it for five weight shapes
// (16384 x 4096, 4096 x 16384, 4096 x 4096, 12288 x 4096, 8192 x 8192) at nine batches from 128 to 4096.
//
// 128 x 256 has the output area of 256 x 128 on twice the waves (two per SIMD hide each other's waits)
// at twice the expansion work per multiply-add.  It wins where it wastes fewer rows (16384 x 4096 at
// 384 rows: 192 workgroups instead of 256 with a quarter of their rows unused, 74.2 against 88.6 us,
// from the streaming layout 62.4 against 83.7) and, on a weight in a streaming layout, whose loads
// are whole KiB, also at the same number of workgroups (16384 x 4096 at 512 rows 76.5 against 81.5 us,
// 12288 x 4096 61.5 against 73.3; on the three variables 87.2 against 86.6 and 73.5 against 76.0: a
// tie goes to 256 x 128 there).  K is not divided over workgroups with this shape, so that the
// workspace a caller sized without knowing of a streaming-layout copy serves either choice.
//
// With a workspace, 2 to 16 workgroups may divide the K loop of a tile (each at least four steps of
// 64) and add their fp32 accumulators through it: priced at 4 us plus the partial sums written and
// read at 5 TB/s.
struct GemmPlan {
  int shape;   // 0: 64 x 64, 1: 128 x 64, 2: 256 x 128, 3: 256 x 256, 4: 128 x 256
  int splits;  // workgroups per output tile
  int64_t tiles, tile_bytes;
  double us;   // expected time
};

// `streamed`: the weight is read from a streaming-layout copy.
GemmPlan plan_gemm(int64_t m_rows, int64_t n_out, int64_t k_in, bool may_split, bool streamed) {
  static const int tile_m[5] = {64, 128, 256, 256, 128}, tile_n[5] = {64, 64, 128, 256, 256};
  const double us_per_1024[5] = {6.3, 8.0, 22.0, 34.0, streamed ? 20.7 : 22.0};
  static const int order[5] = {3, 2, 4, 1, 0};  // (ties go to the earlier one)
  GemmPlan best = {1, 1, 0, 0, 1e30};
  for (int o = 0; o < 5; ++o) {
    const int shape = order[o];
    if (shape == 0 && k_in % 256 != 0) continue;
    const int groups = (shape <= 1 && k_in % 256 == 0) ? 2 : 1;  // groups of waves that split K inside a workgroup
    const int64_t tiles = ((m_rows + tile_m[shape] - 1) / tile_m[shape]) * ((n_out + tile_n[shape] - 1) / tile_n[shape]);
    for (int splits = 1; splits <= (may_split && shape != 4 ? 16 : 1); splits *= 2) {
      const int64_t steps = k_in / 64;
      if (steps % (groups * splits) != 0 || steps / (groups * splits) < 4 || (splits > 1 && tiles > kGemmCounters)) break;
      const int64_t wgs = tiles * splits, full = wgs / 256, rest = wgs % 256;
      const int64_t tile_bytes = (int64_t)tile_m[shape] * tile_n[shape] * 4;
      double t = ((double)full + (rest ? 0.7 + 0.3 * (double)rest / 256.0 : 0.0)) * us_per_1024[shape] * (double)k_in /
                 (1024.0 * splits);
      if (splits > 1) t += 4.0 + 2.0 * (double)(wgs * tile_bytes) / 5.0e6;
      if (t < best.us) best = GemmPlan{shape, splits, tiles, tile_bytes, t};
    }
  }
  return best;
}

bool gemm_pipelined_ok(const uint16_t *x, const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, int64_t k_in,
                       int64_t group_size) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  if (!(pow2 && group_size >= 32 && k_in % BK == 0 && k_in > 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)packed % 16) == 0))
    return false;
  // the pipelined kernel fetches scale and bias as aligned dwords (two groups at a time)
  return (k_in / group_size) % 2 == 0 && ((uintptr_t)scale % 4) == 0 && ((uintptr_t)bias % 4) == 0;
}

}  // namespace

// What the choice above expects the pipelined kernel to take (us) -- for callers that weigh it against
// other ways of running a batch.
double gemm_expected_us(int64_t m_rows, int64_t n_out, int64_t k_in, bool may_split) {
  return plan_gemm(m_rows, n_out, k_in, may_split, false).us;
}

// Bytes of workspace with which launch_gemm may divide K over workgroups (0: it would not): 16 KiB of
// arrival counters, then the fp32 accumulators of every (slab, tile).  (Pointer alignment is the
// caller's to meet: this is the figure for 16-byte aligned operands.)
int64_t gemm_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  if (m_rows < 1 || n_out < 1 || !pow2 || group_size < 32 || k_in <= 0 || k_in % BK != 0 || (k_in / group_size) % 2 != 0) return 0;
  const GemmPlan plan = plan_gemm(m_rows, n_out, k_in, true, false);
  return plan.splits == 1 ? 0 : (int64_t)kGemmCounters * 4 + plan.splits * plan.tiles * plan.tile_bytes;
}

// `workspace`: NULL, or gemm_workspace_bytes() bytes of device memory whose first 16 KiB (the counters)
// are zero; the kernel leaves them zero.
// `blob`: NULL, or the same weight in the streaming layout of gq_gemv_prepack_f16 (group_size 64, k_in % 512 == 0,
// 16-byte aligned: the caller has checked); the pipelined kernel then reads it instead of the three variables.
int launch_gemm(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, int act, void *workspace, hipStream_t stream, const void *blob) {
  const bool pow2 = (group_size & (group_size - 1)) == 0;
  const bool fast_ok = pow2 && group_size >= 32 && k_in % BK == 0 && k_in > 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)packed % 16) == 0;
  if (!fast_ok)
    return launch_gemv_generic_rows(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, act, stream);
  const int gs_shift = __builtin_ctzll((unsigned long long)group_size);
#define GQ_PIPE2(WM, WN, FM, FN, XS, OCC, ...)                                                                              \
  (blob ? launch_pipe2<true, WM, WN, FM, FN, XS, OCC, ##__VA_ARGS__>(x, m_rows, static_cast<const uint16_t *>(blob), nullptr,    \
                                                                     nullptr, out_bias, y, n_out, k_in, gs_shift, act,           \
                                                                     plan.splits, plan.splits > 1 ? workspace : nullptr, stream) \
        : launch_pipe2<false, WM, WN, FM, FN, XS, OCC, ##__VA_ARGS__>(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in,  \
                                                                      gs_shift, act, plan.splits,                                \
                                                                      plan.splits > 1 ? workspace : nullptr, stream))
  if (gemm_pipelined_ok(x, packed, scale, bias, k_in, group_size)) {
    const GemmPlan plan = plan_gemm(m_rows, n_out, k_in, workspace != nullptr, blob != nullptr);
    if (plan.shape == 0) return GQ_PIPE2(2, 2, 1, 1, 3, 2, 2);  // 64 x 64, two groups of 4 waves of 32 x 32
    if (plan.shape == 4) return GQ_PIPE2(1, 8, 4, 1, 4, 1);     // 128 x 256, 8 waves of 128 x 32
    if (plan.shape == 3) return GQ_PIPE2(1, 8, 8, 1, 4, 2);     // 256 x 256, 8 waves of 256 x 32
    if (plan.shape == 2) return GQ_PIPE2(1, 4, 8, 1, 3, 1);     // 256 x 128, 4 waves of 256 x 32
    // 128 x 64 (a workgroup on every compute unit at n_out = 16384), 4 waves of 64 x 32; two such
    // groups of waves split K when the K tiles divide between them (and the scale / bias dwords)
    if (k_in % 256 == 0) return GQ_PIPE2(2, 2, 2, 1, 3, 1, 2);
    return GQ_PIPE2(2, 2, 2, 1, 3, 2);
  }
#undef GQ_PIPE2
  const dim3 grid((unsigned)((n_out + BN - 1) / BN), (unsigned)((m_rows + BM - 1) / BM));
  if (grid.y > 65535) return fail(GQ_ERR_UNSUPPORTED, "gq_gemm_f16: m_rows=%lld too large", (long long)m_rows);
  gemm_tile_kernel<<<grid, dim3(256), 0, stream>>>(
      reinterpret_cast<const half_t *>(x), (int)m_rows, reinterpret_cast<const uint4_t *>(packed),
      reinterpret_cast<const half_t *>(scale), reinterpret_cast<const half_t *>(bias),
      reinterpret_cast<const half_t *>(out_bias), reinterpret_cast<half_t *>(y), (int)n_out, (int)k_in, gs_shift, act);
  return check_launch("gemm_tile_kernel");
}

// Prefill batches on a weight in the kn streaming layout (n_out % 64 == 0, k_in % 512 == 0, x and the blob
// 16-byte aligned: the caller has checked): the pipelined kernel with the tile shape that plan_gemm
// chooses for the other layout (K is not divided over workgroups: no workspace here).
int launch_gemm_knp(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                    int64_t k_in, int act, hipStream_t stream) {
  const GemmPlan plan = plan_gemm(m_rows, n_out, k_in, false, true);
#define GQ_PIPE2_KN(WM, WN, FM, FN, XS, OCC, ...) \
  launch_pipe2_kn<WM, WN, FM, FN, XS, OCC, ##__VA_ARGS__>(x, m_rows, blob, out_bias, y, n_out, k_in, act, stream)
  if (plan.shape == 0) return GQ_PIPE2_KN(2, 2, 1, 1, 3, 2, 2);
  if (plan.shape == 4) return GQ_PIPE2_KN(1, 8, 4, 1, 4, 1);
  if (plan.shape == 3) return GQ_PIPE2_KN(1, 8, 8, 1, 4, 2);
  if (plan.shape == 2) return GQ_PIPE2_KN(1, 4, 8, 1, 3, 1);
  return GQ_PIPE2_KN(2, 2, 2, 1, 3, 1, 2);
#undef GQ_PIPE2_KN
}

}  // namespace gq
