// The data-flow kernel of the GEMV sequence: a persistent kernel for launches whose weights are in
// the streaming layout and whose dependencies all travel through the exchange (a decoder's layer
// stack at batch 1; the arithmetic is laid out for up to four batch rows, but measured at batch 4
// the LDS-ring kernel is faster, so only one row is instantiated).  The LDS-ring kernel of
// gq_gemv_stream.hip serves everything else.
//
// Why a second kernel: a stack of dependent GEMVs stalls at every layer boundary (the next layer
// needs every output of this one), and a stall only costs nothing if the weights keep streaming
// into a buffer meanwhile AND the arithmetic then catches up faster than memory delivers.  This
// kernel is built for few instructions per byte: 16 waves per compute unit (four per SIMD), a work
// unit of 16 weight rows x 256 input features (2304 bytes: three direct-to-LDS loads into a
// three-slot ring per wave, 110 KiB per compute unit in flight or buffered, issued across entry
// boundaries -- weights never depend on results), and no staging of x at all.
//
// Arithmetic (v_mfma_f32_16x16x32_f16, one per 512 weights).  B operand = raw codes: the nibble
// or-ed into the mantissa of 64.0 or 1024.0, five VALU instructions per eight weights; the offsets
// are taken out of the accumulator before the first product (it starts at -sum off_k x_k), scale
// and bias are applied to GROUP SUMS.  A operand = x, laid out so that one accumulator separates the
// four groups of a unit and up to four batch rows: A row i = (group g = i >> 2, batch row m = i & 3)
// holds x[m] on the 64 features of group g and zero elsewhere.  The two 1 KiB loads of a unit
// (128 features each) share their four A registers and have an accumulator each; a row is valid
// in the accumulator of the load its group lies in.  Lane (n, kc) -- weight row n, 32-feature
// slice kc -- finds in the accumulator registers e the rows 4 kc + e = (group kc, batch row e): the
// group whose scale and bias it reads as two 16-bit LDS loads.  sum x and sum off x per row come
// out of eight MFMAs against constant B operands, in the same registers.
//
// x comes straight from memory into the A registers: 64 contiguous bytes per active lane, 8 lanes
// per batch row.  Results that a later entry of the launch reads travel through the exchange in
// the form the consumer wants: the fp16 bits of -y (zero as -0.0: an all-zero word means "not
// written yet"; the sign is taken out again where the sums leave the wave), eight at a time in the
// order (0,4,1,5,2,6,3,7) in which the raw codes of a 32-bit word come out.  A wave polls exactly
// the 256 features it multiplies, so a dependency is between 16 producing workgroups and one wave,
// not a barrier of the device; nothing is reported, counted or flushed.
//
// What a dependency costs is decided by how early its data is published, not by how fast it is
// polled: a result travels about 2 us, the waves of a workgroup finish an entry over about 4 us,
// and a wave that finds its x missing is sent on at another time than its neighbours.  So an
// entry that a later one reads publishes its first row blocks while its last ones still stream
// (kEarlyRows below), and the entries of a layer are best ordered so that every reader has
// another entry's worth of units between it and its producer.
#include "gq_gemv_sequence.h"

namespace gq {
namespace {

// cache policy of the weight loads: every byte is read once per launch (0.5 to 1.5 % of a pass
// against the default policy)
#define GQ_FLOW_WEIGHT_POLICY " nt"
constexpr int kFlowWaves = 16;
constexpr int kFlowThreads = kFlowWaves * 64;
constexpr int kUnitBytes = 2048 + 256;  // two 1 KiB loads of packed words; 32 words of scales, 32 of biases
constexpr int kFlowPR = 4;              // row blocks per pass at most (their running sums stay in registers)
// An entry whose results a later entry of the launch reads, and that has kEarlyMinBlocks row blocks
// or more in a workgroup, passes them on kEarlyRows row blocks at a time (a reduction each) instead
// of all at the end.  The reader's first pieces are the producer's first row blocks: they are then
// on their way while the rest of the producer still streams, and the reader's waves do not
// meet a wait that sends them on at different times.  Measured on the 6B decoder stack (up feeds
// down, four row blocks a workgroup): 693 -> 627 us a pass with two row blocks at a time; 674 us
// with one at a time (a reduction costs more than it gains there), 672 us with three and one,
// 650 us if the three row blocks of the fused q, k, v are split as well.
constexpr int kEarlyRows = 2, kEarlyMinBlocks = 4;
// A ring slot also has room for the 256 values of x that its unit multiplies (512 bytes): they are
// requested one unit ahead, in front of the weight loads issued at the same time, and in the order
// of the wave's loads they arrive before that unit -- no wait for x drains the ring.
constexpr int flow_slot_bytes(int) { return kUnitBytes + 512; }
// ring slots per wave and sets of mailboxes, by batch capacity (160 KiB of LDS)
constexpr int flow_depth(int) { return 3; }
constexpr int flow_sets(int) { return 2; }

struct FlowEntry {  // what the kernel needs of an entry, in LDS
  // the 16 bytes the work loop reads per entry, as one LDS read
  int k_in;
  int x_word;        // where x starts in the exchange (-1: in memory at x)
  short nrb, x_src;  // row blocks of this workgroup; producer of x in this launch (-1: none)
  short x_id;        // the first entry of the launch that reads the same x (same values at the same place)
  char m_rows, act;
  const char *blob;
  const half_t *x, *out_bias;
  half_t *y;
  int n_out;
  int ex_word;  // where the results go in the exchange (-1: nowhere)
  int pad[2];
};
static_assert(sizeof(FlowEntry) == 64 && offsetof(FlowEntry, blob) == 16, "entry cache layout");
struct FlowHot {  // the first 16 bytes of a FlowEntry, wave-uniform
  int k_in, x_word, nrb, x_src, x_id, m_rows;
  int pr;  // row blocks per pass
};
constexpr int kEarlyBit = 0x40;  // in the m_rows byte: kEarlyRows row blocks per pass

struct FlowControl {
  unsigned deposited[2];  // mailbox deposits into the set since it was last emptied
  unsigned reduced[2];    // reductions done on the set
  unsigned failed;        // a wave gave up waiting
  unsigned stored;        // entries whose results this workgroup has stored (stores issued)
  unsigned waves_done;
  unsigned half;          // the half of the exchange this launch uses
  unsigned pad[8];
  unsigned zeros[16];     // what the lanes of an A row without data read
};
static_assert(sizeof(FlowControl) == 128, "control block");

template <int MC>
constexpr int flow_lds_bytes() {
  return kFlowWaves * flow_depth(MC) * flow_slot_bytes(MC) + kMaxEntries * (int)sizeof(FlowEntry) +
         flow_sets(MC) * kFlowWaves * kFlowPR * MC * 16 * 4 + (int)sizeof(FlowControl);
}

typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));

// raw_codes() of the other kernel without inline assembly: the compiler's hazard recogniser does
// not look into assembly -- here only part of an accumulator is live at batch 1, the register
// allocator re-uses the rest for the next B operand, and a VALU write to a register that an MFMA in
// flight is still going to write needs wait states that only the compiler can place.  The masks
// and magic numbers come in vector registers the compiler cannot see through, which is what makes
// it select v_and_or_b32 (as literals they would cost a v_and and a v_or each).
__device__ __forceinline__ half8_t raw_codes_c(uint32_t w, uint32_t mask_lo, uint32_t mask_hi, uint32_t magic_lo,
                                               uint32_t magic_hi) {
  const uint32_t hi = w >> 8;
  uint4_t v;
  v.x = (hi & mask_hi) | magic_hi;  // codes 0, 4: 64 + c
  v.y = (hi & mask_lo) | magic_lo;  // codes 1, 5: 1024 + c
  v.z = (w & mask_hi) | magic_hi;   // codes 2, 6: 64 + c
  v.w = (w & mask_lo) | magic_lo;   // codes 3, 7: 1024 + c
  return __builtin_bit_cast(half8_t, v);
}

// EARLY: some entry of the launch passes its results on in parts (else the row blocks per pass are a
// constant of the code: 85 fewer scalar registers spilled, 18 % fewer vector instructions)
template <int MC, bool EARLY>
__device__ __forceinline__ void flow_body(const Entry *__restrict__ entries, int n_entries, int *__restrict__ status,
                                          unsigned *words, unsigned spin_limit, const SequencePlan *plan) {
  constexpr int D = flow_depth(MC), S = flow_sets(MC), PR = kFlowPR;
  constexpr int kSlot = flow_slot_bytes(MC);
  constexpr int kMail = PR * MC * 16;  // floats a wave deposits per pass: [row block][m][n]
  extern __shared__ __attribute__((aligned(64))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int n = lane & 15, kc = lane >> 4;
  const int G = gridDim.x, b = blockIdx.x;
  char *const ring = lds + wave * (D * kSlot);
  FlowEntry *const cache = reinterpret_cast<FlowEntry *>(lds + kFlowWaves * D * kSlot);
  float *const mail = reinterpret_cast<float *>(lds + kFlowWaves * D * kSlot + kMaxEntries * sizeof(FlowEntry));
  FlowControl *const ctl = reinterpret_cast<FlowControl *>(mail + S * kFlowWaves * kMail);

  for (int i = tid; i < n_entries; i += kFlowThreads) {
    const Entry e = entries[i];
    FlowEntry c;
    c.blob = reinterpret_cast<const char *>(e.packed);
    c.x = e.x;
    c.out_bias = e.out_bias;
    c.y = e.y;
    c.n_out = e.n_out;
    c.k_in = e.k_in;
    c.x_word = plan->x_word[i];
    c.ex_word = plan->ex_word[i];
    c.x_src = plan->x_src[i];
    const int rb = (e.n_out + 15) >> 4;
    c.nrb = (short)(rb > b ? (rb - b + G - 1) / G : 0);
    const bool early = EARLY && plan->ex_word[i] >= 0 && c.nrb >= kEarlyMinBlocks;
    c.m_rows = (char)(e.m_rows | (early ? kEarlyBit : 0));
    c.act = (char)e.activation;
    c.x_id = plan->x_id[i];
    c.pad[0] = c.pad[1] = 0;
    cache[i] = c;
  }
  if (tid == 0) {
    const unsigned epoch = __hip_atomic_load(words + kFlowEpochWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *ctl = FlowControl{{0u, 0u}, {0u, 0u}, 0u, 0u, 0u, epoch & 1u, {}, {}};
  }
  __syncthreads();
  const unsigned half = (unsigned)uni((int)ctl->half);
  unsigned short *const ex_all = reinterpret_cast<unsigned short *>(words + kFlowExchangeWord);
  unsigned short *const ex16 = ex_all + (size_t)half * kFlowHalfValues;
  {
    // what the launch before this one left in the other half (that launch is complete; the one after
    // this one, which will use that half, starts when these stores are)
    const unsigned dirty = __hip_atomic_load(words + kFlowExtentWord + (1u - half), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint4_t *other = reinterpret_cast<uint4_t *>(ex_all + (size_t)(1u - half) * kFlowHalfValues);
    for (unsigned i = (unsigned)b * kFlowThreads + tid; i < dirty / 8; i += (unsigned)G * kFlowThreads)
      other[i] = uint4_t{0u, 0u, 0u, 0u};
  }
  // (nothing the compiler knows of is pending when the work loop starts: it would guard registers
  // against those loads on every trip, with a wait for ALL loads of the ring)
  wait_vm<0>();

  // ---- lane constants
  const uint32_t ring_rd = (uint32_t)(uintptr_t)ring;
  const uint32_t lane16 = (uint32_t)lane * 16u, lane4 = (uint32_t)lane * 4u;
  const int hpar = wave & 1;  // which half of a 4608-byte block of the streaming layout this wave's units are
  // the scales and biases of a unit: lanes 0..31 fetch the 32-bit words (row l >> 1, pair l & 1) of the
  // block's scales that belong to this half, lanes 32..63 those of its biases (the instruction
  // adds its offset, 2048, to both the address and the place in the slot)
  const uint32_t sb_fetch = 2048u - hpar * 2048u + (uint32_t)(lane >> 5) * 256u + (uint32_t)((lane & 31) >> 1) * 16u + hpar * 8u +
                            (uint32_t)(lane & 1) * 4u;
  // ... and where lane (n, kc) finds the scale of (row n, group kc) among them; its bias 128 bytes on
  const uint32_t sb_read = (uint32_t)(2 * n + (kc >> 1)) * 4u + (uint32_t)(kc & 1) * 2u;
  uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x00F000F0u, kMagicLo = 0x64006400u, kMagicHi = 0x54005400u;
  asm volatile("" : "+v"(kMaskLo), "+v"(kMaskHi), "+v"(kMagicLo), "+v"(kMagicHi));
  // A row of this lane: group a_g of the unit, batch row a_m; its slice kc lies in that group or not
  const int a_g = n >> 2, a_m = n & 3;
  const bool a_match = (kc >> 1) == (a_g & 1);
  const int a_off = a_g * 64 + (kc & 1) * 32;  // first feature (within the unit's 256) of this lane's 32

  // what lane (row i, slice kc) of the A operand reads of a unit's 512 bytes of x in a ring slot; a lane
  // without data reads zeros
  const uint32_t zeros_rd = (uint32_t)(uintptr_t)ctl->zeros;
  const uint32_t xa_rd = kUnitBytes + (uint32_t)a_off * 2u;
  const bool a_lane = a_match && a_m == 0;  // (batch 1)

  // the hot 16 bytes of entry d as they come out of LDS, and made wave-uniform
  auto read_hot = [&](int d) { return *reinterpret_cast<const uint4_t *>(&cache[d]); };
  auto uniform_hot = [&](uint4_t v) {
    FlowHot h;
    h.k_in = uni((int)v.x);
    h.x_word = uni((int)v.y);
    const int z = uni((int)v.z), w = uni((int)v.w);
    h.nrb = (short)(z & 0xFFFF);
    h.x_src = (short)(z >> 16);
    h.x_id = (short)(w & 0xFFFF);
    h.m_rows = (w >> 16) & 0x3F;
    h.pr = EARLY && ((w >> 16) & kEarlyBit) ? kEarlyRows : kFlowPR;
    return h;
  };

  // ---- the producer: walks this wave's units D ahead of the consumer; all of it wave-uniform
  struct Walk {
    int d, pass, hcp, j;  // entry, pass of row blocks, this wave's how-manieth 256-feature piece, row block in pass
    int nrb, n_hc, nj, chunks, pr;
    const char *blob;
  };
  auto enter = [&](Walk &w) {  // first unit of entry w.d (n_hc == 0 or nrb == 0: none)
    w.pass = w.hcp = w.j = 0;
    w.nrb = w.n_hc = w.nj = 0;
    if (w.d >= n_entries) return;
    const FlowHot h = uniform_hot(read_hot(w.d));
    w.nrb = h.nrb;
    const int k_in = h.k_in;
    w.chunks = k_in >> 9;
    const int pieces = k_in >> 8;
    w.n_hc = wave < pieces ? (pieces - wave + kFlowWaves - 1) / kFlowWaves : 0;
    w.pr = h.pr;
    w.nj = min(w.pr, w.nrb);
    w.blob = uni_ptr(cache[w.d].blob);
  };
  auto next_entry = [&](Walk &w) {
    do {
      ++w.d;
      enter(w);
    } while (w.d < n_entries && (w.n_hc == 0 || w.nrb == 0));
  };
  auto advance = [&](Walk &w) {
    if (++w.j < w.nj) return;
    w.j = 0;
    if (++w.hcp < w.n_hc) return;
    w.hcp = 0;
    ++w.pass;
    w.nj = min(w.pr, w.nrb - w.pass * w.pr);
    if (w.nj > 0) return;
    next_entry(w);
  };
  // where the x of entry d starts, in the form the A operand wants or not
  auto x_row = [&](int d) -> const char * {
    const int x_word = uni(cache[d].x_word);
    return x_word >= 0 ? reinterpret_cast<const char *>(ex16 + x_word) : uni_ptr(cache[d].x);
  };
  // piece hc of x into the x part of a ring slot (two loads of 256 bytes)
  auto issue_x = [&](const char *xrow, int hc, int slot) {
    const char *src = xrow + hc * 512;
    const uint32_t dst = ring_rd + (uint32_t)slot * kSlot + kUnitBytes;
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %1, %2 sc1\n\t"
        "global_load_lds_dword %1, %2 offset:256 sc1"
        :
        : "s"(dst), "v"(lane4), "s"(src)
        : "memory");
  };
  auto issue = [&](const Walk &w, int slot) {
    const int64_t block = (int64_t)(b + (w.pass * w.pr + w.j) * G) * w.chunks + (wave >> 1) + 8 * w.hcp;
    const char *src = w.blob + block * (2 * kUnitBytes) + hpar * 2048;
    const uint32_t dst = ring_rd + (uint32_t)slot * kSlot;
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %3" GQ_FLOW_WEIGHT_POLICY "\n\t"
        "global_load_lds_dwordx4 %1, %3 offset:1024" GQ_FLOW_WEIGHT_POLICY "\n\t"
        "global_load_lds_dword %2, %3 offset:2048" GQ_FLOW_WEIGHT_POLICY
        :
        : "s"(dst), "v"(lane16), "v"(sb_fetch), "s"(src)
        : "memory");
  };

  Walk prod;
  prod.d = -1;
  prod.blob = nullptr;
  prod.chunks = 0;
  next_entry(prod);
  int ahead = 0;  // units issued and not yet consumed
  while (ahead < D && prod.d < n_entries) {
    issue(prod, ahead);
    ++ahead;
    advance(prod);
  }
  int slot = 0;    // ring slot of the consumer's unit
  unsigned q = 0;  // passes so far (the same count in every wave)

  // ---- the A registers and what they hold
  half8_t xa[4];
  float4_t negcorr = {0.f, 0.f, 0.f, 0.f}, xsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < 4; ++w) xa[w] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  int key_id = -1, key_hc = -1;  // the piece of x they hold
  bool x_requested = false;      // the x of the next unit is on its way into that unit's slot
  int g1 = 3, g2 = 3;            // loads in the groups issued with the unit before the last, and with the last

  auto give_up = [&]() {
    if (lane == 0) {
      __hip_atomic_store(&ctl->failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (status) __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  // a value that has not arrived is a zero half-word
  auto any_missing = [&](const uint4_t (&t)[4], bool active) {
    ushort2_t lo = __builtin_bit_cast(ushort2_t, t[0][0]);
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int c = 0; c < 4; ++c) lo = __builtin_elementwise_min(lo, __builtin_bit_cast(ushort2_t, t[w][c]));
    return __builtin_amdgcn_ballot_w64(active && (lo[0] == 0 || lo[1] == 0)) != 0;
  };
  // x in memory order -> the form of the exchange: sign flipped, eight at a time in the order of the raw codes
  auto to_exchange_form = [&](uint4_t (&t)[4]) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint4_t f = t[w];
#pragma unroll
      for (int c = 0; c < 4; ++c) f[c] ^= 0x80008000u;
      t[w] = __builtin_bit_cast(uint4_t, permute_x(f));
    }
  };
  // per A row: -sum off_k x_k (where every accumulator starts) and sum x_k, off = 64 or 1024 as the
  // raw codes of a word come out: (64 + c, 64 + c, 1024 + c, 1024 + c) twice
  auto finish_build = [&](const uint4_t (&t)[4]) {
#pragma unroll
    for (int w = 0; w < 4; ++w) xa[w] = __builtin_bit_cast(half8_t, t[w]);
    const half8_t neg_off = {(half_t)-64.f, (half_t)-64.f, (half_t)-1024.f, (half_t)-1024.f,
                             (half_t)-64.f, (half_t)-64.f, (half_t)-1024.f, (half_t)-1024.f};
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    negcorr = float4_t{0.f, 0.f, 0.f, 0.f};
    xsum = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      negcorr = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[w], neg_off, negcorr, 0, 0, 0);
      xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[w], ones, xsum, 0, 0, 0);
    }
  };
  // nothing can have arrived from everywhere before this workgroup's own share (if it has one) is stored
  auto wait_own_share = [&](int x_src) {
    // (an entry that passes its results on in parts has what this wave needs before its last part)
    if (uni(cache[x_src].nrb) > 0 && !(uni((int)cache[x_src].m_rows) & kEarlyBit))
      while (lds_load(&ctl->stored) <= (unsigned)x_src && !lds_load(&ctl->failed)) __builtin_amdgcn_s_sleep(1);
  };

  // batch 1, a unit that brought x along found values that their producer had not delivered when
  // they were fetched: fetch the piece again until it is complete (these loads are the youngest of
  // the wave: everything in its ring lands with them)
  // The units behind this one in the ring that bring further pieces of the same x along (an entry
  // with several pieces per wave) fetched theirs at about the same time: they are fetched again with it.
  auto refetch = [&](int s, int d, int hc, uint32_t xat, uint4_t (&t)[4], int x_src) {
    if (x_src >= 0) wait_own_share(x_src);
    const unsigned polls_allowed = spin_limit >> 4;  // (a poll is a memory round trip)
    unsigned polls = 0;
    for (;;) {
      issue_x(x_row(d), hc, s);
      wait_vm<0>();
      asm volatile(
          "ds_read_b128 %0, %4\n\t"
          "ds_read_b128 %1, %4 offset:16\n\t"
          "ds_read_b128 %2, %4 offset:32\n\t"
          "ds_read_b128 %3, %4 offset:48\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(t[0]), "=&v"(t[1]), "=&v"(t[2]), "=&v"(t[3])
          : "v"(xat)
          : "memory");
      if (x_src < 0 || !any_missing(t, a_lane)) break;
      if (polls++ >= polls_allowed || lds_load(&ctl->failed)) {  // some workgroup is not running: give up
        give_up();
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
  };

  // one unit: ring slot -> registers -> 8 MFMAs -> this lane's group sums into tot.  fresh (batch 1):
  // the unit brought another piece of x along; it goes into the A registers first, and its sums are
  // taken while the unit's products run
  auto consume = [&](int s, float (&tot)[MC], bool fresh, bool requested, int d, int hc, int x_word, int x_src) {
    const uint32_t at = ring_rd + (uint32_t)s * kSlot;
    uint4_t w0, w1;
    uint32_t sc, bi;
    if (fresh) {
      const uint32_t xat = a_lane ? at + xa_rd : zeros_rd;
      uint4_t t[4];
      asm volatile(
          "ds_read_b128 %4, %10\n\t"
          "ds_read_b128 %5, %10 offset:16\n\t"
          "ds_read_b128 %6, %10 offset:32\n\t"
          "ds_read_b128 %7, %10 offset:48\n\t"
          "ds_read_b128 %0, %8\n\t"
          "ds_read_b128 %1, %8 offset:1024\n\t"
          "ds_read_u16 %2, %9 offset:2048\n\t"
          "ds_read_u16 %3, %9 offset:2176\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(w0), "=&v"(w1), "=&v"(sc), "=&v"(bi), "=&v"(t[0]), "=&v"(t[1]), "=&v"(t[2]), "=&v"(t[3])
          : "v"(at + lane16), "v"(at + sb_read), "v"(xat)
          : "memory");
      const bool from_exchange = x_word >= 0;
      // (not requested: the first unit of the launch, or an entry after one without work for this wave)
      if (!requested || (from_exchange && any_missing(t, a_lane))) refetch(s, d, hc, xat, t, from_exchange ? x_src : -1);
      if (!from_exchange) to_exchange_form(t);
      finish_build(t);
    } else {
      asm volatile(
          "ds_read_b128 %0, %4\n\t"
          "ds_read_b128 %1, %4 offset:1024\n\t"
          "ds_read_u16 %2, %5 offset:2048\n\t"
          "ds_read_u16 %3, %5 offset:2176\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(w0), "=&v"(w1), "=&v"(sc), "=&v"(bi)
          : "v"(at + lane16), "v"(at + sb_read)
          : "memory");
    }
    float4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[w], raw_codes_c(w0[w], kMaskLo, kMaskHi, kMagicLo, kMagicHi), acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[w], raw_codes_c(w1[w], kMaskLo, kMaskHi, kMagicLo, kMagicHi), acc1, 0, 0, 0);
    }
    const float scale = (float)__builtin_bit_cast(half_t, (unsigned short)sc);
    const float bias = (float)__builtin_bit_cast(half_t, (unsigned short)bi);
#pragma unroll
    for (int e = 0; e < MC; ++e) {
      // (the offsets of the raw codes come out here rather than where the accumulators start, so
      // that a unit's products do not wait for the sums of a fresh x)
      const float sum = ((kc & 2) ? acc1[e] : acc0[e]) + negcorr[e];
      tot[e] = __builtin_fmaf(scale, sum, __builtin_fmaf(bias, xsum[e], tot[e]));
    }
  };

  // ---- the consumer
  uint4_t hot_ahead = n_entries > 0 ? read_hot(0) : uint4_t{0u, 0u, 0u, 0u};
  for (int d = 0; d < n_entries; ++d) {
    // (the next entry's parameters are read from LDS while this one runs: a transition does not wait for them)
    const FlowHot hot = uniform_hot(hot_ahead);
    if (d + 1 < n_entries) hot_ahead = read_hot(d + 1);
    const int nrb = hot.nrb;
    if (nrb == 0) continue;
    const int k_in = hot.k_in, m_rows = hot.m_rows;
    const int pieces = k_in >> 8;
    const int n_hc = wave < pieces ? (pieces - wave + kFlowWaves - 1) / kFlowWaves : 0;
    const int active_waves = min(kFlowWaves, pieces);
    const int x_word = hot.x_word, x_src = hot.x_src, x_id = hot.x_id;
    const char *const xrow = x_word >= 0 ? reinterpret_cast<const char *>(ex16 + x_word) : uni_ptr(cache[d].x);
    const int pr = hot.pr;
    for (int pass = 0; pass * pr < nrb; ++pass, ++q) {
      if (n_hc == 0) continue;
      const int nj = min(pr, nrb - pass * pr);
      float tot[PR][MC];
#pragma unroll
      for (int j = 0; j < PR; ++j)
#pragma unroll
        for (int e = 0; e < MC; ++e) tot[j][e] = 0.f;
      for (int hcp = 0; hcp < n_hc; ++hcp) {
        const int hc = wave + kFlowWaves * hcp;
#pragma unroll
        for (int j = 0; j < PR; ++j) {
          if (j >= nj) break;
          const bool fresh = x_id != key_id || hc != key_hc;
          const bool requested = fresh && x_requested;
          if (fresh) {
            key_id = x_id;
            key_hc = hc;
          }
          // Loads of a wave land in the order issued.  After this unit's three came the groups issued
          // with the two units before it (three loads each, two more with a request for x); a
          // requested x came just before the last of those groups.
          if (ahead < D || (requested && g2 == 2)) {
            wait_vm<0>();
          } else if (requested) {
            wait_vm<3>();
          } else {
            const int after = g1 + g2;
            if (after == 6) wait_vm<6>();
            else if (after == 8) wait_vm<8>();
            else wait_vm<10>();
          }
          consume(slot, tot[j], fresh, requested, d, hc, x_word, x_src);
          // ---- what this wave multiplies next: another piece of x is requested now, one unit ahead.
          // (Further ahead, results of an entry just before are not there yet, and what a request
          // brings instead has to be fetched again with every load of the ring in front of it.)
          int nx_hc = -1, nx_id = x_id;  // nx_hc < 0: the same piece, or nothing known
          const char *nx_row = xrow;
          if (j + 1 < nj) {
          } else if (hcp + 1 < n_hc) {
            nx_hc = hc + kFlowWaves;
          } else if ((pass + 1) * pr < nrb) {
            if (n_hc > 1) nx_hc = wave;
          } else if (d + 1 < n_entries) {
            const FlowHot next = uniform_hot(hot_ahead);
            if (next.nrb > 0 && wave < (next.k_in >> 8)) {
              nx_hc = wave;
              nx_id = next.x_id;
              if (nx_id != x_id)
                nx_row = next.x_word >= 0 ? reinterpret_cast<const char *>(ex16 + next.x_word) : uni_ptr(cache[d + 1].x);
            }
          }
          const int next_slot = slot + 1 == D ? 0 : slot + 1;
          x_requested = nx_hc >= 0 && (nx_id != key_id || nx_hc != key_hc);
          g1 = g2;
          g2 = 0;
          if (x_requested) {
            issue_x(nx_row, nx_hc, next_slot);
            g2 = 2;
          }
          if (prod.d < n_entries) {
            issue(prod, slot);
            advance(prod);
            g2 += 3;
          } else {
            --ahead;
          }
          slot = next_slot;
        }
      }
      // ---- the pass is done for this wave: its sums go to the mailbox
      const unsigned set = q % S, use = q / S;
      const unsigned emptied = lds_load(&ctl->reduced[set]);
      // this wave's sums over its four slices: two swaps of half-waves put the sums of row blocks
      // (0, 1) and (2, 3) side by side, a swap of 16-lane rows finishes both; lane (n, r) then holds
      // the sum of row block (0, 2, 1, 3)[r] for weight row n
      // (in assembly: the compiler's builtin for these swaps lost the second result here and added
      // a register to itself; the wait states are those the compiler puts between a VALU write
      // and a swap that reads it)
      float red[MC];
#pragma unroll
      for (int e = 0; e < MC; ++e) {
        float a0 = tot[0][e], a1 = tot[1][e], a2 = tot[2][e], a3 = tot[3][e];
        asm volatile(
            "s_nop 1\n\t"
            "v_permlane32_swap_b32 %0, %1\n\t"
            "v_permlane32_swap_b32 %2, %3"
            : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
        float s01 = a0 + a1, s23 = a2 + a3;
        asm volatile(
            "s_nop 1\n\t"
            "v_permlane16_swap_b32 %0, %1"
            : "+v"(s01), "+v"(s23));
        red[e] = s01 + s23;
      }
      if (emptied < use)
        while (lds_load(&ctl->reduced[set]) < use) __builtin_amdgcn_s_sleep(1);  // the set has been emptied
      float *const set_mail = mail + set * kFlowWaves * kMail;  // [e][wave][lane]
#pragma unroll
      for (int e = 0; e < MC; ++e) set_mail[(e * kFlowWaves + wave) * 64 + lane] = red[e];
      // LDS operations of a wave execute in order: the count follows the sums.  (A release fence
      // would also wait for every load of the ring.)
      asm volatile("" ::: "memory");
      // the wave that completes the set adds the sums up and stores the results (nobody waits for anybody)
      unsigned before = 0;
      if (lane == 0) before = __hip_atomic_fetch_add(&ctl->deposited[set], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      before = (unsigned)uni((int)before);
      // The arbiter of a SIMD prefers its oldest wave, and an entry is finished when its slowest wave
      // is: whoever arrives late here gets ahead of the others in the next entry
      {
        const unsigned rank = before * 4u / (unsigned)active_waves;
        if (rank >= 3u) __builtin_amdgcn_s_setprio(3);
        else if (rank == 2u) __builtin_amdgcn_s_setprio(2);
        else if (rank == 1u) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
      }
      if (before + 1u != (unsigned)active_waves) continue;
      asm volatile("" ::: "memory");
      {
        const int n_out = uni(cache[d].n_out), act = uni(cache[d].act), ex_word = uni(cache[d].ex_word);
        unsigned short *y = reinterpret_cast<unsigned short *>(const_cast<char *>(uni_ptr(cache[d].y)));
        const half_t *out_bias = reinterpret_cast<const half_t *>(uni_ptr(cache[d].out_bias));
        const int j = ((kc & 1) << 1) | (kc >> 1);
        const int row = (b + (pass * pr + j) * G) * 16 + n;
#pragma unroll
        for (int e = 0; e < MC; ++e) {
          float sum = 0.f;
          for (int w = 0; w < active_waves; ++w) sum += set_mail[(e * kFlowWaves + w) * 64 + lane];
          sum = -sum;  // (the A registers hold -x)
          if (j < nj && e < m_rows && row < n_out) {
            if (out_bias) sum += (float)out_bias[row];
            const unsigned short hv = __builtin_bit_cast(unsigned short, (half_t)apply_activation(sum, act));
            const int64_t flat = (int64_t)e * n_out + row;
            __hip_atomic_store(y + flat, hv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (ex_word >= 0) {
              // -y, zero as -0.0; value 8 q + e at place 8 q + (0,2,4,6,1,3,5,7)[e]
              const unsigned short neg = (hv & 0x7FFFu) == 0 ? (unsigned short)0x8000u : (unsigned short)(hv ^ 0x8000u);
              const int e8 = (int)(flat & 7);
              const int64_t place = (flat & ~(int64_t)7) + ((e8 & 3) * 2 + (e8 >> 2));
              __hip_atomic_store(ex16 + ex_word + place, neg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // (the mailbox reads are done)
        if (lane == 0) {
          __hip_atomic_store(&ctl->deposited[set], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          __hip_atomic_store(&ctl->reduced[set], use + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          if ((pass + 1) * pr >= nrb)  // the entry's last pass in this workgroup
            // (a maximum: the wave that finishes the next entry may get here first)
            __hip_atomic_fetch_max(&ctl->stored, (unsigned)d + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
  }
  wait_vm<0>();  // no load may land in LDS after this workgroup has gone

  // ---- the last wave of the last workgroup turns the exchange over: the next launch uses the other half
  unsigned done = 0;
  if (lane == 0) done = __hip_atomic_fetch_add(&ctl->waves_done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  if ((unsigned)uni((int)done) != kFlowWaves - 1) return;
  unsigned last = 0;
  if (lane == 0) last = atomicAdd(words + kFlowExitedWord, 1u) == (unsigned)G - 1;
  if (!uni((int)last)) return;
  if (lane == 0) {
    __hip_atomic_store(words + kFlowExtentWord + half, (unsigned)plan->exchange_values, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(words + kFlowExtentWord + (1u - half), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(words + kFlowEpochWord, half ^ 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(words + kFlowExitedWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace

template <int MC, bool EARLY>
__global__ __launch_bounds__(kFlowThreads) void gemv_flow_kernel(const void *entries, int n_entries, int *status,
                                                                 unsigned *words, unsigned spin_limit,
                                                                 const SequencePlan plan) {
  flow_body<MC, EARLY>(reinterpret_cast<const Entry *>(entries), n_entries, status, words, spin_limit, &plan);
}

// Can this launch run on the data-flow kernel?  Every weight in the streaming layout, one batch
// row (measured at batch 4: the LDS-ring kernel is faster there), and no entry that has to wait
// for reported completion.
bool flow_eligible(const gq_gemv_desc *e, int n, const SequencePlan &plan) {
  for (int i = 0; i < n; ++i)
    if (e[i].scale != nullptr || e[i].bias != nullptr || e[i].m_rows != 1 || plan.need[i] != 0 || e[i].k_in % 512 != 0) return false;
  return true;
}

int launch_flow(const gq_gemv_desc *host, const gq_gemv_desc *device, int n, int *status, unsigned *words, unsigned spins,
                const SequencePlan &plan, int grid, int dev, hipStream_t stream) {
  constexpr int kMaxDevices = 64;
  if (dev < 0 || dev >= kMaxDevices) return fail(GQ_ERR_UNSUPPORTED, "device index %d", dev);
  // does any entry pass its results on in parts?  (the kernel's own rule, for the row blocks of a full grid)
  bool early = false;
  for (int i = 0; i < n; ++i)
    early |= plan.ex_word[i] >= 0 && (host[i].n_out + 15) / 16 > (int64_t)(kEarlyMinBlocks - 1) * grid;
#define GQ_FLOW(MC, EARLY)                                                                                    \
  do {                                                                                                        \
    constexpr int lds_bytes = flow_lds_bytes<MC>();                                                           \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                    \
    static bool configured[kMaxDevices] = {false};                                                            \
    if (!configured[dev]) {                                                                                   \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_flow_kernel<MC, EARLY>),   \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);        \
      if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));              \
      configured[dev] = true;                                                                                 \
    }                                                                                                         \
    gemv_flow_kernel<MC, EARLY><<<dim3(grid), dim3(kFlowThreads), lds_bytes, stream>>>(device, n, status, words, spins, \
                                                                                      plan);                 \
  } while (0)
  if (early) GQ_FLOW(1, true);
  else GQ_FLOW(1, false);
#undef GQ_FLOW
  return GQ_OK;
}

}  // namespace gq
