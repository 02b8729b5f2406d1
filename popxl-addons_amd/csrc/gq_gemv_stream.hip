// A sequence of fused dequant-GEMVs as ONE persistent kernel (decode of a layer stack).
//
// Launching a GEMV per weight matrix leaves HBM idle between kernels: ~2 us of launch, ramp and
// drain for every 1.3 - 5 us of weight streaming.  Here one workgroup per compute unit walks the
// whole list of entries.  Packed weights, scales and biases never depend on earlier results, so
// every wave streams them through a private LDS ring with direct-to-LDS loads that run several
// work items ahead -- across entry boundaries -- while only the small activation vector x waits
// for the entries it depends on (per-workgroup progress words, bounded spin).
//
// Work decomposition of one entry (n_out x k_in, k_in % 512 == 0, group 64, m_rows <= 4):
//   row block  = 16 weight rows; workgroup b of G owns row blocks b, b + G, ... in passes of 4 (2 when MC = 4)
//   phase      = 4096 contraction indices; wave w owns chunk 8 p + w (512 indices) of phase p
//   work item  = (row block, chunk): 4 KiB of packed words + 2 x 256 B of scale / bias
// An entry may bring its weight in the streaming layout instead (scale == bias == nullptr, made by
// gq_gemv_prepack_f16): work item (row block rb, chunk c) is the 4608-byte block number
// rb * (k_in / 512) + c, byte for byte what the item's ring slot holds, so that its loads are
// 1 KiB contiguous each instead of sixteen 64-byte or 16-byte pieces 128+ bytes apart.
//
// Arithmetic.  Once the weights stream without gaps the loop is bound by instruction issue, not by
// HBM, so the expansion of the codes is kept to 5 VALU instructions per 8 weights: a code is only
// or-ed into the mantissa of 64.0 or 1024.0 (exact: 64 + c or 1024 + c) and goes to the MFMA as
// it is.  Scale and bias are applied to SUMS instead of weights:
//   y[n] = sum_g scale[n][g] * ( sum_{k in g} (off_k + c[n][k]) x[k]  -  sum_{k in g} off_k x[k] )
//        + sum_g bias[n][g]  *   sum_{k in g} x[k]
// v_mfma_f32_16x16x32_f16 computes D[i][n] += sum_k A[i][k] B[k][n].  B holds the raw codes of 16
// weight rows n; A holds x, its sixteen rows i used as (group, batch row) combinations: row i of A
// is x[m(i)] on the contraction indices of group g(i) and zero elsewhere.  One accumulator thus
// separates the groups of a whole item (MC = 2: 8 groups x 2 batch rows) or of half an item
// (MC = 4: 4 groups x 4 batch rows), and a lane finds in its 4 accumulator registers group sums of
// ITS weight row.  The per-group corrections sum off_k x[k] and sum x[k] are computed once per x
// chunk (v_dot2_f32_f16, fp32 accumulation).
#include "gq_gemv_sequence.h"

namespace gq {
namespace {

__device__ __attribute__((aligned(256))) unsigned int g_sequence_words[kSequenceWords];

// MC: batch rows a launch can hold (2 or 4; the x stage of a wave holds MC KiB); NS: depth of the
// weight ring.  (A __device__ function: a __global__ template is also instantiated for the host,
// where the target builtins and inline assembly do not exist.)
//
// Waves 0..7 compute; they never meet at a workgroup barrier.  After the last chunk of a pass a
// wave drops its 16 x m partial sums into its mailbox (two sets, used by passes in turn, so a wave
// may run a pass ahead of the slowest) and goes on with the next pass or entry.
// Wave 8, the reducer, adds the eight mailboxes in a fixed order, stores y and, for entries that
// somebody waits for, publishes the workgroup's progress.  Wave 9, the poller, keeps the LDS word
// `ready` (how many entries are complete everywhere) up to date: the watcher's from the progress
// words of all workgroups, everybody else's from the watcher's announcement; a compute wave that
// needs an earlier result waits for that number only.  (The LDS reads of `ready` and `consumed`
// in the compute waves are visible to the compiler, which therefore waits for all loads of the
// ring before them; hiding them in assembly was measured and gains nothing.)
//
// Visibility of results between compute units needs no cache flush: y is written with device-scope
// stores (sc1, write-through to the coherent level), the reducer waits for its stores before it
// publishes, and x is read with device-coherent loads.
// SINGLE: the sequence is the one entry `single`, passed by value (no descriptor in memory).
template <int MC, int NS, bool SINGLE>
__device__ __forceinline__ void gemv_stream_body(const Entry *__restrict__ entries, int n_entries,
                                                 int *__restrict__ status, unsigned *words, unsigned spin_limit,
                                                 const SequencePlan *plan, const Entry single) {
  static_assert(MC == 2 || MC == 4, "batch capacity");
  constexpr int PR = pass_rows(MC);
  extern __shared__ __attribute__((aligned(64))) char lds[];
  constexpr int kWaveBytes = NS * kItemBytes + kStageBytes;
  static_assert(kWaveBytes % 64 == 0 && (NS * kItemBytes) % 64 == 0, "the x stage starts on a 64-byte boundary");
  constexpr int kMailFloats = PR * MC * 16;  // per wave: [row block][m][n]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uni(tid >> 6);
  const int r = lane & 15, kc = lane >> 4;
  const int G = gridDim.x, b = blockIdx.x;
  unsigned *const g_progress = words, *const g_announced = words + kAnnouncedWord, *const g_exited = words + kExitedWord;
  unsigned *const g_epoch = words + kEpochWord, *const exchange = words + kExchangeWord;
  CachedEntry *cache = reinterpret_cast<CachedEntry *>(lds + kWaves * kWaveBytes);
  float *mail = reinterpret_cast<float *>(lds + kWaves * kWaveBytes + kMaxEntries * 64);
  Control *ctl = reinterpret_cast<Control *>(mail + 2 * kWaves * kMailFloats);  // two sets of mailboxes
  // MC == 4 only: per wave, the group sums of the current x chunk, [half][kc][corr e0..3, xsum e0..3]
  // (registers are short in that variant)
  float *table = reinterpret_cast<float *>(ctl) + 16 + wave * 64;
  // the watcher's copy of the progress words
  unsigned *seen = reinterpret_cast<unsigned *>(ctl) + 16 + kWaves * 64;

  for (int i = tid; i < n_entries; i += kThreadsAll) {
    const Entry e = SINGLE ? single : entries[i];
    CachedEntry c;
    c.packed = reinterpret_cast<const char *>(e.packed);
    c.scale = reinterpret_cast<const char *>(e.scale);
    c.bias = reinterpret_cast<const char *>(e.bias);
    c.x = e.x;
    c.out_bias = e.out_bias;
    c.y = e.y;
    c.n_out = e.n_out;
    c.k_in = e.k_in;
    c.m_rows = (short)e.m_rows;
    c.wait = SINGLE ? (short)0 : plan->need[i];  // (entries of earlier launches are complete)
    const int rb = (e.n_out + 15) >> 4;
    c.nrb = (short)(rb > b ? (rb - b + G - 1) / G : 0);
    c.publish = 0;
    c.act = (char)e.activation;
    cache[i] = c;
  }
  if (tid < kMaxGroups) seen[tid] = 0u;
  if (tid == 0) {
    unsigned tag = 0;
    if (!SINGLE && plan->uses_exchange) {
      tag = __hip_atomic_load(g_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (tag == 0) tag = 1;  // a fresh block
    }
    *ctl = Control{{0u, 0u}, 0u, 0u, 0u, 0u, {0u, 0u, 0u, 0u}, tag << 16, 0u};
  }
  __syncthreads();
  // completion is reported only where an entry waits for it (a report costs the reducer a round
  // trip to memory)
  for (int i = tid; i < n_entries; i += kThreadsAll) {
    const int w = cache[i].wait;
    if (w > 0) {
      cache[w - 1].publish = 1;
      atomicOr(&ctl->targets[(w - 1) >> 5], 1u << ((w - 1) & 31));
    }
  }
  __syncthreads();

  // ============================================================================ poller
  if (wave == kWaves + 1) {
    // the counts somebody waits for, in increasing order: the next one after `ready`
    const unsigned t0 = (unsigned)uni((int)ctl->targets[0]), t1 = (unsigned)uni((int)ctl->targets[1]);
    const unsigned t2 = (unsigned)uni((int)ctl->targets[2]), t3 = (unsigned)uni((int)ctl->targets[3]);
    auto next_target = [&](unsigned ready) -> unsigned {  // smallest waited-for count > ready, 0 if none
      const unsigned words[4] = {t0, t1, t2, t3};
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        unsigned bits = words[w];
        if (ready >= 32u * (w + 1)) continue;
        if (ready > 32u * w) bits &= ~0u << (ready - 32u * w);
        if (bits) return 32u * w + (unsigned)__builtin_ctz(bits) + 1u;
      }
      return 0u;
    };
    // Reads of memory are direct-to-LDS loads that nobody waits for one by one: a new one is issued
    // every ~100 ns with several in flight, so a change is seen one memory latency after it
    // happened instead of up to two round trips later.  The values only grow, loads return in the
    // order issued, so the LDS copies only grow too.
    //   watcher: 4 loads copy the 256 progress words into `seen`; a count is complete everywhere
    //            when every word has reached it; the result goes to ctl->ready and g_announced
    //   others : one lane copies g_announced straight into ctl->ready, where the compute waves look
    unsigned ready = 0, spins = 0;
    unsigned target = next_target(0u);
    const bool watcher = b == 0;
    unsigned last_seen[4] = {0u, 0u, 0u, 0u};  // watcher: this lane's four progress words as last read
    int lane_zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(lane_zero));
    while (target) {
      // nothing can be complete everywhere before it is complete here: stay off the memory system
      // until this workgroup has reported the count in question
      while (lds_peek(&ctl->published) < target) __builtin_amdgcn_s_sleep(2);
      bool advanced = false;
      if (!watcher) {
        // (the address must come from a vector register: with a uniform address the compiler
        // emits a malformed instruction)
        if (lane == 0)
          __builtin_amdgcn_global_load_lds(g_announced + lane_zero, reinterpret_cast<unsigned *>(&ctl->ready), 4, 0,
                                           kAuxDeviceCoherent);
        wait_vm<7>();
        __builtin_amdgcn_s_sleep(2);
        const unsigned now = (unsigned)uni((int)lds_peek(&ctl->ready));
        while (target && now >= target) {
          ready = target;
          target = next_target(ready);
          advanced = true;
        }
      } else {
        // only the words that have not reached the target yet: once most workgroups are through,
        // a sweep is a handful of loads, and the watcher's own compute unit keeps its bandwidth
#pragma unroll
        for (int i = 0; i < 4; ++i)  // (indices past the last workgroup read its word again)
          if (last_seen[i] < target)
            __builtin_amdgcn_global_load_lds(g_progress + min(i * 64 + lane, G - 1) * kProgressStride, seen + i * 64, 4, 0,
                                             kAuxDeviceCoherent);
        wait_vm<8>();  // bounds the loads in flight (a sweep is at most 4)
        __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int i = 0; i < 4; ++i) last_seen[i] = lds_peek(&seen[i * 64 + lane]);
        unsigned lo = min(min(last_seen[0], last_seen[1]), min(last_seen[2], last_seen[3]));
        while (target && __builtin_amdgcn_ballot_w64(lo < target) == 0) {  // no lane below the target
          ready = target;
          target = next_target(ready);
          advanced = true;
        }
        if (advanced && lane == 0) {
          __hip_atomic_store(&ctl->ready, ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          __hip_atomic_store(g_announced, ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      if (advanced) {
        spins = 0;
      } else if (++spins > spin_limit) {  // some workgroup is not running: give up, let everybody finish
        if (lane == 0) {
          __hip_atomic_store(&ctl->failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          if (status) atomicExch(status, 1);
        }
        break;
      }
    }
    wait_vm<0>();  // no load may land in LDS after this workgroup has gone
    return;
  }

  // =========================================================================== reducer
  if (wave == kWaves) {
    unsigned q = 0;  // passes reduced so far
    for (int d = 0; d < n_entries; ++d) {
      const int nrb = uni(cache[d].nrb), m_rows = uni(cache[d].m_rows), n_out = uni(cache[d].n_out);
      half_t *y = cache[d].y;
      const half_t *out_bias = cache[d].out_bias;
      const int act = uni(cache[d].act);
      // a later entry of this launch reads these results as its x: they also go to the exchange, tagged
      const int ex_word = SINGLE ? -1 : plan->ex_word[d];
      unsigned *const ex = ex_word >= 0 ? exchange + ex_word : nullptr;
      const unsigned tag = ex ? (unsigned)uni((int)lds_load(&ctl->tag)) : 0u;
      for (int pass = 0; pass * PR < nrb; ++pass, ++q) {
        const int nj = min(PR, nrb - pass * PR);
        while (lds_load(&ctl->deposited[q & 1]) < ((q >> 1) + 1) * kWaves) __builtin_amdgcn_s_sleep(1);
        const float *box = mail + (q & 1) * kWaves * kMailFloats;
        // one sum per (row block j, batch row m, output n): consecutive lanes, consecutive n
        for (int t = lane; t < nj * MC * 16; t += 64) {
          const int n16 = t & 15, m = (t >> 4) % MC, j = t / (16 * MC);
          float sum = 0.f;
#pragma unroll
          for (int w = 0; w < kWaves; ++w) sum += box[w * kMailFloats + t];
          const int n = (b + (pass * PR + j) * G) * 16 + n16;
          if (m < m_rows && n < n_out) {
            if (out_bias) sum += (float)out_bias[n];
            const half_t hv = (half_t)apply_activation(sum, act);
            // device-scope store: written through to where every compute unit reads it
            __hip_atomic_store(reinterpret_cast<unsigned short *>(y) + (int64_t)m * n_out + n,
                               __builtin_bit_cast(unsigned short, hv), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (ex)
              __hip_atomic_store(ex + (int64_t)m * n_out + n, tag | __builtin_bit_cast(unsigned short, hv), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        // the mailboxes have been read (the sums above depend on them): free them
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_store(&ctl->consumed, q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      // (consumers in this workgroup start to look for the results on the whole device from here)
      if (ex && lane == 0) __hip_atomic_store(&ctl->stored, (unsigned)d + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (uni(cache[d].publish)) {
        wait_vm<0>();  // every lane's stores of this and of all earlier entries are complete ...
        if (lane == 0) {  // ... then publish
          __hip_atomic_store(&g_progress[b * kProgressStride], (unsigned)d + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(&ctl->published, (unsigned)d + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
    // a sequence without dependencies has touched neither the progress words nor the exchange
    const unsigned any_target = ctl->targets[0] | ctl->targets[1] | ctl->targets[2] | ctl->targets[3];
    const bool uses_exchange = !SINGLE && plan->uses_exchange;
    if (uni((int)any_target) == 0 && !uses_exchange) return;
    // the last workgroup out clears the progress words and advances the epoch: by then every
    // poller has seen all it needs and nobody reads the exchange any more (a workgroup's compute
    // waves have finished before its reducer gets here)
    wait_vm<0>();  // this workgroup's last progress word is in memory before it counts itself out
    unsigned last = 0;
    if (lane == 0) last = atomicAdd(g_exited, 1u) == (unsigned)G - 1;
    if (uni((int)last)) {
      wait_vm<0>();
      if (uni((int)any_target)) {
        for (int i = lane; i < G; i += 64)
          __hip_atomic_store(&g_progress[i * kProgressStride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) __hip_atomic_store(g_announced, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (uses_exchange) {
        unsigned epoch = (unsigned)uni((int)lds_load(&ctl->tag)) >> 16;
        if (epoch == 0xFFFFu) {
          // the tags are about to repeat: no word of an earlier launch may survive
          for (int i = lane; i < kExchangeWords / 4; i += 64)
            __builtin_nontemporal_store(uint4_t{0u, 0u, 0u, 0u}, reinterpret_cast<uint4_t *>(exchange) + i);
          wait_vm<0>();
          epoch = 0;
        }
        if (lane == 0) __hip_atomic_store(g_epoch, epoch + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (lane == 0) __hip_atomic_store(g_exited, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
  }

  // ==================================================================== compute waves
  char *ring = lds + wave * kWaveBytes;
  char *xstage = ring + NS * kItemBytes;
  const uint32_t ring_rd = (uint32_t)(uintptr_t)ring, x_rd = (uint32_t)(uintptr_t)xstage;

  // ---- the producer walks the same item list as the consumer, NS items ahead.  Everything it
  // needs is wave-uniform (scalar registers): advancing the cursor costs no vector instruction.
  struct ProducerEntry {
    const char *packed, *scale, *bias;
    int n_out, k_in, nrb, phases;
  } pe = {nullptr, nullptr, nullptr, 1, 512, 0, 1};  // (scale == nullptr: streaming layout)
  auto load_producer_entry = [&](int d) {
    if (d >= n_entries) return;
    pe.packed = uni_ptr(cache[d].packed);
    pe.scale = uni_ptr(cache[d].scale);
    pe.bias = uni_ptr(cache[d].bias);
    pe.n_out = uni(cache[d].n_out);
    pe.k_in = uni(cache[d].k_in);
    pe.nrb = uni(cache[d].nrb);
    pe.phases = (pe.k_in + 4095) >> 12;
  };
  // does cursor c name a work item of this wave?  (entries without rows for this workgroup and
  // chunks past k_in are skipped)
  auto valid = [&](const Cursor &c) {
    if (c.d >= n_entries) return true;  // the end is a valid resting place
    return c.pass * PR + c.j < pe.nrb && (c.phase * kWaves + wave) * 512 < pe.k_in;
  };
  auto step = [&](Cursor &c) {
    if (++c.j < PR && c.pass * PR + c.j < pe.nrb) return;
    c.j = 0;
    if (++c.phase < pe.phases) return;
    c.phase = 0;
    if (++c.pass * PR < pe.nrb) return;
    c.pass = 0;
    ++c.d;
    load_producer_entry(c.d);
  };
  auto next_item = [&](Cursor &c) {
    do step(c);
    while (c.d < n_entries && !valid(c));
  };
  // direct-to-LDS loads of the item at cursor c into ring slot `slot`: scalar base of the row
  // block's chunk + one 32-bit offset per lane
  auto issue_item = [&](const Cursor &c, int slot) {
    const int rb = b + (c.pass * PR + c.j) * G;
    const int chunk = c.phase * kWaves + wave;
    const int row = min(r, pe.n_out - 1 - rb * 16);  // rows past n_out re-read the last one
    char *dst = ring + slot * kItemBytes;
    if (pe.scale == nullptr) {
      const char *blk = pe.packed + ((int64_t)rb * (pe.k_in >> 9) + chunk) * kItemBytes + lane * 16;
#pragma unroll
      for (int s = 0; s < 4; ++s)
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(blk + s * 1024), dst + s * 1024, 16, 0, kAuxWeights);
      // (two loads of 256 bytes, like the other layout: every item counts kItemOps loads)
      if (kc == 0) __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(blk + 4096), dst + 4096, 16, 0, kAuxWeights);
      if (kc == 1) __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(blk + 4096), dst + 4096, 16, 0, kAuxWeights);
      return;
    }
    const char *src = pe.packed + (int64_t)rb * 16 * (pe.k_in >> 1) + chunk * 256;
    const uint32_t off = (uint32_t)row * (uint32_t)(pe.k_in >> 1) + (uint32_t)kc * 16u;
#pragma unroll
    for (int s = 0; s < 4; ++s)
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(src + off + s * 64), dst + s * 1024, 16, 0, kAuxWeights);
    // lanes 0..15 fetch the 8 scales of their row's chunk, lanes 16..31 the 8 biases
    const uint32_t off2 = (uint32_t)row * (uint32_t)(pe.k_in >> 5);
    const int64_t base2 = (int64_t)rb * 16 * (pe.k_in >> 5) + chunk * 16;
    if (kc == 0)
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(pe.scale + base2 + off2), dst + 4096, 16, 0, kAuxWeights);
    if (kc == 1)
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(pe.bias + base2 + off2), dst + 4096, 16, 0, kAuxWeights);
  };

  Cursor prod = {0, 0, 0, 0};  // the producer's position: first item of this wave
  load_producer_entry(0);
  if (n_entries > 0 && !valid(prod)) next_item(prod);
  int n_ahead = 0;  // items issued and not yet consumed
  while (n_ahead < NS && prod.d < n_entries) {
    issue_item(prod, n_ahead);
    ++n_ahead;
    next_item(prod);
  }
  int slot = 0;    // ring slot of the consumer's item
  unsigned q = 0;  // passes finished so far (same count in every wave)

  // ---- lane roles
  // B operand / loader: weight row r, 16-byte piece kc of every 64-byte stretch.
  // A operand: combination i = r of (group, batch row); contraction slice kc.
  // D: column n = r (weight row), rows 4 kc + e = combinations.
  //   MC == 2: i = 2 g + m, g = 0..7: one accumulator per item; a lane's rows are groups 2kc, 2kc+1
  //   MC == 4: i = 4 g + m, g = 0..3: accumulator A for groups 0..3 (loads 0, 1), B for 4..7
  const int a_g = MC == 2 ? (r >> 1) : (r >> 2);  // group of this lane's A row (within its half for MC 4)
  const int a_m = MC == 2 ? (r & 1) : (r & 3);
  const int a_load = a_g >> 1;                     // the 16-byte load (128 indices) holding that group
  const bool a_match = (kc >> 1) == (a_g & 1);     // ... and whether this lane's slice is in the group
  const uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x00F000F0u, kMagicLo = 0x64006400u, kMagicHi = 0x54005400u;
  const half2_t kOnes = {(half_t)1.0f, (half_t)1.0f};
  const half2_t kOffsets = {(half_t)64.0f, (half_t)1024.0f};  // even index of a word: 64 + c, odd: 1024 + c

  half8_t xa[4][4];                  // A operands of the 16 MFMA steps of an item
  float corr[4] = {0.f, 0.f, 0.f, 0.f};  // MC 2: sum of off_k x[k] over the group of accumulator row e
  float xsum[4] = {0.f, 0.f, 0.f, 0.f};  // MC 2: sum of x[k] over that group
  const uint32_t table_rd = (uint32_t)(uintptr_t)table + kc * 32;
#pragma unroll
  for (int L = 0; L < 4; ++L)
#pragma unroll
    for (int j = 0; j < 4; ++j) xa[L][j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  if (MC == 4 && r == 0) {
    // the table must hold numbers before the first x chunk arrives (0 * NaN would poison a sum)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) table[(h * 4 + kc) * 8 + e] = 0.f;
  }
  // Layout of an x chunk in the stage: row m (1 KiB) holds its sixty-four 16-byte units permuted,
  // unit g at position g ^ ((m ^ (g >> 4)) & 3).  The operand build reads, per instruction, one
  // unit from each (batch row, 256-byte quarter, slice) combination: unpermuted, all combinations
  // of a slice fall on the same four banks (8-way conflicts, measured: 53 M conflict cycles per
  // pass of 4096 x 16384 entries at batch 4); permuted, they spread over the sixteen bank groups.
  // The permutation is its own inverse: the lane that fills position l fetches unit x_unit(m).
  auto x_unit = [&](int m) { return lane ^ ((m ^ (lane >> 4)) & 3); };
  const half_t *x_loaded = nullptr;  // the operands in registers belong to (x_loaded, chunk x_chunk)
  int x_chunk = -1, x_k = 0, x_m = 0;
  const half_t *st_x = nullptr;  // the stage holds this wave's chunk of EVERY phase of (st_x, st_k, st_m)
  int st_k = 0, st_m = 0;
  unsigned known_ready = 0;  // entries this wave has seen complete on the whole device
  int x_from = -1;           // the entry of this launch that produced the x in the registers / the stage (-1: memory)

  // Rows of x out of the exchange.  Row j (of n_rows <= 4) is 512 tagged words starting at exchange
  // word rw[j]; its values go to the stage at byte rd[j] as fp16, in the permuted unit order of batch
  // row rm[j].  Every lane fetches the 8 words of one unit, again and again until every word of
  // every row carries this launch's tag -- then all of them have arrived, whatever else the
  // producers still have in flight.  (These loads are the youngest: everything in the ring lands
  // with them.)
  auto fetch_tagged = [&](int n_rows, const int (&rw)[4], const int (&rd)[4], const int (&rm)[4], int src) {
    const unsigned tag = lds_peek(&ctl->tag);
    // nothing can have arrived from everywhere before this workgroup's own share has been stored
    while (lds_peek(&ctl->stored) <= (unsigned)src && !lds_peek(&ctl->failed)) __builtin_amdgcn_s_sleep(1);
    const unsigned polls_allowed = spin_limit >> 4;  // (a poll here is a memory round trip, not a look at LDS)
    unsigned polls = 0;
    uint4_t t[4][2];
    for (;;) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (j < n_rows) {
          const unsigned *p = exchange + rw[j] + (lane ^ ((rm[j] ^ (lane >> 4)) & 3)) * 8;
          asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(t[j][0]) : "v"(p) : "memory");
          asm volatile("global_load_dwordx4 %0, %1, off offset:16 sc1" : "=v"(t[j][1]) : "v"(p) : "memory");
        }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      unsigned bad = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (j < n_rows) {
          asm volatile("" : "+v"(t[j][0]), "+v"(t[j][1]));  // (read below the wait)
#pragma unroll
          for (int e = 0; e < 4; ++e) bad |= (t[j][0][e] ^ tag) | (t[j][1][e] ^ tag);
        }
      if (__builtin_amdgcn_ballot_w64((bad >> 16) != 0u) == 0) break;
      if (polls++ >= polls_allowed || lds_peek(&ctl->failed)) {  // some workgroup is not running: give up
        if (lane == 0) {
          __hip_atomic_store(&ctl->failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          if (status) atomicExch(status, 1);
        }
        break;
      }
      __builtin_amdgcn_s_sleep(4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < n_rows) {
        uint4_t q;  // the low halves of the eight words
        q.x = __builtin_amdgcn_perm(t[j][0].y, t[j][0].x, 0x05040100u);
        q.y = __builtin_amdgcn_perm(t[j][0].w, t[j][0].z, 0x05040100u);
        q.z = __builtin_amdgcn_perm(t[j][1].y, t[j][1].x, 0x05040100u);
        q.w = __builtin_amdgcn_perm(t[j][1].w, t[j][1].z, 0x05040100u);
        asm volatile("ds_write_b128 %0, %1" : : "v"(x_rd + rd[j] + lane * 16), "v"(q) : "memory");
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  // an entry whose x chunks do not fit the stage together fetches the chunk of its NEXT phase as
  // soon as the operands of the current one are in registers, instead of draining the ring for it
  int ahead_d = -1, ahead_chunk = -1;  // the stage holds (or will hold) this chunk of entry ahead_d
  int ahead_after = 0;                 // items issued after that request (loads return in order)

  for (int d = 0; d < n_entries; ++d) {
    const int nrb = uni(cache[d].nrb), m_rows = uni(cache[d].m_rows), k_in = uni(cache[d].k_in);
    const half_t *x = reinterpret_cast<const half_t *>(uni_ptr(cache[d].x));
    const int phases = (k_in + 4095) >> 12;
    const unsigned need = (unsigned)uni(cache[d].wait);
    if (need > known_ready) {
      // every workgroup has finished the first `need` entries (published by the poller)
      while ((known_ready = lds_load(&ctl->ready)) < need && !lds_load(&ctl->failed)) __builtin_amdgcn_s_sleep(1);
      x_loaded = nullptr;
      st_x = nullptr;
    }
    // x out of the exchange (the host's plan: x is what entry x_src of this launch produces)
    const int x_src = SINGLE ? -1 : (int)plan->x_src[d];
    const int x_word = SINGLE ? -1 : plan->x_word[d];
    if (x_src != x_from) {  // another producer: other values, even at the same address
      x_loaded = nullptr;
      st_x = nullptr;
      x_from = x_src;
    }
    // an entry with several phases whose x chunks all fit the stage fetches them in one go: one
    // drain of the ring per entry instead of one per phase
    const bool fits_all = phases > 1 && phases * m_rows * 1024 <= kStageBytes;
    bool staged = fits_all && st_x == x && st_k == k_in && st_m == m_rows;
    if (fits_all && !staged && nrb > 0) {
      if (x_word >= 0) {
        int rw[4] = {0, 0, 0, 0}, rd[4] = {0, 0, 0, 0}, rm[4] = {0, 0, 0, 0}, n_rows = 0;
        for (int phase = 0; phase < phases; ++phase) {
          const int chunk = phase * kWaves + wave;
          if (chunk * 512 >= k_in) continue;
          for (int m = 0; m < m_rows; ++m, ++n_rows) {
            rw[n_rows & 3] = x_word + m * k_in + chunk * 512;
            rd[n_rows & 3] = (phase * m_rows + m) * 1024;
            rm[n_rows & 3] = m;
          }
        }
        fetch_tagged(n_rows, rw, rd, rm, x_src);
      } else {
        for (int phase = 0; phase < phases; ++phase) {
          const int chunk = phase * kWaves + wave;
          if (chunk * 512 >= k_in) continue;
          for (int m = 0; m < m_rows; ++m)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(x + (int64_t)m * k_in + chunk * 512) + x_unit(m),
                                             xstage + (phase * m_rows + m) * 1024, 16, 0, kAuxDeviceCoherent);
        }
      }
      wait_vm<0>();
      st_x = x;
      st_k = k_in;
      st_m = m_rows;
      staged = true;
    }
    for (int pass = 0; pass * PR < nrb; ++pass, ++q) {
      const int nj = min(PR, nrb - pass * PR);
      float4_t tot[PR];  // running sums: scale and bias applied, groups not yet added up
#pragma unroll
      for (int j = 0; j < PR; ++j) tot[j] = float4_t{0.f, 0.f, 0.f, 0.f};
      for (int phase = 0; phase < phases; ++phase) {
        const int chunk = phase * kWaves + wave;
        if (chunk * 512 >= k_in) continue;
        // ---- A operands and group sums of this chunk (kept when the previous entry used the same x)
        const bool reload_x = !(x_loaded == x && x_chunk == chunk && x_k == k_in && x_m == m_rows);
        bool drained = false;
        if (reload_x) {
          if (!staged) {
            if (ahead_d == d && ahead_chunk == chunk) {
              // requested ahead of time: older than the loads of ahead_after items
              if (ahead_after >= 3) wait_vm<3 * kItemOps>();
              else if (ahead_after == 2) wait_vm<2 * kItemOps>();
              else if (ahead_after == 1) wait_vm<kItemOps>();
              else wait_vm<0>();
            } else if (x_word >= 0) {
              int rw[4] = {0, 0, 0, 0}, rd[4] = {0, 0, 0, 0}, rm[4] = {0, 0, 0, 0};
              for (int m = 0; m < m_rows; ++m) {
                rw[m & 3] = x_word + m * k_in + chunk * 512;
                rd[m & 3] = m * 1024;
                rm[m & 3] = m;
              }
              fetch_tagged(m_rows, rw, rd, rm, x_src);
              drained = true;
            } else {
              for (int m = 0; m < m_rows; ++m)
                __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(x + (int64_t)m * k_in + chunk * 512) + x_unit(m),
                                                 xstage + m * 1024, 16, 0, kAuxDeviceCoherent);
              wait_vm<0>();  // x is the youngest load: everything in flight lands with it
              drained = true;
            }
            ahead_d = -1;
            st_x = nullptr;
          }
          const uint32_t xs_rd = x_rd + (staged ? phase * m_rows * 1024 : 0);
          // a lane whose slice lies outside its group, or whose batch row does not exist, supplies
          // zeros: it keeps no operand (my_load matches no step) and its sums are dropped
          const bool active = a_match && a_m < m_rows;
          const int my_load = active ? a_load : -1;
          constexpr int HALVES = MC == 2 ? 1 : 2;
          float part_sum[HALVES], part_corr[HALVES];
#pragma unroll
          for (int h = 0; h < HALVES; ++h) {
            // this lane's 32 indices of its group: 4 x 8 consecutive fp16 at (load, slice kc)
            const int load = a_load + 2 * h;
            uint4_t xq[4];
            // unit 4 (4 load + kc) + j of row a_m, at its permuted position
            const uint32_t piece = (xs_rd + a_m * 1024 + (4 * load + kc) * 64) | (((a_m ^ load) & 3) << 4);
#pragma unroll
            for (int j = 0; j < 4; ++j)
              asm volatile("ds_read_b128 %0, %1" : "=v"(xq[j]) : "v"(piece ^ (j << 4)));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xq[0]), "+v"(xq[1]), "+v"(xq[2]), "+v"(xq[3]));
            float s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                s1 = __builtin_amdgcn_fdot2(as_half2(xq[j][t]), kOnes, s1, false);
                s2 = __builtin_amdgcn_fdot2(as_half2(xq[j][t]), kOffsets, s2, false);
              }
              const half8_t p = permute_x(xq[j]);
              if (MC == 2) {
#pragma unroll
                for (int L = 0; L < 4; ++L) xa[L][j] = my_load == L ? p : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
              } else {
#pragma unroll
                for (int L = 0; L < 2; ++L) xa[L + 2 * h][j] = my_load == L ? p : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
              }
            }
            if (!active) s1 = s2 = 0.f;  // (rows of x that were not loaded may hold anything)
            // the other half of the group sits in the neighbouring slice
            part_sum[h] = s1 + lane_read(s1, lane ^ 16);
            part_corr[h] = s2 + lane_read(s2, lane ^ 16);
          }
          // accumulator row e of lane (n, kc) is combination 4 kc + e: fetch its sums from a lane
          // that holds that A row and whose slice lies in the group
#pragma unroll
          for (int h = 0; h < HALVES; ++h) {
            float4_t cs, xs;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int i = 4 * kc + e;
              const int g = MC == 2 ? (i >> 1) : (i >> 2);
              const int src = i + 32 * (g & 1);
              xs[e] = lane_read(part_sum[h], src);
              cs[e] = lane_read(part_corr[h], src);
            }
            if (MC == 2) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                xsum[e] = xs[e];
                corr[e] = cs[e];
              }
            } else if (r == 0) {
              *reinterpret_cast<float4_t *>(table + (h * 4 + kc) * 8) = cs;
              *reinterpret_cast<float4_t *>(table + (h * 4 + kc) * 8 + 4) = xs;
            }
          }
          x_loaded = x;
          x_chunk = chunk;
          x_k = k_in;
          x_m = m_rows;
          if (!staged && phases > 1) {
            // the stage has been read: request this wave's chunk of the next phase (or of the first
            // phase of the next pass) into it
            int next_chunk = (phase + 1) * kWaves + wave;
            if (phase + 1 >= phases || next_chunk * 512 >= k_in) next_chunk = (pass + 1) * PR < nrb ? wave : -1;
            if (next_chunk >= 0 && next_chunk * 512 < k_in) {
              for (int m = 0; m < m_rows; ++m)
                __builtin_amdgcn_global_load_lds(
                    reinterpret_cast<const uint4_t *>(x + (int64_t)m * k_in + next_chunk * 512) + x_unit(m), xstage + m * 1024,
                    16, 0, kAuxDeviceCoherent);
              ahead_d = d;
              ahead_chunk = next_chunk;
              ahead_after = 0;
            }
          }
        }
#pragma unroll
        for (int j = 0; j < PR; ++j) {
          if (j >= nj) break;
          // ---- this item's loads are older than those of the n_ahead - 1 items issued after it
          if (!drained || j > 0) {
            if (n_ahead >= 4) wait_vm<3 * kItemOps>();
            else if (n_ahead == 3) wait_vm<2 * kItemOps>();
            else if (n_ahead == 2) wait_vm<kItemOps>();
            else wait_vm<0>();
          }
          const uint32_t src = ring_rd + slot * kItemBytes;
          uint4_t wq[4];
          uint32_t sA = 0, bA = 0, sB = 0, bB = 0;
#pragma unroll
          for (int L = 0; L < 4; ++L) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(wq[L]) : "v"(src + lane * 16), "n"(L * 1024));
          if (MC == 2) {
            // (scale[2kc], scale[2kc+1]) of row r: the groups of this lane's accumulator rows
            asm volatile("ds_read_b32 %0, %1 offset:4096" : "=v"(sA) : "v"(src + r * 16 + kc * 4));
            asm volatile("ds_read_b32 %0, %1 offset:4352" : "=v"(bA) : "v"(src + r * 16 + kc * 4));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wq[0]), "+v"(wq[1]), "+v"(wq[2]), "+v"(wq[3]), "+v"(sA), "+v"(bA));
          } else {
            // scale[kc] (half A) and scale[4 + kc] (half B) of row r
            asm volatile("ds_read_u16 %0, %1 offset:4096" : "=v"(sA) : "v"(src + r * 16 + kc * 2));
            asm volatile("ds_read_u16 %0, %1 offset:4104" : "=v"(sB) : "v"(src + r * 16 + kc * 2));
            asm volatile("ds_read_u16 %0, %1 offset:4352" : "=v"(bA) : "v"(src + r * 16 + kc * 2));
            asm volatile("ds_read_u16 %0, %1 offset:4360" : "=v"(bB) : "v"(src + r * 16 + kc * 2));
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(wq[0]), "+v"(wq[1]), "+v"(wq[2]), "+v"(wq[3]), "+v"(sA), "+v"(bA), "+v"(sB), "+v"(bB));
          }
          // ---- the slot is free: fetch the item NS ahead into it
          --n_ahead;
          if (prod.d < n_entries) {
            issue_item(prod, slot);
            ++n_ahead;
            ++ahead_after;
            next_item(prod);
          }
          slot = slot + 1 == NS ? 0 : slot + 1;
          // ---- multiply raw codes, then scale the group sums
          if (MC == 2) {
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int L = 0; L < 4; ++L)
#pragma unroll
              for (int w = 0; w < 4; ++w)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[L][w], raw_codes(wq[L][w], kMaskLo, kMaskHi, kMagicLo, kMagicHi),
                                                             acc, 0, 0, 0);
            const half2_t s2 = as_half2(sA), b2 = as_half2(bA);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              tot[j][e] = __builtin_fmaf((float)s2[e >> 1], acc[e] - corr[e], __builtin_fmaf((float)b2[e >> 1], xsum[e], tot[j][e]));
          } else {
            float4_t accA = {0.f, 0.f, 0.f, 0.f}, accB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int L = 0; L < 2; ++L)
#pragma unroll
              for (int w = 0; w < 4; ++w) {
                accA = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[L][w], raw_codes(wq[L][w], kMaskLo, kMaskHi, kMagicLo, kMagicHi),
                                                              accA, 0, 0, 0);
                accB = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[L + 2][w], raw_codes(wq[L + 2][w], kMaskLo, kMaskHi, kMagicLo, kMagicHi),
                                                              accB, 0, 0, 0);
              }
            float4_t cA, xA, cB, xB;  // group sums of this lane's accumulator rows, halves A and B
            asm volatile("ds_read_b128 %0, %1 offset:0" : "=v"(cA) : "v"(table_rd));
            asm volatile("ds_read_b128 %0, %1 offset:16" : "=v"(xA) : "v"(table_rd));
            asm volatile("ds_read_b128 %0, %1 offset:128" : "=v"(cB) : "v"(table_rd));
            asm volatile("ds_read_b128 %0, %1 offset:144" : "=v"(xB) : "v"(table_rd));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(cA), "+v"(xA), "+v"(cB), "+v"(xB));
            const float sa = (float)as_half2(sA)[0], sb = (float)as_half2(sB)[0];
            const float ba = (float)as_half2(bA)[0], bb = (float)as_half2(bB)[0];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float t = __builtin_fmaf(ba, xA[e], tot[j][e]);
              t = __builtin_fmaf(bb, xB[e], t);
              t = __builtin_fmaf(sa, accA[e] - cA[e], t);
              tot[j][e] = __builtin_fmaf(sb, accB[e] - cB[e], t);
            }
          }
        }
      }
      // ---- add up the groups: within the lane (MC 2: rows e and e + 2 are the same batch row),
      // then over the four slices kc; lanes kc == 0 drop the result into this wave's mailbox once
      // the reducer has emptied it
      float out[PR][MC];
#pragma unroll
      for (int j = 0; j < PR; ++j)
#pragma unroll
        for (int m = 0; m < MC; ++m) {
          float v = MC == 2 ? tot[j][m] + tot[j][m + 2] : tot[j][m];
          v += lane_read(v, lane ^ 16);
          v += lane_read(v, lane ^ 32);
          out[j][m] = v;
        }
      while (lds_load(&ctl->consumed) + 1 < q) __builtin_amdgcn_s_sleep(1);  // the box of pass q - 2 is free
      if (kc == 0) {
#pragma unroll
        for (int j = 0; j < PR; ++j)
          if (j < nj) {
#pragma unroll
            for (int m = 0; m < MC; ++m) mail[((q & 1) * kWaves + wave) * kMailFloats + (j * MC + m) * 16 + r] = out[j][m];
          }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the deposit is in LDS before it is counted
      if (lane == 0) __hip_atomic_fetch_add(&ctl->deposited[q & 1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  wait_vm<0>();
}

}  // namespace

// (external linkage: the host takes its address for hipFuncSetAttribute)
template <int MC, int NS>
__global__ __launch_bounds__(kThreadsAll) void gemv_stream_kernel(const void *entries, int n_entries, int *status, unsigned *words,
                                                                  unsigned spin_limit, const SequencePlan plan) {
  gemv_stream_body<MC, NS, false>(reinterpret_cast<const Entry *>(entries), n_entries, status, words, spin_limit, &plan, Entry{});
}

// one GEMV through the same body: what gq_gemv_f16 launches for large weights
template <int MC, int NS>
__global__ __launch_bounds__(kThreadsAll) void gemv_stream_single_kernel(const gq_gemv_desc desc) {
  Entry e;
  e.x = reinterpret_cast<const half_t *>(desc.x);
  e.packed = reinterpret_cast<const uint4_t *>(desc.packed);
  e.scale = reinterpret_cast<const half_t *>(desc.scale);
  e.bias = reinterpret_cast<const half_t *>(desc.bias);
  e.out_bias = reinterpret_cast<const half_t *>(desc.out_bias);
  e.y = reinterpret_cast<half_t *>(desc.y);
  e.m_rows = desc.m_rows;
  e.n_out = desc.n_out;
  e.k_in = desc.k_in;
  e.group_size = desc.group_size;
  e.wait_entries = 0;
  e.activation = desc.activation;
  // (an entry without a wait touches neither progress words nor exchange: no plan is read)
  gemv_stream_body<MC, NS, true>(nullptr, 1, nullptr, nullptr, 0u, nullptr, e);
}

namespace {

bool prepacked(const gq_gemv_desc &d) { return d.scale == nullptr && d.bias == nullptr; }

bool stream_shape_ok(const gq_gemv_desc &d) {
  return d.group_size == 64 && d.k_in % 512 == 0 && d.k_in > 0 && d.k_in <= (1 << 24) && d.m_rows >= 1 &&
         d.m_rows <= 4 && d.n_out >= 1 && d.n_out <= (1 << 22) && ((uintptr_t)d.x % 16) == 0 &&
         ((uintptr_t)d.packed % 16) == 0 && ((uintptr_t)d.scale % 16) == 0 && ((uintptr_t)d.bias % 16) == 0;
}

constexpr int kMaxDevices = 64;

// one workgroup per compute unit, all resident together; 0 with the error recorded
int stream_grid(int *dev_out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "hipGetDevice: %s", hipGetErrorString(e)), 0;
  static int cu_count[kMaxDevices] = {0};
  if (dev < 0 || dev >= kMaxDevices) return fail(GQ_ERR_UNSUPPORTED, "device index %d", dev), 0;
  if (cu_count[dev] == 0) {
    int n = 0;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || n <= 0) return fail((int)e, "cannot query the compute unit count"), 0;
    cu_count[dev] = n;
  }
  *dev_out = dev;
  return cu_count[dev] < kMaxGroups ? cu_count[dev] : kMaxGroups;
}

template <int MC, int NS>
constexpr int stream_lds_bytes() {
  return kWaves * (NS * kItemBytes + kStageBytes) + kMaxEntries * 64 + 2 * kWaves * pass_rows(MC) * MC * 16 * 4 + 64 +
         kWaves * 256 + kMaxGroups * 4;
}

}  // namespace

// One GEMV as a single-entry run of the persistent kernel; GQ_ERR_UNSUPPORTED (without an error
// text) if the shape is outside it.
int launch_gemv_streamed(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                         const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                         int64_t group_size, int act, hipStream_t stream) {
  if (m_rows > 4 || n_out > (1 << 22) || k_in > (1 << 24) || group_size != 64) return GQ_ERR_UNSUPPORTED;
  gq_gemv_desc d;
  d.x = x;
  d.packed = packed;
  d.scale = scale;
  d.bias = bias;
  d.out_bias = out_bias;
  d.y = y;
  d.m_rows = (int)m_rows;
  d.n_out = (int)n_out;
  d.k_in = (int)k_in;
  d.group_size = (int)group_size;
  d.wait_entries = 0;
  d.activation = act;
  if (!stream_shape_ok(d)) return GQ_ERR_UNSUPPORTED;
  int dev = 0;
  const int grid = stream_grid(&dev);
  if (grid == 0) return GQ_ERR_NO_DEVICE;
#define GQ_SINGLE(MC, NS)                                                                                     \
  do {                                                                                                        \
    constexpr int lds_bytes = stream_lds_bytes<MC, NS>();                                                     \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                    \
    auto kern = gemv_stream_single_kernel<MC, NS>;                                                            \
    static bool configured[kMaxDevices] = {false};                                                            \
    if (!configured[dev]) {                                                                                   \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                          \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);        \
      if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));              \
      configured[dev] = true;                                                                                 \
    }                                                                                                         \
    kern<<<dim3(grid), dim3(kThreadsAll), lds_bytes, stream>>>(d);                                            \
  } while (0)
  if (m_rows <= 2) GQ_SINGLE(2, 3);
  else GQ_SINGLE(4, 3);
#undef GQ_SINGLE
  return check_launch("gemv_stream_single_kernel");
}

int64_t gemv_sequence_workspace_bytes() { return (int64_t)kSequenceWords * 4; }

namespace {

bool overlap(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes) {
  const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
  return a0 < b0 + (uintptr_t)b_bytes && b0 < a0 + (uintptr_t)a_bytes;
}

// The plan of one launch (entries e[0..n), `first` entries of the sequence precede them and are
// complete when the launch starts; the launch runs on `grid` workgroups).
//
// Entry i reads its x through the exchange when x lies inside the results of an earlier entry p of
// the launch (the latest one that writes any of it) -- or, at batch 1, inside the results of several
// earlier entries that lie end to end in memory, each the latest to write its part -- and waiting
// for the tags is all the synchronisation the entry needs:
//   * what it declares to wait for is covered by the arrival of x.  Once every workgroup has
//     delivered its share of a producer q, every workgroup has also finished reading the inputs of
//     all entries up to q (a wave works through the entries in order) -- provided every workgroup
//     HAS a share of q, that is, q has at least one row block per workgroup.  So either the entry
//     waits for nothing past such a producer (wait_entries <= q + 1), or none of the entries it
//     waits for reads memory that this entry's y overwrites (then the declared wait orders nothing
//     but the arrival of x);
//   * out_bias is not a result of this launch, and results of the launch that y overwrites were
//     written with the same base and shape (then the same lane of the same workgroup wrote them, in
//     program order);
//   * the x chunks of a wave fit its stage at once (one phase, or all phases together), x starts
//     on a 16-byte unit of the first producer's results, and the exchange has room for the
//     producers, end to end like their results.
// Any other entry that reads results of this launch (x or out_bias) waits for the reported
// completion of their producer, whatever it declares: reported completion is what makes plain
// loads see them.
// any_fit: the consumer has no stage that the x chunks must fit (the data-flow kernel).
void plan_launch(const gq_gemv_desc *e, int n, int64_t first, bool any_fit, int grid, SequencePlan &plan) {
  constexpr int kMaxProducers = 4;
  struct Sources {
    int count;
    int16_t entry[kMaxProducers];  // in the order of their results in memory
  };
  static thread_local Sources sources[kMaxEntries];
  int64_t used_words = 0;
  plan.uses_exchange = 0;
  plan.exchange_values = 0;
  auto y_bytes_of = [&](int j) { return (int64_t)e[j].m_rows * e[j].n_out * 2; };
  for (int i = 0; i < n; ++i) {
    plan.ex_word[i] = plan.x_word[i] = -1;
    plan.x_src[i] = -1;
    Sources &from = sources[i];
    from.count = 0;
    const gq_gemv_desc &d = e[i];
    int need = (int)(d.wait_entries > first ? d.wait_entries - first : 0);
    const int64_t x_bytes = (int64_t)d.m_rows * d.k_in * 2, y_bytes = (int64_t)d.m_rows * d.n_out * 2;
    int src = -1, bias_src = -1;
    bool same_owner = true;
    for (int j = i - 1; j >= 0; --j) {
      if (src < 0 && overlap(d.x, x_bytes, e[j].y, y_bytes_of(j))) src = j;
      if (bias_src < 0 && d.out_bias && overlap(d.out_bias, (int64_t)d.n_out * 2, e[j].y, y_bytes_of(j))) bias_src = j;
      if (overlap(d.y, y_bytes, e[j].y, y_bytes_of(j)) && !(e[j].y == d.y && e[j].n_out == d.n_out && e[j].m_rows == d.m_rows))
        same_owner = false;
    }
    if (src >= 0) {
      // the producers of x, from its first byte on: each the latest entry that writes the byte
      // where the one before ends, and nothing later writes into its part
      const char *at = (const char *)d.x, *const end = at + x_bytes;
      bool whole = true;
      int latest = -1;
      while (at < end && whole) {
        int p = -1;
        for (int j = i - 1; j >= 0 && p < 0; --j)
          if ((const char *)e[j].y <= at && at < (const char *)e[j].y + y_bytes_of(j)) p = j;
        whole = p >= 0 && from.count < kMaxProducers;
        if (!whole) break;
        const char *p_end = (const char *)e[p].y + y_bytes_of(p);
        const char *part_end = p_end < end ? p_end : end;
        for (int j = p + 1; j < i && whole; ++j) whole = !overlap(at, part_end - at, e[j].y, y_bytes_of(j));
        // several producers: batch 1 only (rows of x would not be contiguous otherwise), each but
        // the first read from its first result on
        if (from.count > 0 || part_end < end) whole = whole && d.m_rows == 1 && e[p].m_rows == 1;
        if (from.count > 0) whole = whole && at == (const char *)e[p].y;
        from.entry[from.count++] = (int16_t)p;
        if (p > latest) latest = p;
        at = part_end;
      }
      const int64_t off = (const char *)d.x - (const char *)e[from.entry[0]].y;
      const int phases = (d.k_in + 4095) / 4096;
      const bool fits = any_fit || phases == 1 || (int64_t)phases * d.m_rows * 1024 <= kStageBytes;
      // what the declared wait asks for beyond the arrival of x
      bool covered = need == 0;
      for (int s = 0; s < from.count && whole && !covered; ++s) {
        const int q = from.entry[s];
        covered = need <= q + 1 && (e[q].n_out + 15) / 16 >= grid;
      }
      if (whole && !covered && need <= latest + 1) {
        covered = true;  // unless an entry it waits for reads what y overwrites
        for (int j = 0; j < need && covered; ++j)
          covered = !overlap(d.y, y_bytes, e[j].x, (int64_t)e[j].m_rows * e[j].k_in * 2) &&
                    !(e[j].out_bias && overlap(d.y, y_bytes, e[j].out_bias, (int64_t)e[j].n_out * 2));
      }
      const bool tagged = whole && off % 16 == 0 && fits && covered && bias_src < 0 && same_owner;
      if (tagged) {
        plan.x_src[i] = (int16_t)latest;
      } else {
        from.count = 0;
        if (need < src + 1) need = src + 1;
      }
    }
    if (bias_src >= 0 && need < bias_src + 1) need = bias_src + 1;
    plan.need[i] = (int16_t)need;
  }
  // room in the exchange: the producers of one x end to end, in the order of their results
  for (int i = 0; i < n; ++i) {
    const Sources &from = sources[i];
    for (int s = 0; s < from.count; ++s) {
      const int p = from.entry[s];
      if (plan.ex_word[p] >= 0) continue;
      const int64_t words = ((int64_t)e[p].m_rows * e[p].n_out + 63) / 64 * 64;
      if (used_words + words > kExchangeWords) break;
      plan.ex_word[p] = (int32_t)used_words;
      used_words += words;
      plan.uses_exchange = 1;
    }
  }
  plan.exchange_values = (int32_t)used_words;
  for (int i = 0; i < n; ++i) {
    const Sources &from = sources[i];
    if (from.count == 0) continue;
    bool placed = true;
    for (int s = 0; s < from.count && placed; ++s) {
      const int p = from.entry[s];
      placed = plan.ex_word[p] >= 0 &&
               (s == 0 || plan.ex_word[p] == plan.ex_word[from.entry[s - 1]] + e[from.entry[s - 1]].n_out);
    }
    if (!placed) {  // no room, or not end to end: wait for the producers' reported completion instead
      const int latest = plan.x_src[i];
      plan.x_src[i] = -1;
      if (plan.need[i] < latest + 1) plan.need[i] = (int16_t)(latest + 1);
      continue;
    }
    plan.need[i] = 0;
    const int p0 = from.entry[0];
    plan.x_word[i] = plan.ex_word[p0] + (int32_t)(((const char *)e[i].x - (const char *)e[p0].y) / 2);
  }
  for (int i = 0; i < n; ++i) {
    plan.x_id[i] = (int16_t)i;
    for (int j = 0; j < i; ++j)
      if (e[j].x == e[i].x && plan.x_word[j] == plan.x_word[i] && plan.x_src[j] == plan.x_src[i] && e[j].k_in == e[i].k_in &&
          e[j].m_rows == e[i].m_rows) {
        plan.x_id[i] = (int16_t)j;
        break;
      }
  }
}

}  // namespace

int launch_gemv_sequence(const gq_gemv_desc *host, const gq_gemv_desc *device, int64_t count, int *status,
                         void *workspace, int64_t spin_limit, hipStream_t stream) {
  if (count > (1 << 20)) return fail(GQ_ERR_UNSUPPORTED, "gq_gemv_sequence_f16: more than 2^20 entries");
  // Runs of consecutive entries that the persistent kernels cover (group 64, k_in % 512 == 0, m_rows <= 4,
  // 16-byte aligned, groups along the input features) go to them, up to kMaxEntries per launch; every
  // other entry is a launch of its own.  Launches execute in stream order, so whatever an entry
  // waits for in an earlier launch is complete when it starts.
  auto persistent = [&](int64_t i) { return !(host[i].activation & GQ_DESC_KN_LAYOUT) && stream_shape_ok(host[i]); };
  bool any_persistent = false;
  for (int64_t i = 0; i < count; ++i) {
    if (persistent(i)) {
      any_persistent = true;
    } else if (prepacked(host[i]) && !(host[i].activation & GQ_DESC_KN_LAYOUT)) {
      // (a launch of its own: batches of 5 to 16 rows; the one-shot kernel reads the streaming layout too)
      const gq_gemv_desc &d = host[i];
      if (!(d.group_size == 64 && d.k_in > 0 && d.k_in % 512 == 0 && ((uintptr_t)d.x % 16) == 0 && ((uintptr_t)d.packed % 16) == 0))
        return fail(GQ_ERR_UNSUPPORTED,
                    "gq_gemv_sequence_f16: entry %lld is in the streaming layout, which needs group 64, k_in %% 512 == 0 "
                    "and 16-byte aligned x and weight", (long long)i);
    }
  }
  int dev = 0, grid = 0;
  unsigned *words = static_cast<unsigned *>(workspace);
  if (any_persistent) {
    grid = stream_grid(&dev);
    if (grid == 0) return GQ_ERR_NO_DEVICE;
    if (!words) {
      // the library's own block of this device (its address differs from device to device)
      static SharedBlockGuard guard = {};
      const int claimed = claim_shared_block(guard, dev, stream, "gq_gemv_sequence_f16");
      if (claimed != GQ_OK) return claimed;
      static unsigned *own[kMaxDevices] = {nullptr};
      if (!own[dev]) {
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_sequence_words));
        if (e != hipSuccess || !ptr) return fail((int)e, "hipGetSymbolAddress(progress words): %s", hipGetErrorString(e));
        own[dev] = static_cast<unsigned *>(ptr);
      }
      words = own[dev];
    }
  }
  const unsigned spins = spin_limit > 0 ? (unsigned)(spin_limit < 0x7fffffff ? spin_limit : 0x7fffffff) : kDefaultSpinLimit;
#define GQ_STREAM(MC, NS)                                                                                     \
  do {                                                                                                        \
    constexpr int lds_bytes = stream_lds_bytes<MC, NS>();                                                     \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                    \
    auto kern = gemv_stream_kernel<MC, NS>;                                                                   \
    static bool configured[kMaxDevices] = {false};                                                            \
    if (!configured[dev]) {                                                                                   \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                          \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);        \
      if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));              \
      configured[dev] = true;                                                                                 \
    }                                                                                                         \
    kern<<<dim3(grid), dim3(kThreadsAll), lds_bytes, stream>>>(device + first, n, status, words, spins, plan); \
  } while (0)
  int64_t first = 0;
  while (first < count) {
    if (!persistent(first)) {
      const gq_gemv_desc &d = host[first];
      const int act = d.activation & ~GQ_DESC_KN_LAYOUT;
      const int rc = (d.activation & GQ_DESC_KN_LAYOUT)
                         ? launch_gemv_knp(d.x, d.m_rows, d.packed, d.out_bias, d.y, d.n_out, d.k_in, act, stream)
                         : launch_gemv(d.x, d.m_rows, d.packed, d.scale, d.bias, d.out_bias, d.y, d.n_out, d.k_in,
                                       d.group_size, act, stream, prepacked(d) ? d.packed : nullptr);
      if (rc != GQ_OK) return rc;
      ++first;
      continue;
    }
    int n = 0, max_m = 1;
    while (n < kMaxEntries && first + n < count && persistent(first + n)) {
      if (host[first + n].m_rows > max_m) max_m = host[first + n].m_rows;
      ++n;
    }
    SequencePlan plan;
    // launches of weights in the streaming layout whose dependencies all travel through the exchange
    // run on the data-flow kernel of gq_gemv_flow.hip
    plan_launch(host + first, n, first, true, grid, plan);
    if (flow_eligible(host + first, n, plan)) {
      const int rc = launch_flow(host + first, device + first, n, status, words, spins, plan, grid, dev, stream);
      if (rc != GQ_OK) return rc;
    } else {
      plan_launch(host + first, n, first, false, grid, plan);
      if (max_m <= 2) GQ_STREAM(2, 3);
      else GQ_STREAM(4, 3);
      const int rc = check_launch("gemv_stream_kernel");
      if (rc != GQ_OK) return rc;
    }
    first += n;
  }
#undef GQ_STREAM
  return GQ_OK;
}

// ---- the streaming layout: block (rb, c) = what the ring slot of work item (rb, c) holds
namespace {

__global__ __launch_bounds__(256) void prepack_kernel(const char *__restrict__ packed, const char *__restrict__ scale,
                                                      const char *__restrict__ bias, uint4_t *__restrict__ blob, int n_out,
                                                      int k_in, int64_t units) {
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;  // 16-byte unit of the blob
  if (u >= units) return;
  constexpr int kUnits = kItemBytes / 16;
  const int64_t block = u / kUnits;
  const int w = (int)(u % kUnits), chunks = k_in >> 9;
  const int64_t rb = block / chunks;
  const int c = (int)(block % chunks);
  const int r = w & 15;
  const int64_t row = rb * 16 + r;
  uint4_t v = {0u, 0u, 0u, 0u};  // rows past n_out: code 0, scale 0, bias 0
  if (row < n_out) {
    if (w < 256) {
      const int s = w >> 6, kc = (w >> 4) & 3;  // slot layout [s][kc][r]: bytes s * 64 + kc * 16 of the row's chunk
      v = *reinterpret_cast<const uint4_t *>(packed + row * (k_in >> 1) + c * 256 + s * 64 + kc * 16);
    } else {
      const char *src = w < 272 ? scale : bias;  // the 8 values of the row's chunk
      v = *reinterpret_cast<const uint4_t *>(src + row * (k_in >> 5) + c * 16);
    }
  }
  blob[u] = v;
}

}  // namespace

int64_t gemv_prepacked_bytes(int64_t n_out, int64_t k_in) { return ((n_out + 15) / 16) * (k_in / 512) * kItemBytes; }

int launch_gemv_prepack(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob, int64_t n_out,
                        int64_t k_in, hipStream_t stream) {
  const int64_t units = gemv_prepacked_bytes(n_out, k_in) / 16;
  const int64_t blocks = (units + 255) / 256;
  if (blocks > 0x7fffffff) return fail(GQ_ERR_UNSUPPORTED, "gq_gemv_prepack_f16: weight too large");
  prepack_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
      reinterpret_cast<const char *>(packed), reinterpret_cast<const char *>(scale), reinterpret_cast<const char *>(bias),
      reinterpret_cast<uint4_t *>(blob), (int)n_out, (int)k_in, units);
  return check_launch("prepack_kernel");
}

}  // namespace gq
