// Declarations shared by the two persistent GEMV-sequence kernels of libgq_hip (gfx950): the
// layout of the per-sequence block of progress words and of the two exchanges, the launch plan
// that the host works out, and small device helpers.
#pragma once
#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {

constexpr int kWaves = 8;                         // compute waves
constexpr int kThreadsAll = (kWaves + 2) * 64;    // + reducer + poller
constexpr int kItemBytes = 4096 + 512;  // packed words, 16 rows x 16 B of scale, 16 rows x 16 B of bias
constexpr int kItemOps = 6;             // direct-to-LDS loads per item: 4 packed + scale + bias
// row blocks per pass (a wave holds their running sums in registers and re-uses the x operands
// for them); the variant for 4 batch rows has fewer registers to spare
constexpr int pass_rows(int mc) { return mc == 2 ? 4 : 2; }
constexpr unsigned kDefaultSpinLimit = 1u << 18;  // polls without progress before a poller gives up
constexpr int kStageBytes = 4096;       // x stage of a wave: 1 KiB per (chunk, batch row)

// Progress of a running sequence: a block of words in device memory that the caller provides per
// sequence (gq_gemv_sequence_ws_f16) or that the library keeps per device (gq_gemv_sequence_f16: one
// sequence at a time).  Every workgroup publishes the number of
// entries it has completed in its own word (plain device-scope stores: 256 read-modify-writes of
// one counter per entry would serialise at the memory side); the last workgroup to leave the
// kernel clears the words.  Each word has a 128-byte line to itself: with 32 words to a line every
// store hit a line that all 256 pollers were reading, and the stream of weights lost 4 - 5 us per
// published entry (measured: polling lines that nobody writes, or writing lines that nobody
// polls, costs nothing).
// For the same reason only ONE poller, the watcher (workgroup 0), reads those words; it announces
// the count that is complete everywhere in a word of its own, which all other pollers watch (one
// more hop for a wait that is exposed; measured: one watcher beats eight, and a watcher workgroup
// without rows of its own loses more to the uneven split of the row blocks than it gains).
constexpr int kMaxGroups = 256;  // (the watcher keeps a copy of every progress word in LDS)
constexpr int kMaxEntries = 128;  // per launch (8 KiB of LDS)
constexpr int kProgressStride = 32;  // words
// layout of the block: [kMaxGroups] progress lines, the watcher's announcement, the count of
// workgroups that have left the kernel (a line each); all zero between launches
constexpr int kAnnouncedWord = kMaxGroups * kProgressStride;
constexpr int kExitedWord = kAnnouncedWord + kProgressStride;
constexpr int kEpochWord = kExitedWord + kProgressStride;
// The exchange: results that a later entry of the same launch reads as its x are also written here
// as 32-bit words (tag << 16 | fp16 value), the tag being the launch's epoch (1..65535, kept in the
// block, advanced by the last workgroup to leave).  A consumer loads the words and knows from the
// tags alone that every value has arrived: no wait for the producers' stores to complete, no
// progress report, no reload of x after a flag -- three memory round trips less per dependency.
// Stale words carry older tags; when the epoch wraps, the last workgroup out clears the exchange.
constexpr int kExchangeWord = (kEpochWord + kProgressStride + 63) / 64 * 64;  // 256-byte aligned
constexpr int kExchangeWords = (16 << 20) / 4;
// The exchange of the data-flow kernel (gq_gemv_flow.hip): two halves of kExchangeWords fp16 values
// each, used by launches in turn.  A result y is stored as the fp16 bits of -y (zero as -0.0), so
// that the all-zero pattern means "not written yet"; a launch finds its half clean and cleans,
// while it starts, what the launch before it left in the other half.  Words of its own, a line
// each: the count of launches so far (its parity selects the half), the fp16 values that may be
// non-zero in either half, the count of workgroups that have left.
constexpr int kFlowEpochWord = kExchangeWord + kExchangeWords;
constexpr int kFlowExtentWord = kFlowEpochWord + kProgressStride;  // [2]
constexpr int kFlowExitedWord = kFlowExtentWord + kProgressStride;
constexpr int kFlowExchangeWord = kFlowExitedWord + kProgressStride + 32;  // 256-byte aligned
constexpr int kFlowHalfValues = kExchangeWords;                             // fp16 values per half
constexpr int kSequenceWords = kFlowExchangeWord + 2 * (kFlowHalfValues / 2);
static_assert(kFlowExchangeWord % 64 == 0, "alignment of the exchange");

}  // namespace

// What the host works out for a launch (a kernel argument): which entries read results of the
// launch through the exchange, and which have to wait for reported completion.
struct SequencePlan {
  int32_t ex_word[kMaxEntries];  // producer: where the entry's tagged results start in the exchange (-1: none)
  int32_t x_word[kMaxEntries];   // consumer: where its x starts in the exchange (-1: x is read from memory)
  int16_t x_src[kMaxEntries];    // consumer: the entry (of this launch) that produces its x (-1: none)
  int16_t x_id[kMaxEntries];     // the first entry of the launch that reads the same x (same place, same producer, same shape)
  int16_t need[kMaxEntries];     // entries of this launch that must be reported complete before this one starts
  int32_t uses_exchange;
  int32_t exchange_values;       // results the launch puts into the exchange (a multiple of 64)
};

// the data-flow kernel (gq_gemv_flow.hip): launches of weights in the streaming layout whose
// dependencies all travel through the exchange
bool flow_eligible(const gq_gemv_desc *entries, int n, const SequencePlan &plan);
int launch_flow(const gq_gemv_desc *host, const gq_gemv_desc *device, int n, int *status, unsigned *words,
                unsigned spin_limit, const SequencePlan &plan, int grid, int dev, hipStream_t stream);

namespace {

struct Entry {  // = gq_gemv_desc
  const half_t *x;
  const uint4_t *packed;
  const half_t *scale;
  const half_t *bias;
  const half_t *out_bias;
  half_t *y;
  int32_t m_rows, n_out, k_in, group_size, wait_entries, activation;
};
static_assert(sizeof(Entry) == sizeof(gq_gemv_desc), "descriptor layout");

template <int N>
__device__ __forceinline__ void wait_vm() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// position of a wave in the list of its work items
struct Cursor {
  int d, pass, phase, j;  // entry, pass of row blocks, phase of 4096 indices, row block in pass
};

// what the kernel needs of an entry, kept in LDS: descriptor reads from global memory in the
// work loop cost microseconds each
struct CachedEntry {
  const char *packed, *scale, *bias;
  const half_t *x, *out_bias;
  half_t *y;
  int n_out, k_in;
  short m_rows, wait;  // wait: entries of this launch that must be complete before this one starts
  short nrb;           // row blocks owned by this workgroup
  char publish;        // somebody waits for exactly this entry and its predecessors: report its completion
  char act;            // GQ_ACT_* epilogue
};
static_assert(sizeof(CachedEntry) == 64, "entry cache layout");

// cache policy of a direct-to-LDS load: sc1 = device (agent) scope, the policy the compiler gives an
// agent-scope atomic load; it pairs with the agent-scope stores of y and of the progress words
// (sc0 | sc1, system scope, costs another 2 % of a pass)
constexpr int kAuxDeviceCoherent = 1 << 4;
// cache policy of the weight loads (read once)
#ifndef GQ_WEIGHT_AUX
#define GQ_WEIGHT_AUX 0
#endif
constexpr int kAuxWeights = GQ_WEIGHT_AUX;

// LDS words shared by the waves of a workgroup
struct Control {
  unsigned deposited[2];  // mailbox deposits so far, passes of even and of odd number (8 per pass)
  unsigned consumed;      // passes whose mailboxes the reducer has read
  unsigned ready;         // entries known to be complete on the whole device
  unsigned failed;        // a poller gave up
  unsigned published;     // entries this workgroup has reported complete (progress word written)
  unsigned targets[4];    // bit w - 1 set: some entry waits for the first w entries (kMaxEntries bits)
  unsigned tag;           // this launch's epoch << 16
  unsigned stored;        // entries whose results this workgroup's reducer has stored (stores issued)
};
static_assert(sizeof(Control) <= 64, "control block");

__device__ __forceinline__ unsigned lds_load(const unsigned *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// LDS read the compiler does not see as such: after a direct-to-LDS load it makes every LDS read
// that might alias wait for ALL outstanding loads
__device__ __forceinline__ unsigned lds_peek(const unsigned *p) {
  unsigned v;
  asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"((uint32_t)(uintptr_t)p) : "memory");
  return v;
}

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const char *uni_ptr(const void *p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  return (const char *)(uintptr_t)(((uint64_t)(uint32_t)uni((int)(v >> 32)) << 32) | (uint32_t)uni((int)v));
}
__device__ __forceinline__ float lane_read(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v)));
}

// 8 codes of `w` as fp16 (64 + c) or (1024 + c), order (0,4,1,5,2,6,3,7): 5 VALU instructions.
// Codes 0,2 (and 4,6) sit at bits 7:4 of a byte and land in the mantissa of 64.0 (ulp 1/16 x 16);
// codes 1,3 (5,7) sit at bits 3:0 and land in the mantissa of 1024.0 (ulp 1).
__device__ __forceinline__ half8_t raw_codes(uint32_t w, uint32_t mask_lo, uint32_t mask_hi, uint32_t magic_lo,
                                             uint32_t magic_hi) {
  const uint32_t hi = w >> 8;
  uint4_t v;
  v.x = and_or(hi, mask_hi, magic_hi);  // codes 0, 4: 64 + c
  v.y = and_or(hi, mask_lo, magic_lo);  // codes 1, 5: 1024 + c
  v.z = and_or(w, mask_hi, magic_hi);   // codes 2, 6: 64 + c
  v.w = and_or(w, mask_lo, magic_lo);   // codes 3, 7: 1024 + c
  return __builtin_bit_cast(half8_t, v);
}

}  // namespace
}  // namespace gq
