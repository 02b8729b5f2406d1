// A sequence of fused dequant-GEMVs as ONE persistent kernel (decode of a layer stack).
//
// Launching a GEMV per weight matrix leaves HBM idle between kernels: ~2 us of launch, ramp and
// drain for every 1.3 - 5 us of weight streaming.  Here one workgroup per compute unit walks the
// whole list of entries.  Packed weights, scales and biases never depend on earlier results, so
// every wave streams them through a private LDS ring with direct-to-LDS loads that run several
// work items ahead -- across entry boundaries -- while only the small activation vector x waits
// for the entries it depends on (a device-wide counter, bounded spin).
//
// Work decomposition of one entry (n_out x k_in, k_in % 512 == 0, group 64, m_rows <= MCAP):
//   row block  = 16 weight rows; workgroup b of G owns row blocks b, b + G, ... in passes of 4
//   phase      = 4096 contraction indices; wave w owns chunk 8 p + w (512 indices) of phase p
//   work item  = (row block, chunk): 4 KiB of packed words + 2 x 256 B of scale / bias
// A wave keeps the permuted x fragments of its chunk in registers and re-uses them for the row
// blocks of the pass; the 16 x 16 partial sums of the 8 waves meet in LDS at the end of a pass.
// The arithmetic is that of gemv_mfma_kernel (v_mfma_f32_16x16x32_f16, codes expanded in pair
// order, x permuted to match).
#include "gq_common.h"
#include "gq_gemv_dequant.h"

namespace gq {
namespace {

constexpr int kWaves = 8;                         // compute waves
constexpr int kThreadsAll = (kWaves + 2) * 64;    // + reducer + poller
constexpr int kItemBytes = 4096 + 512;  // packed words, 16 rows x 16 B of scale, 16 rows x 16 B of bias
constexpr int kItemOps = 5;             // direct-to-LDS loads per item: 4 packed + 1 scale/bias
constexpr int kPassRows = 4;            // row blocks per pass (accumulators held by a wave)
constexpr unsigned kSpinLimit = 1u << 18;

// Progress of the running sequence on this device.  Every workgroup publishes the number of
// entries it has completed in its own word (plain device-scope stores: 256 read-modify-writes of
// one counter per entry would serialise at the memory side); the last workgroup to leave the
// kernel clears the words.
constexpr int kMaxGroups = 1024;
__device__ __attribute__((aligned(16))) unsigned int g_progress[kMaxGroups];
__device__ unsigned int g_exited;  // workgroups that left the kernel

struct Entry {  // = gq_gemv_desc
  const half_t *x;
  const uint4_t *packed;
  const half_t *scale;
  const half_t *bias;
  const half_t *out_bias;
  half_t *y;
  int32_t m_rows, n_out, k_in, group_size, wait_previous, reserved;
};
static_assert(sizeof(Entry) == sizeof(gq_gemv_desc), "descriptor layout");

template <int N>
__device__ __forceinline__ void wait_vm() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// position of a wave in the list of its work items
struct Cursor {
  int d, pass, phase, j;  // entry, pass of 4 row blocks, phase of 4096 indices, row block in pass
};

// what the kernel needs of an entry, kept in LDS: descriptor reads from global memory in the
// work loop cost microseconds each
struct CachedEntry {
  const uint4_t *packed;
  const half_t *scale, *bias, *x, *out_bias;
  half_t *y;
  int n_out, k_in;
  short m_rows, wait_previous;
  int nrb;  // row blocks owned by this workgroup
};
static_assert(sizeof(CachedEntry) == 64, "entry cache layout");
constexpr int kMaxEntries = 128;  // per launch (8 KiB of LDS)

// cache policy of a direct-to-LDS load: sc0 | sc1 = coherent at device scope (bypasses the L1 of
// the compute unit and the non-coherent part of the L2 of its XCD)
constexpr int kAuxDeviceCoherent = (1 << 0) | (1 << 4);

// LDS words shared by the waves of a workgroup
struct Control {
  unsigned deposited;  // mailbox deposits so far (8 per pass)
  unsigned consumed;   // passes whose mailboxes the reducer has read
  unsigned ready;      // entries known to be complete on the whole device
  unsigned failed;     // the poller gave up
};

__device__ __forceinline__ unsigned lds_load(const unsigned *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// MCAP: largest batch (the x stage of a wave holds MCAP KiB); NS: depth of the weight ring.
// (A __device__ function: a __global__ template is also instantiated for the host, where the
// target builtins and inline assembly do not exist.)
//
// Waves 0..7 compute; they never meet at a workgroup barrier.  After the last chunk of a pass a
// wave drops its 16 x m partial sums into its mailbox and goes on with the next pass or entry.
// Wave 8, the reducer, adds the eight mailboxes in a fixed order, stores y and counts the
// workgroup as arrived for the entry.  Wave 9, the poller, watches the device-wide arrival count
// and publishes in LDS how many entries are complete; a compute wave that needs an earlier result
// waits for that number only.
//
// Visibility of results between compute units needs no cache flush: y is written with device-scope
// stores (sc1, write-through to the coherent level), the reducer waits for its stores before it
// counts, and x is read with device-coherent loads.
template <int MCAP, int NS>
__device__ __forceinline__ void gemv_stream_body(const Entry *__restrict__ entries, int n_entries,
                                                 int *__restrict__ status) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int kWaveBytes = NS * kItemBytes + MCAP * 1024;
  constexpr int kMailBytes = kPassRows * 4 * MCAP * 16;  // per wave: [row block][kc][m] float4
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int G = gridDim.x, b = blockIdx.x;
  CachedEntry *cache = reinterpret_cast<CachedEntry *>(lds + kWaves * kWaveBytes);
  char *mail = lds + kWaves * kWaveBytes + kMaxEntries * 64;
  Control *ctl = reinterpret_cast<Control *>(mail + kWaves * kMailBytes);

  for (int i = tid; i < n_entries; i += kThreadsAll) {
    const Entry e = entries[i];
    CachedEntry c;
    c.packed = e.packed;
    c.scale = e.scale;
    c.bias = e.bias;
    c.x = e.x;
    c.out_bias = e.out_bias;
    c.y = e.y;
    c.n_out = e.n_out;
    c.k_in = e.k_in;
    c.m_rows = (short)e.m_rows;
    c.wait_previous = (short)(e.wait_previous != 0);
    const int rb = (e.n_out + 15) >> 4;
    c.nrb = rb > b ? (rb - b + G - 1) / G : 0;
    cache[i] = c;
  }
  if (tid == 0) *ctl = Control{0u, 0u, 0u, 0u};
  __syncthreads();  // the only workgroup barrier

  auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };

  // ============================================================================ poller
  if (wave == kWaves + 1) {
    int last_waited = 0;
    for (int d = 1; d < n_entries; ++d)
      if (cache[d].wait_previous) last_waited = d;
    // one 16-byte device-coherent load per lane covers 256 workgroups; the minimum over all of them
    // is the number of entries complete everywhere
    unsigned ready = 0, spins = 0;
    const int rounds = (G + 255) >> 8;
    while (ready < (unsigned)last_waited) {
      unsigned lo = 0xffffffffu;
      for (int k = 0; k < rounds; ++k) {
        const int first = (k * 64 + lane) * 4;
        uint4_t v;
        asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)"
                     : "=v"(v)
                     : "v"(g_progress + first)
                     : "memory");
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (first + i < G) lo = min(lo, v[i]);
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) lo = min(lo, (unsigned)__shfl_xor((int)lo, off, 64));
      if (lo > ready) {
        ready = lo;
        if (lane == 0) __hip_atomic_store(&ctl->ready, ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        spins = 0;
      } else if (++spins > kSpinLimit) {  // some workgroup is not running: give up, let everybody finish
        if (lane == 0) {
          __hip_atomic_store(&ctl->failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          if (status) atomicExch(status, 1);
        }
        break;
      }
    }
    return;
  }

  // =========================================================================== reducer
  if (wave == kWaves) {
    unsigned q = 0;  // passes reduced so far
    for (int d = 0; d < n_entries; ++d) {
      const int nrb = uni(cache[d].nrb), m_rows = uni(cache[d].m_rows), n_out = uni(cache[d].n_out);
      half_t *y = cache[d].y;
      const half_t *out_bias = cache[d].out_bias;
      for (int pass = 0; pass * kPassRows < nrb; ++pass, ++q) {
        const int nj = min(kPassRows, nrb - pass * kPassRows);
        while (lds_load(&ctl->deposited) < (q + 1) * kWaves) __builtin_amdgcn_s_sleep(1);
        // lane -> (row block j, kc, m): 16 lanes per row block when MCAP == 4
        for (int t = lane; t < nj * 4 * MCAP; t += 64) {
          const int m = t % MCAP, kq = (t / MCAP) & 3, j = t / (4 * MCAP);
          float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int w = 0; w < kWaves; ++w) sum += *reinterpret_cast<const float4_t *>(mail + w * kMailBytes + t * 16);
          if (m < m_rows) {
            const int n0 = (b + (pass * kPassRows + j) * G) * 16 + 4 * kq;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int n = n0 + i;
              if (n < n_out) {
                float v = sum[i];
                if (out_bias) v += (float)out_bias[n];
                const half_t hv = (half_t)v;
                // device-scope store: written through to where every compute unit reads it
                __hip_atomic_store(reinterpret_cast<unsigned short *>(y) + (int64_t)m * n_out + n,
                                   __builtin_bit_cast(unsigned short, hv), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              }
            }
          }
        }
        // the mailboxes have been read (the sums above depend on them): free them
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_store(&ctl->consumed, q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      wait_vm<0>();  // every lane's stores of this entry are complete ...
      if (lane == 0)   // ... then publish
        __hip_atomic_store(&g_progress[b], (unsigned)d + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // the last workgroup out clears the progress words: by then every poller has seen all it needs
    wait_vm<0>();  // this workgroup's last progress word is in memory before it counts itself out
    unsigned last = 0;
    if (lane == 0) last = atomicAdd(&g_exited, 1u) == (unsigned)G - 1;
    if (__builtin_amdgcn_readfirstlane((int)last)) {
      wait_vm<0>();
      for (int i = lane; i < G; i += 64) __hip_atomic_store(&g_progress[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0) __hip_atomic_store(&g_exited, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
  }

  // ==================================================================== compute waves
  char *ring = lds + wave * kWaveBytes;
  char *xstage = ring + NS * kItemBytes;
  const uint32_t ring_rd = (uint32_t)(uintptr_t)ring, x_rd = (uint32_t)(uintptr_t)xstage;
  const uint32_t half_sel = (kc & 2) ? 0x07060706u : 0x05040504u;  // lane's group within a slot: kc / 2

  // The producer walks the same item list as the consumer, NS items ahead.  Its entry is held in
  // scalar registers (values read from LDS are made wave-uniform explicitly), so that advancing
  // the cursor is a handful of scalar instructions.
  auto uni_ptr = [&](const void *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    return (const char *)(uintptr_t)(((uint64_t)(uint32_t)uni((int)(v >> 32)) << 32) | (uint32_t)uni((int)v));
  };
  struct ProducerEntry {
    const char *packed, *scale, *bias;
    int n_out, k_in, nrb, phases;
  } pe = {nullptr, nullptr, nullptr, 1, 512, 0, 1};
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
    return c.pass * kPassRows + c.j < pe.nrb && (c.phase * kWaves + wave) * 512 < pe.k_in;
  };
  auto step = [&](Cursor &c) {
    if (++c.j < kPassRows && c.pass * kPassRows + c.j < pe.nrb) return;
    c.j = 0;
    if (++c.phase < pe.phases) return;
    c.phase = 0;
    if (++c.pass * kPassRows < pe.nrb) return;
    c.pass = 0;
    ++c.d;
    load_producer_entry(c.d);
  };
  auto next_item = [&](Cursor &c) {
    do step(c);
    while (c.d < n_entries && !valid(c));
  };
  // direct-to-LDS loads of the item at cursor c into ring slot `slot`
  auto issue_item = [&](const Cursor &c, int slot) {
    const int rb = b + (c.pass * kPassRows + c.j) * G;
    const int row = min(rb * 16 + r, pe.n_out - 1);
    const int chunk = c.phase * kWaves + wave;
    char *dst = ring + slot * kItemBytes;
    const uint4_t *src = reinterpret_cast<const uint4_t *>(pe.packed) + (int64_t)row * (pe.k_in >> 5) + chunk * 16 + kc;
#pragma unroll
    for (int s = 0; s < 4; ++s) __builtin_amdgcn_global_load_lds(src + s * 4, dst + s * 1024, 16, 0, 0);
    // lanes kc == 0 fetch the 8 scales of their row's chunk, lanes kc == 1 the 8 biases
    if (kc < 2) {
      const half_t *sb = reinterpret_cast<const half_t *>(kc == 0 ? pe.scale : pe.bias) + (int64_t)row * (pe.k_in >> 6) + chunk * 8;
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(sb), dst + 4096, 16, 0, 0);
    }
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

  half8_t xp[4][4];
  const half_t *x_loaded = nullptr;  // x fragments in registers belong to (x_loaded, chunk x_chunk)
  int x_chunk = -1, x_k = 0, x_m = 0;

  for (int d = 0; d < n_entries; ++d) {
    const int nrb = uni(cache[d].nrb), m_rows = uni(cache[d].m_rows), k_in = uni(cache[d].k_in);
    const half_t *x = reinterpret_cast<const half_t *>(uni_ptr(cache[d].x));
    const int phases = (k_in + 4095) >> 12;
    if (uni(cache[d].wait_previous) && d > 0) {
      // every workgroup has finished every earlier entry (published by the poller)
      while (lds_load(&ctl->ready) < (unsigned)d && !lds_load(&ctl->failed)) __builtin_amdgcn_s_sleep(1);
      x_loaded = nullptr;
    }
    for (int pass = 0; pass * kPassRows < nrb; ++pass, ++q) {
      const int nj = min(kPassRows, nrb - pass * kPassRows);
      float4_t acc[kPassRows];
#pragma unroll
      for (int j = 0; j < kPassRows; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
      for (int phase = 0; phase < phases; ++phase) {
        const int chunk = phase * kWaves + wave;
        if (chunk * 512 >= k_in) continue;
        // ---- x fragments of this chunk (kept when the previous entry used the same ones)
        const bool reload_x = !(x_loaded == x && x_chunk == chunk && x_k == k_in && x_m == m_rows);
        if (reload_x) {
          for (int m = 0; m < m_rows; ++m)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(x + (int64_t)m * k_in + chunk * 512) + lane,
                                             xstage + m * 1024, 16, 0, kAuxDeviceCoherent);
          wait_vm<0>();  // x is the youngest load: everything in flight lands with it
          uint4_t xq[4][4];
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
            for (int s = 0; s < 4; ++s) xq[j4][s] = uint4_t{0u, 0u, 0u, 0u};
          if (r < m_rows) {
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
              for (int s = 0; s < 4; ++s)
                asm volatile("ds_read_b128 %0, %1 offset:%2"
                             : "=v"(xq[j4][s])
                             : "v"(x_rd + r * 1024 + kc * 64), "n"((j4 * 16 + s) * 16));
          }
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              asm volatile("" : "+v"(xq[j4][s]));  // consumed after the wait
              xp[j4][s] = permute_x(xq[j4][s]);
            }
          x_loaded = x;
          x_chunk = chunk;
          x_k = k_in;
          x_m = m_rows;
        }
#pragma unroll
        for (int j = 0; j < kPassRows; ++j) {
          if (j >= nj) break;
          // ---- this item's loads are older than those of the n_ahead - 1 items issued after it
          if (!reload_x || j > 0) {
            if (n_ahead >= 4) wait_vm<3 * kItemOps>();
            else if (n_ahead == 3) wait_vm<2 * kItemOps>();
            else if (n_ahead == 2) wait_vm<kItemOps>();
            else wait_vm<0>();
          }
          const uint32_t src = ring_rd + slot * kItemBytes;
          uint4_t wq[4], sv, bv;
#pragma unroll
          for (int s = 0; s < 4; ++s) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(wq[s]) : "v"(src + lane * 16), "n"(s * 1024));
          asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(sv) : "v"(src + r * 16));
          asm volatile("ds_read_b128 %0, %1 offset:4352" : "=v"(bv) : "v"(src + r * 16));
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wq[0]), "+v"(wq[1]), "+v"(wq[2]), "+v"(wq[3]), "+v"(sv), "+v"(bv));
          // ---- the slot is free: fetch the item NS ahead into it
          --n_ahead;
          if (prod.d < n_entries) {
            issue_item(prod, slot);
            ++n_ahead;
            next_item(prod);
          }
          slot = slot + 1 == NS ? 0 : slot + 1;
          // ---- expand and multiply
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4) {
            const half2_t s2 = as_half2(__builtin_amdgcn_perm(sv[j4], sv[j4], half_sel));
            const half2_t b2 = as_half2(__builtin_amdgcn_perm(bv[j4], bv[j4], half_sel));
#pragma unroll
            for (int s = 0; s < 4; ++s)
              acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(dequant_word(wq[j4][s], s2, b2), xp[j4][s], acc[j], 0, 0, 0);
          }
        }
      }
      // ---- drop the partial sums into this wave's mailbox once the reducer has emptied it
      while (lds_load(&ctl->consumed) < q) __builtin_amdgcn_s_sleep(1);
      if (r < MCAP) {
#pragma unroll
        for (int j = 0; j < kPassRows; ++j)
          if (j < nj) *reinterpret_cast<float4_t *>(mail + wave * kMailBytes + ((j * 4 + kc) * MCAP + r) * 16) = acc[j];
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the deposit is in LDS before it is counted
      if (lane == 0) __hip_atomic_fetch_add(&ctl->deposited, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  wait_vm<0>();
}

}  // namespace

// (external linkage: the host takes its address for hipFuncSetAttribute)
template <int MCAP, int NS>
__global__ __launch_bounds__(kThreadsAll) void gemv_stream_kernel(const void *entries, int n_entries, int *status) {
  gemv_stream_body<MCAP, NS>(reinterpret_cast<const Entry *>(entries), n_entries, status);
}

int launch_gemv_sequence(const gq_gemv_desc *host, const gq_gemv_desc *device, int64_t count, int *status,
                         hipStream_t stream) {
  int max_m = 1;
  bool supported = count <= (1 << 20);
  for (int64_t i = 0; i < count && supported; ++i) {
    const gq_gemv_desc &d = host[i];
    if (d.m_rows > max_m) max_m = d.m_rows;
    supported = d.group_size == 64 && d.k_in % 512 == 0 && d.k_in > 0 && d.m_rows >= 1 && d.m_rows <= 4 &&
                d.n_out >= 1 && ((uintptr_t)d.x % 16) == 0 && ((uintptr_t)d.packed % 16) == 0 &&
                ((uintptr_t)d.scale % 16) == 0 && ((uintptr_t)d.bias % 16) == 0;
  }
  if (!supported || option_gemv_variant() == 3) {
    // any other shape: one launch per entry; stream order provides every dependency
    for (int64_t i = 0; i < count; ++i) {
      const gq_gemv_desc &d = host[i];
      const int rc = launch_gemv(d.x, d.m_rows, d.packed, d.scale, d.bias, d.out_bias, d.y, d.n_out, d.k_in,
                                 d.group_size, stream);
      if (rc != GQ_OK) return rc;
    }
    return GQ_OK;
  }
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "hipGetDevice: %s", hipGetErrorString(e));
  static int cu_count[64] = {0};
  if (dev < 0 || dev >= 64) return fail(GQ_ERR_UNSUPPORTED, "device index %d", dev);
  if (cu_count[dev] == 0) {
    int n = 0;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || n <= 0) return fail((int)e, "cannot query the compute unit count");
    cu_count[dev] = n;
  }
  const int grid = cu_count[dev] < kMaxGroups ? cu_count[dev] : kMaxGroups;  // one workgroup per compute unit, all resident together
#define GQ_STREAM(MCAP, NS)                                                                                   \
  do {                                                                                                        \
    constexpr int lds_bytes =                                                                                 \
        kWaves * (NS * kItemBytes + MCAP * 1024) + kMaxEntries * 64 + kWaves * kPassRows * 4 * MCAP * 16 + 64;  \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                    \
    auto kern = gemv_stream_kernel<MCAP, NS>;                                                                 \
    static bool configured = false;                                                                           \
    if (!configured) {                                                                                        \
      e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                              lds_bytes);                                                                     \
      if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));              \
      configured = true;                                                                                      \
    }                                                                                                         \
    for (int64_t first = 0; first < count; first += kMaxEntries) {                                            \
      const int n = (int)(count - first < kMaxEntries ? count - first : kMaxEntries);                         \
      kern<<<dim3(grid), dim3(kThreadsAll), lds_bytes, stream>>>(device + first, n, status);                     \
    }                                                                                                         \
  } while (0)
  GQ_STREAM(4, 3);
#undef GQ_STREAM
  return check_launch("gemv_stream_kernel");
}

}  // namespace gq
