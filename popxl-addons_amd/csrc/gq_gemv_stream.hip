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

constexpr int kWaves = 8, kThreads = kWaves * 64;
constexpr int kItemBytes = 4096 + 512;  // packed words, 16 rows x 16 B of scale, 16 rows x 16 B of bias
constexpr int kItemOps = 5;             // direct-to-LDS loads per item: 4 packed + 1 scale/bias
constexpr int kPassRows = 4;            // row blocks per pass (accumulators held by a wave)
constexpr unsigned kSpinLimit = 1u << 18;

// progress of the running sequence on this device; the last workgroup to leave resets them
__device__ unsigned int g_arrived;  // (workgroup, entry) completions
__device__ unsigned int g_exited;   // workgroups that left the kernel

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

// MCAP: largest batch the x stage of a wave holds (KiB); NS: depth of the weight ring.
// (A __device__ function: a __global__ template is also instantiated for the host, where the
// target builtins and inline assembly do not exist.)
template <int MCAP, int NS>
__device__ __forceinline__ void gemv_stream_body(const Entry *__restrict__ entries, int n_entries,
                                                 int *__restrict__ status) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int kWaveBytes = NS * kItemBytes + MCAP * 1024;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kc = lane >> 4;
  const int G = gridDim.x, b = blockIdx.x;
  char *ring = lds + wave * kWaveBytes;
  char *xstage = ring + NS * kItemBytes;
  const uint32_t ring_rd = (uint32_t)(uintptr_t)ring, x_rd = (uint32_t)(uintptr_t)xstage;
  const uint32_t half_sel = (kc & 2) ? 0x07060706u : 0x05040504u;  // lane's group within a slot: kc / 2

  // number of row blocks this workgroup owns in entry e
  auto my_row_blocks = [&](const Entry &e) {
    const int rb = (e.n_out + 15) >> 4;
    return rb > b ? (rb - b + G - 1) / G : 0;
  };
  // does cursor c name a work item of this wave?  (entries without rows for this workgroup and
  // chunks past k_in are skipped)
  auto valid = [&](const Cursor &c) {
    if (c.d >= n_entries) return true;  // the end is a valid resting place
    const Entry &e = entries[c.d];
    const int nrb = my_row_blocks(e);
    return c.pass * kPassRows + c.j < nrb && (c.phase * kWaves + wave) * 512 < e.k_in;
  };
  auto step = [&](Cursor &c) {
    const Entry &e = entries[c.d];
    const int nrb = my_row_blocks(e);
    const int phases = (e.k_in + 4095) >> 12;
    if (++c.j < kPassRows && c.pass * kPassRows + c.j < nrb) return;
    c.j = 0;
    if (++c.phase < phases) return;
    c.phase = 0;
    if (++c.pass * kPassRows < nrb) return;
    c.pass = 0;
    ++c.d;
  };
  auto next_item = [&](Cursor &c) {
    do step(c);
    while (c.d < n_entries && !valid(c));
  };
  // direct-to-LDS loads of the item at cursor c into ring slot `slot`
  auto issue_item = [&](const Cursor &c, int slot) {
    const Entry &e = entries[c.d];
    const int rb = b + (c.pass * kPassRows + c.j) * G;
    const int row = min(rb * 16 + r, e.n_out - 1);
    const int chunk = c.phase * kWaves + wave;
    char *dst = ring + slot * kItemBytes;
    const uint4_t *src = e.packed + (int64_t)row * (e.k_in >> 5) + chunk * 16 + kc;
#pragma unroll
    for (int s = 0; s < 4; ++s) __builtin_amdgcn_global_load_lds(src + s * 4, dst + s * 1024, 16, 0, 0);
    // lanes kc == 0 fetch the 8 scales of their row's chunk, lanes kc == 1 the 8 biases
    if (kc < 2) {
      const half_t *sb = (kc == 0 ? e.scale : e.bias) + (int64_t)row * (e.k_in >> 6) + chunk * 8;
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(sb), dst + 4096, 16, 0, 0);
    }
  };

  Cursor prod = {0, 0, 0, 0};  // the producer's position: first item of this wave
  if (n_entries > 0 && !valid(prod)) next_item(prod);
  int n_ahead = 0;  // items issued and not yet consumed
  while (n_ahead < NS && prod.d < n_entries) {
    issue_item(prod, n_ahead);
    ++n_ahead;
    next_item(prod);
  }
  int slot = 0;  // ring slot of the consumer's item
  bool failed = false;

  half8_t xp[4][4];
  const half_t *x_loaded = nullptr;  // x fragments in registers belong to (x_loaded, chunk x_chunk)
  int x_chunk = -1, x_k = 0, x_m = 0;

  for (int d = 0; d < n_entries; ++d) {
    const Entry e = entries[d];
    const int nrb = my_row_blocks(e);
    const int phases = (e.k_in + 4095) >> 12;
    if (e.wait_previous && d > 0) {
      // every workgroup has finished every earlier entry
      if (tid == 0) {
        const unsigned target = (unsigned)d * (unsigned)G;
        unsigned spins = 0;
        while (!failed && __hip_atomic_load(&g_arrived, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
          __builtin_amdgcn_s_sleep(2);
          if (++spins > kSpinLimit) {
            failed = true;
            if (status) atomicExch(status, 1);
          }
        }
        __threadfence();  // acquire: earlier entries' y becomes visible to this compute unit
      }
      __syncthreads();
      x_loaded = nullptr;
    }
    for (int pass = 0; pass * kPassRows < nrb; ++pass) {
      const int nj = min(kPassRows, nrb - pass * kPassRows);
      float4_t acc[kPassRows];
#pragma unroll
      for (int j = 0; j < kPassRows; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
      for (int phase = 0; phase < phases; ++phase) {
        const int chunk = phase * kWaves + wave;
        if (chunk * 512 >= e.k_in) continue;
        // ---- x fragments of this chunk (kept when the previous entry used the same ones)
        const bool reload_x = !(x_loaded == e.x && x_chunk == chunk && x_k == e.k_in && x_m == e.m_rows);
        if (reload_x) {
          for (int m = 0; m < e.m_rows; ++m)
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4_t *>(e.x + (int64_t)m * e.k_in + chunk * 512) + lane,
                                             xstage + m * 1024, 16, 0, 0);
          wait_vm<0>();  // x is the youngest load: everything in flight lands with it
          uint4_t q[4][4];
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
            for (int s = 0; s < 4; ++s) q[j4][s] = uint4_t{0u, 0u, 0u, 0u};
          if (r < e.m_rows) {
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
              for (int s = 0; s < 4; ++s)
                asm volatile("ds_read_b128 %0, %1 offset:%2"
                             : "=v"(q[j4][s])
                             : "v"(x_rd + r * 1024 + kc * 64), "n"((j4 * 16 + s) * 16));
          }
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              asm volatile("" : "+v"(q[j4][s]));  // consumed after the wait
              xp[j4][s] = permute_x(q[j4][s]);
            }
          x_loaded = e.x;
          x_chunk = chunk;
          x_k = e.k_in;
          x_m = e.m_rows;
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
      // ---- partial sums of the 8 waves meet in LDS.  Each wave's x stage doubles as its mailbox:
      //      the fragments it held are in registers by now.
#pragma unroll
      for (int j = 0; j < kPassRows; ++j)
        if (j < nj) *reinterpret_cast<float4_t *>(xstage + j * 1024 + lane * 16) = acc[j];
      __syncthreads();
      for (int t = tid; t < nj * 64; t += kThreads) {
        const int j = t >> 6, l = t & 63;
        float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += *reinterpret_cast<const float4_t *>(lds + w * kWaveBytes + NS * kItemBytes + j * 1024 + l * 16);
        const int m = l & 15;
        if (m < e.m_rows) {
          const int n0 = (b + (pass * kPassRows + j) * G) * 16 + 4 * (l >> 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int n = n0 + i;
            if (n < e.n_out) {
              float v = sum[i];
              if (e.out_bias) v += (float)e.out_bias[n];
              e.y[(int64_t)m * e.n_out + n] = (half_t)v;
            }
          }
        }
      }
      __syncthreads();
    }
    // ---- this workgroup is done with entry d
    if (tid == 0) {
      __threadfence();  // release: y is visible device-wide before the count
      atomicAdd(&g_arrived, 1u);
    }
  }
  wait_vm<0>();
  if (tid == 0) {
    if (atomicAdd(&g_exited, 1u) == (unsigned)G - 1) {  // last one out resets the counters
      __hip_atomic_store(&g_arrived, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&g_exited, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace

// (external linkage: the host takes its address for hipFuncSetAttribute)
template <int MCAP, int NS>
__global__ __launch_bounds__(kThreads) void gemv_stream_kernel(const void *entries, int n_entries, int *status) {
  gemv_stream_body<MCAP, NS>(reinterpret_cast<const Entry *>(entries), n_entries, status);
}

int launch_gemv_sequence(const gq_gemv_desc *host, const gq_gemv_desc *device, int64_t count, int *status,
                         hipStream_t stream) {
  int max_m = 1;
  bool supported = count <= (1 << 20);
  for (int64_t i = 0; i < count && supported; ++i) {
    const gq_gemv_desc &d = host[i];
    if (d.m_rows > max_m) max_m = d.m_rows;
    supported = d.group_size == 64 && d.k_in % 512 == 0 && d.k_in > 0 && d.m_rows >= 1 && d.m_rows <= 8 &&
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
  const int grid = cu_count[dev];  // one workgroup per compute unit: all of them are resident together
  const void *entries = device;
#define GQ_STREAM(MCAP, NS)                                                                                   \
  do {                                                                                                        \
    constexpr int lds_bytes = kWaves * (NS * kItemBytes + MCAP * 1024);                                       \
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");                                                    \
    auto kern = gemv_stream_kernel<MCAP, NS>;                                                                 \
    static bool configured = false;                                                                           \
    if (!configured) {                                                                                        \
      e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                              lds_bytes);                                                                     \
      if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));              \
      configured = true;                                                                                      \
    }                                                                                                         \
    kern<<<dim3(grid), dim3(kThreads), lds_bytes, stream>>>(entries, (int)count, status);                     \
  } while (0)
  if (max_m <= 4) GQ_STREAM(4, 3);
  else GQ_STREAM(8, 2);
#undef GQ_STREAM
  return check_launch("gemv_stream_kernel");
}

}  // namespace gq
