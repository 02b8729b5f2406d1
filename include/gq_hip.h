/*
 * libgq_hip -- 4-bit group-quantized weight decompression and fused dequant-matmul
 * for AMD MI355X (gfx950).  C ABI: plain pointers and sizes, no C++ or torch types.
 *
 * This library stands where the reference's pybind11 extension
 * `group_quantize_decompress_binding` stands
 * (popxl_addons/ops/group_quantize_decompress/group_quantize_decompress_binding.cpp:39-55):
 * the Python wrappers of the reference call `GroupQuantizeDecompressOp.createOpInGraph`
 * there; here they call the functions below with device pointers.
 *
 * Conventions
 *   - Every data pointer is a DEVICE pointer owned by the caller.  binary16 values are
 *     passed as their 16-bit patterns (`uint16_t`).
 *   - Work is enqueued on `stream` (a `hipStream_t` passed as `void*`; NULL = the null
 *     stream) and the call returns without synchronising.
 *   - Return value: 0 on success; a negative GQ_ERR_* code when an argument is rejected
 *     (nothing was launched); a positive value is a `hipError_t` from the runtime.
 *     `gq_last_error()` returns a thread-local, human-readable description of the last
 *     non-zero return on the calling thread.
 *   - Functions allocate nothing and there are no process-wide options.  What the library keeps
 *     between calls, per device: (1) the block of progress words and exchange buffers of
 *     gq_gemv_sequence_f16, (2) the scratch array of gq_linear_kn_act_noalloc_f16, (3) for kernels
 *     that need more than 64 KiB of LDS, the fact that hipFuncSetAttribute has been called for them
 *     (set on first use, never changed).  (1) and (2) are shared by every call on the device: such
 *     calls must be enqueued on ONE stream per device; a call that arrives on another stream while
 *     the previous one's stream still has work pending returns GQ_ERR_UNSUPPORTED and launches
 *     nothing (streams under capture are not checked: ordering graph replays is the caller's job).
 *     Their siblings that take a workspace (gq_gemv_sequence_ws_f16, gq_linear_kn_act_f16) keep
 *     nothing.  All other functions are re-entrant.  Every entry point can be captured in a HIP graph.
 *
 * Packed layout (group_quantize_decompress.py:127-135, group_quantize_decompress_codelet.cpp:11-14)
 *   packed[r][g][i] is a little-endian uint16 holding four 4-bit codes, most significant
 *   nibble first: element 4*i+j of group g of row r is (packed[r][g][i] >> (12 - 4*j)) & 15.
 *   value = f16( f16(code * scale[r][g]) + bias[r][g] )   -- two roundings, never an fma.
 */
#ifndef GQ_HIP_H
#define GQ_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GQ_ABI_VERSION 4

#define GQ_OK 0
#define GQ_ERR_NULL_POINTER (-1) /* a required pointer is NULL */
#define GQ_ERR_BAD_SHAPE (-2)    /* a size is negative, or sizes are inconsistent */
#define GQ_ERR_MISALIGNED (-3)   /* a pointer is not aligned to its element size */
#define GQ_ERR_UNSUPPORTED (-4)  /* well-formed, but outside what the kernels cover */
#define GQ_ERR_NO_DEVICE (-5)    /* no usable gfx950 device / code object */

/* Epilogues of the fused matmul entry points: applied to sum + out_bias in binary32 before the
 * result is rounded to binary16. */
#define GQ_ACT_NONE 0
#define GQ_ACT_RELU 1
#define GQ_ACT_GELU_TANH 2 /* 0.5 v (1 + tanh(sqrt(2/pi) (v + 0.044715 v^3))) */

/* ABI version of the loaded library (GQ_ABI_VERSION it was built with). */
int gq_abi_version(void);

/* Thread-local description of the last failing call on this thread ("" if none). */
const char *gq_last_error(void);

/*
 * Standalone decompress.  Replaces the device op created by
 * group_quantize_decompress() (group_quantize_decompress.py:78-86), whose lowering is
 * GroupQuantizeDecompressOpx::grow (group_quantize_decompressx.cpp:121-135: unpack vertex,
 * then scale and bias as a second pass) with shape rules of
 * GroupQuantizeDecompressOp::setup (group_quantize_decompress.cpp:35-77).
 *
 *   packed [rows, n_groups, n_ids] uint16      scale, bias [rows, n_groups] binary16
 *   out    [rows, n_groups * n_ids * 4] binary16, row-major, bit-exact to
 *          group_quantize_decompress_numpy (group_quantize_decompress.py:95-141).
 * Zero-sized problems succeed without a launch.
 */
int gq_decompress_f16(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                      uint16_t *out, int64_t rows, int64_t n_groups, int64_t n_ids, void *stream);

/*
 * Same values written transposed: out_t [n_groups * n_ids * 4, rows].  This is the
 * `dim=0` result of group_quantize_decompress (group_quantize_decompress.py:87-91 moves
 * the decompressed axis to `dim`), materialised instead of returned as a strided view.
 */
int gq_decompress_f16_transposed(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                                 uint16_t *out_t, int64_t rows, int64_t n_groups, int64_t n_ids,
                                 void *stream);

/*
 * Fused decompress + matmul, groups along the input (K) axis: the computation of
 * LinearGQ.build with dim=0 (popxl_addons/layers/linear_gq.py:99-109):
 *   w = decompress(packed, scale, bias)      [n_out, k_in]
 *   y[m][n] = sum_k x[m][k] * w[n][k] (+ out_bias[n])
 * without writing w to memory.
 *
 *   x        [m_rows, k_in] binary16             y [m_rows, n_out] binary16
 *   packed   [n_out, k_in / group_size, group_size / 4] uint16
 *   scale, bias [n_out, k_in / group_size] binary16
 *   out_bias [n_out] binary16 or NULL
 * Accumulation is binary32; the result is within 1e-2 (max-abs normalised) of a binary32
 * matmul over the bit-exact decompressed weight.
 *
 * gq_gemv_f16  decode-sized batches, 1 <= m_rows <= 16.
 * gq_gemm_f16  prefill-sized batches (any m_rows >= 1; built for m_rows >= 16).
 * gq_linear_f16 picks between them by m_rows (and, for 17 to 128 rows on large weights, runs
 *              several GEMV launches of 16 rows each where those are faster than the GEMM's
 *              mostly empty tiles); it is what the LinearGQ wrapper calls.
 *
 * Requirements: group_size % 4 == 0, k_in % group_size == 0.  Fast kernels need a power-of-two
 * group_size >= 32, k_in % 128 == 0 (GEMV) or % 64 == 0 (GEMM) and 16-byte aligned x / packed;
 * other shapes run slower generic kernels with the same results.
 */
int gq_gemv_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                int64_t k_in, int64_t group_size, void *stream);

int gq_gemm_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                int64_t k_in, int64_t group_size, void *stream);

int gq_linear_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                  const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                  int64_t k_in, int64_t group_size, void *stream);

/*
 * gq_linear_f16 with an activation fused into the epilogue: y = act(x w^T + out_bias), the step
 * that follows the up-projection of a decoder's feed-forward block.  No counterpart in the
 * reference (LinearGQ.build ends at the bias add, popxl_addons/layers/linear_gq.py:102-109, and
 * the activation is a separate op of the model); `activation` is one of GQ_ACT_*.
 */
int gq_linear_act_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                      const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                      int64_t k_in, int64_t group_size, int32_t activation, void *stream);

/*
 * gq_linear_act_f16 with an optional workspace (no counterpart in the reference: LinearGQ.build has
 * nothing to tune, popxl_addons/layers/linear_gq.py:99-109).  A weight with few outputs gives the
 * GEMM kernel few output tiles (4096 outputs at 128 rows: 64 of 128 x 64 for 256 compute units);
 * with the workspace, 2 to 16 workgroups divide the input features of a tile and add their binary32
 * accumulators through it, in a fixed order.  gq_gemm_workspace_bytes() is the size for a problem
 * (0: no division would pay, or m_rows <= 16); device memory, 16-byte aligned; its first 16 KiB hold
 * arrival counters that the caller zeroes once and every call leaves zero, so one workspace serves
 * calls of any shape -- one at a time: calls that share a workspace must not overlap.  A workspace
 * that is NULL, misaligned or too small is not used: the call then is gq_linear_act_f16.
 */
int64_t gq_gemm_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size);
int gq_linear_act_ws_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                         const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                         int64_t k_in, int64_t group_size, int32_t activation, void *workspace,
                         int64_t workspace_bytes, void *stream);

/*
 * gq_linear_act_ws_f16 for a caller that also holds the weight's derived copy in the streaming layout
 * (`blob`, made by gq_gemv_prepack_f16 below from the same packed, scale and bias: group_size 64,
 * k_in % 512 == 0, 16-byte aligned).  No counterpart in the reference (LinearGQ.build reads the three
 * variables, popxl_addons/layers/linear_gq.py:99-109).  Batches of more than 16 rows that run the
 * pipelined GEMM kernel then read the copy, whose pieces are 512 bytes contiguous where a row of
 * `packed` contributes 32 bytes per step of 64 input features: the same results to the tolerance of
 * the fused paths, 5 - 12 % sooner; batches of up to 16 rows and passes of the GEMV kernel read it
 * too (each load 1 KiB contiguous and read once).  Only a call whose x is not 16-byte aligned reads
 * packed, scale and bias (the kernels of gq_linear_act_ws_f16 for such an x): a caller whose x is
 * aligned may keep the copy alone and pass all three as NULL (one of them NULL and another not is
 * GQ_ERR_NULL_POINTER; all three NULL with a misaligned x is GQ_ERR_MISALIGNED).  blob == NULL: the
 * call is gq_linear_act_ws_f16.
 */
int gq_linear_p_act_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                        const uint16_t *bias, const void *blob, const uint16_t *out_bias, uint16_t *y,
                        int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation, void *workspace,
                        int64_t workspace_bytes, void *stream);

/*
 * gq_linear_p_act_f16 at decode batches (m_rows <= 16) for an x whose rows are `x_row_stride` elements
 * apart (>= k_in): a column slice of a wider matrix -- e.g. the part of the output of fused projections
 * (LinearGQ.fuse) that the next layer consumes -- without a copy that gathers it.  No counterpart in the
 * reference (a popxl slice is a view of the static graph, popxl_addons/layers/linear_gq.py:99-109 sees a
 * tensor).  The same kernels and results as the call on a gathered x; x_row_stride == k_in is that call.
 * The fast kernels need every row of x 16-byte aligned (x and x_row_stride % 8 == 0; with packed, scale and
 * bias NULL anything else is GQ_ERR_MISALIGNED).  m_rows > 16: GQ_ERR_UNSUPPORTED (gather x, or call per 16
 * rows); x_row_stride < k_in: GQ_ERR_BAD_SHAPE.  blob may be NULL (the three variables are read).
 */
int gq_linear_p_strided_f16(const uint16_t *x, int64_t x_row_stride, int64_t m_rows, const uint16_t *packed,
                            const uint16_t *scale, const uint16_t *bias, const void *blob, const uint16_t *out_bias,
                            uint16_t *y, int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation,
                            void *stream);

/*
 * Fused decompress + matmul, groups along the OUTPUT features: the computation of LinearGQ.build
 * with dim = -1 or 1, the constructor default (popxl_addons/layers/linear_gq.py:26, 59-62, 99-109):
 *   w = decompress(packed, scale, bias)      [k_in, n_out]
 *   y[m][n] = act( sum_k x[m][k] * w[k][n] (+ out_bias[n]) )
 * without writing w to memory.
 *
 *   x        [m_rows, k_in] binary16             y [m_rows, n_out] binary16
 *   packed   [k_in, n_out / group_size, group_size / 4] uint16
 *   scale, bias [k_in, n_out / group_size] binary16
 *   out_bias [n_out] binary16 or NULL;  activation: GQ_ACT_*
 * Same accumulation and tolerance as gq_linear_act_f16.  Requirements: group_size % 4 == 0,
 * n_out % group_size == 0; the fast kernels need a power-of-two group_size >= 32, n_out % 32 == 0
 * and a 16-byte aligned packed (plus k_in % 64 == 0 and a 16-byte aligned x for m_rows > 16); other
 * shapes run a slower generic kernel with the same results.
 *
 * For m_rows <= 16 the contraction is split between workgroups, whose binary32 partial sums meet
 * in `workspace`: device memory, 16-byte aligned, at least gq_linear_kn_workspace_bytes() bytes
 * for the same sizes (0: none needed, workspace may be NULL).  Its first 16 KiB hold arrival
 * counters: the caller zeroes them once, every call leaves them zero, so one workspace serves
 * calls of any shape -- one at a time: calls that share a workspace must not overlap.
 * For m_rows > 16 the workspace is an option.  gq_linear_kn_workspace_bytes() is non-zero where the
 * 128 x 128 output tiles are too few for the device (a weight with 4096 outputs has 32 per 128 rows):
 * with the workspace the prefill kernel divides the input features over several workgroups per tile,
 * whose binary32 partial sums meet there (or, for 17 to 128 rows, the batch runs as passes of the
 * decode kernel over 16 rows each where those are expected to be faster); without it, or with one
 * that is too small, the prefill kernel runs undivided and gives the same result to the tolerance
 * of the fused paths.
 */
int64_t gq_linear_kn_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size);
int gq_linear_kn_act_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                         const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                         int64_t k_in, int64_t group_size, int32_t activation, void *workspace,
                         int64_t workspace_bytes, void *stream);

/*
 * gq_linear_kn_act_f16 for callers that cannot allocate device memory or pass a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The partial sums and arrival counters live in a device array
 * inside the library (one copy per GPU, 16 KiB + GQ_LINEAR_KN_NOALLOC_PARTIAL_BYTES, held until the
 * process ends); the call allocates and frees nothing.  Same arguments, results bit for bit those
 * of gq_linear_kn_act_f16.  A problem of up to 16 rows whose gq_linear_kn_workspace_bytes() exceeds
 * that size is rejected with GQ_ERR_UNSUPPORTED (every problem of up to 8 rows fits; of the 6B layer
 * shapes, 4096 and 16384 outputs fit up to 16 rows, the fused 12288-wide projection up to 8).  Above
 * 16 rows nothing is rejected: where the 16-row passes that gq_linear_kn_act_f16 would run do not
 * fit, the prefill kernel, which needs no scratch, runs (the same result to the tolerance of the
 * fused paths, not bit for bit).
 * All calls on one GPU share the array: calls that overlap on one GPU (different streams) race.
 * Enqueue them on one stream per GPU: a call on another stream while the previous call's stream
 * still has work pending returns GQ_ERR_UNSUPPORTED (nothing launched); calls under stream capture
 * are not checked.
 */
#define GQ_LINEAR_KN_NOALLOC_PARTIAL_BYTES (4 << 20)
int gq_linear_kn_act_noalloc_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                                 const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                                 int64_t k_in, int64_t group_size, int32_t activation, void *stream);

/*
 * A sequence of decode GEMVs (a layer stack) as one call.  No counterpart in the reference, where
 * a model is a chain of LinearGQ.build calls (popxl_addons/layers/linear_gq.py:99-109) compiled
 * into one static device program; this entry point is the analogue for a chain of gq_gemv_f16
 * calls: entry i computes what gq_gemv_f16 would, to the tolerance of the fused paths (the
 * summation order differs).  Dependencies between entries are
 * declared, not implied: entry i starts only after the first wait_entries[i] entries of the
 * sequence have completed (0 <= wait_entries <= i; 0 = no dependency, i = every earlier entry).
 * Set it past the entry that produces x or out_bias of entry i.  Entries may otherwise overlap
 * and complete in any order: an entry that overwrites memory which an earlier entry reads or
 * writes must wait for that entry as well.  The x of an entry may be (part of) the y of one earlier
 * entry or, at one batch row, of several earlier entries whose y lie end to end in memory (two
 * projections whose results are added, as one entry over the concatenation of their inputs).
 *
 * Runs of consecutive entries with group_size 64, k_in % 512 == 0, m_rows <= 4 and 16-byte aligned
 * pointers execute as one persistent kernel per run of up to 128 entries (one workgroup per compute
 * unit) that streams the packed weights without a gap between entries; every other entry is a launch
 * of its own, in stream order.  There are two such kernels: launches of one batch row whose weights are
 * all in the streaming layout (below) and whose entries need nothing but the results they read as x run
 * on the faster of the two; every other launch runs on the general one.  The choice is made per launch and
 * changes no result beyond the tolerance of the fused paths.
 *
 *   descs         host copy of the entries (validated here, not read after the call returns)
 *   descs_device  device copy of the same `count` entries (read by the kernel)
 *   status        device int32 or NULL; set to 1 if the kernel gave up waiting for earlier entries
 *                 (it then still terminates; results are invalid).  The caller zeroes it.
 *
 * The persistent kernel launches one workgroup per compute unit and relies on all of them being
 * resident together: nothing else should occupy the compute units while it runs.  Every wait is
 * bounded: a poller that sees no progress `spin_limit` polls in a row gives up, sets *status and
 * lets the kernel drain (results are then invalid, the progress words are back at zero).
 *
 * gq_gemv_sequence_f16     keeps the per-workgroup progress words in a block that the library
 *                          holds per device: at most ONE sequence may run on a device at a time.
 *                          Calls are ordered by their stream; a call on a different stream while the
 *                          stream of the previous call still has work pending is refused with
 *                          GQ_ERR_UNSUPPORTED (nothing launched) rather than left to corrupt both.
 * gq_gemv_sequence_ws_f16  takes them from `workspace` (device memory, 256-byte aligned,
 *                          gq_gemv_sequence_workspace_bytes() bytes -- progress words and the
 *                          buffers through which results travel from entry to entry inside a
 *                          launch -- zeroed by the caller once, before its first use; after that
 *                          the calls that use it keep it in the state the next one expects), so
 *                          that the library holds no state for the call: sequences with
 *                          workspaces of their own may be enqueued on
 *                          different streams and captured in different graphs, as long as the
 *                          caller orders them (events) so that two persistent kernels never run at
 *                          the same time -- each needs every compute unit.  spin_limit <= 0 selects
 *                          the default (2^18 polls).
 */
typedef struct gq_gemv_desc {
  const uint16_t *x;        /* [m_rows, k_in] binary16 */
  const uint16_t *packed;   /* [n_out, k_in / group_size, group_size / 4]; or, with scale == bias == NULL,
                               the weight in the streaming layout written by gq_gemv_prepack_f16 */
  const uint16_t *scale;    /* [n_out, k_in / group_size] binary16 */
  const uint16_t *bias;     /* [n_out, k_in / group_size] binary16 */
  const uint16_t *out_bias; /* [n_out] binary16 or NULL */
  uint16_t *y;              /* [m_rows, n_out] binary16 */
  int32_t m_rows, n_out, k_in, group_size;
  int32_t wait_entries;     /* entries [0, wait_entries) complete before this one starts */
  int32_t activation;       /* GQ_ACT_*: epilogue of this entry; or-ed with GQ_DESC_KN_LAYOUT for a weight
                               grouped along the OUTPUT features (below) */
} gq_gemv_desc;

/*
 * An entry whose weight is grouped along the output features (LinearGQ with dim = -1 / 1, the
 * constructor default, popxl_addons/layers/linear_gq.py:26, 59-62): `packed` is the blob written by
 * gq_gemv_kn_prepack_f16 (below), scale == bias == NULL, group_size 64, n_out % 64 == 0,
 * k_in % 512 == 0, m_rows <= 16, x and blob 16-byte aligned, y 8-byte.  The entry computes what
 * gq_linear_knp_act_f16 computes.  Such entries run as a launch of their own inside the sequence
 * (stream order provides whatever they wait for), next to runs of entries that the persistent
 * kernels cover.
 */
#define GQ_DESC_KN_LAYOUT 0x100

/*
 * Streaming layout of one weight for gq_gemv_sequence_f16.  No counterpart in the reference, whose
 * three variables (popxl_addons/layers/linear_gq.py:74-97) stay what the rest of the API takes;
 * this is a derived copy made once when the weights are loaded.  The persistent kernel fetches a
 * weight in pieces of 16 rows x 512 input features: 4 KiB of packed words in sixteen 256-byte
 * stretches one row apart, plus sixteen 16-byte pieces each of scale and bias.  The streaming
 * layout stores every such piece as one contiguous 4608-byte block in the order the kernel keeps
 * it in LDS (rows past n_out zero-filled), so that all of its loads are contiguous; the bytes per
 * weight stay 0.5625.  Needs group_size 64 and k_in % 512 == 0.
 *
 *   gq_gemv_prepacked_bytes  size of the blob in bytes, or a negative GQ_ERR_* code
 *   gq_gemv_prepack_f16      writes the blob (device memory, 16-byte aligned) from packed / scale /
 *                            bias (16-byte aligned) on `stream`
 * An entry of a sequence uses the blob by passing it as `packed` with scale == bias == NULL (up to
 * 16 rows; like any entry it joins a run of the persistent kernels up to 4 rows and is a launch of
 * its own above).  gq_linear_p_act_f16 takes the blob beside the three variables.
 */
int64_t gq_gemv_prepacked_bytes(int64_t n_out, int64_t k_in, int64_t group_size);
int gq_gemv_prepack_f16(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob,
                        int64_t n_out, int64_t k_in, int64_t group_size, void *stream);

int gq_gemv_sequence_f16(const gq_gemv_desc *descs, const gq_gemv_desc *descs_device, int64_t count,
                         int32_t *status, void *stream);
int64_t gq_gemv_sequence_workspace_bytes(void);
int gq_gemv_sequence_ws_f16(const gq_gemv_desc *descs, const gq_gemv_desc *descs_device, int64_t count,
                            int32_t *status, void *workspace, int64_t workspace_bytes, int64_t spin_limit,
                            void *stream);

/*
 * The default layout of LinearGQ (groups along the OUTPUT features, dim = -1 / 1:
 * popxl_addons/layers/linear_gq.py:26, 59-62, 99-101) for decode batches, on a derived copy of the
 * weight.  No counterpart in the reference, whose three variables stay what the rest of the API
 * takes; this copy is made once when the weights are loaded, like the streaming layout above.
 *
 * In the variables a packed word holds 8 consecutive outputs of ONE input feature; a GEMV wants the
 * codes of an output contiguous along the input features.  With
 *   y[m][n] = sum_k (x[m][k] scale[k][g]) code[k][n] + sum_k x[m][k] bias[k][g],   g = n / 64,
 * the scale moves to the activations, so the copy only has to transpose the codes: the KN STREAMING
 * LAYOUT holds, per group of 64 outputs and chunk of 512 input features, 16 KiB of codes (contiguous
 * along the input features, in the order the kernel hands them to the matrix instruction) followed by
 * the group's 512 scales and 512 biases of that chunk: 18432 bytes, the same 0.5625 bytes per weight.
 * Needs group_size 64, n_out % 64 == 0, k_in % 512 == 0.
 *
 *   gq_gemv_kn_prepacked_bytes  size of the blob in bytes, or a negative GQ_ERR_* code
 *   gq_gemv_kn_prepack_f16      writes the blob (device memory, 16-byte aligned) from the variables
 *                               packed [k_in, n_out / 64, 16], scale / bias [k_in, n_out / 64] on `stream`
 *   gq_linear_knp_act_f16       y = act(x w + out_bias) as gq_linear_kn_act_f16 computes it, from the
 *                               blob, for any m_rows >= 1 (x, blob 16-byte aligned, y 8-byte); needs no
 *                               workspace and keeps no state.  Up to 16 rows (and 17 to 32 as two passes)
 *                               run the decode kernel: the products x scale are rounded to binary16
 *                               before they are multiplied with the exact codes.  More rows run the
 *                               pipelined MFMA kernel of gq_gemm_f16 with the blob as its weight source
 *                               (every input feature brings its own scale and bias to the expansion).
 *                               Either way the result is within the tolerance of the fused paths.
 *   gq_linear_knp_strided_f16   gq_linear_knp_act_f16 at decode batches (m_rows <= 16) for an x whose rows are
 *                               `x_row_stride` elements apart (>= k_in, a multiple of 8: every row 16-byte
 *                               aligned): a column slice of a wider matrix, read where it lies (see
 *                               gq_linear_p_strided_f16).  The same kernel and results as on a gathered x.
 *                               m_rows > 16: GQ_ERR_UNSUPPORTED; x_row_stride < k_in: GQ_ERR_BAD_SHAPE.
 */
int64_t gq_gemv_kn_prepacked_bytes(int64_t n_out, int64_t k_in, int64_t group_size);
int gq_gemv_kn_prepack_f16(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob,
                           int64_t n_out, int64_t k_in, int64_t group_size, void *stream);
int gq_linear_knp_act_f16(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias,
                          uint16_t *y, int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation,
                          void *stream);
int gq_linear_knp_strided_f16(const uint16_t *x, int64_t x_row_stride, int64_t m_rows, const void *blob,
                              const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in, int64_t group_size,
                              int32_t activation, void *stream);

/*
 * Device-side compress for binary16 input: bit-identical packed/scale/bias to
 * group_quantize_compress_numpy on a float16 array (group_quantize_decompress.py:178-196)
 * wherever that function is defined (every group has max > min; all values finite).
 * A constant group yields scale 0, codes 0, bias = the constant.
 *
 *   t [rows, n_groups * group_size] binary16  ->  packed [rows, n_groups, group_size/4],
 *   scale, bias [rows, n_groups].
 * `nonfinite_flag` (device int32, may be NULL) is set to 1 when any input is Inf/NaN
 * (the reference raises ValueError there, :182-183); outputs are then unspecified.
 */
int gq_compress_f16(const uint16_t *t, uint16_t *packed, uint16_t *scale, uint16_t *bias,
                    int32_t *nonfinite_flag, int64_t rows, int64_t n_groups, int64_t group_size,
                    void *stream);

/*
 * The same for binary32 input, which is what LinearGQ.torch_mapping feeds the packer
 * (popxl_addons/layers/linear_gq.py:130: nn_layer.weight.T, float32): max / min are taken in
 * binary32 and cast to binary16, the scale is binary16 arithmetic, (x - bias) / scale is a binary32
 * subtraction and division (group_quantize_decompress.py:186-192).
 */
int gq_compress_f32(const float *t, uint16_t *packed, uint16_t *scale, uint16_t *bias,
                    int32_t *nonfinite_flag, int64_t rows, int64_t n_groups, int64_t group_size,
                    void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GQ_HIP_H */
