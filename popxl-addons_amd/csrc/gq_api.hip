// C-ABI layer of libgq_hip: argument validation, error text, dispatch to the launchers.
// Shape rules follow GroupQuantizeDecompressOp::setup (group_quantize_decompress.cpp:35-77)
// and LinearGQ.build (popxl_addons/layers/linear_gq.py:58-110).
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "gq_common.h"

namespace gq {

namespace {
thread_local char g_error[512] = "";
}  // namespace

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return GQ_OK;
  return fail((int)e, "%s: %s", what, hipGetErrorString(e));
}

int claim_shared_block(SharedBlockGuard &guard, int dev, hipStream_t stream, const char *who) {
  static std::mutex lock;
  if (dev < 0 || dev >= SharedBlockGuard::kMaxDevices) return fail(GQ_ERR_UNSUPPORTED, "%s: device index %d", who, dev);
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) (void)hipGetLastError();
  if (capture != hipStreamCaptureStatusNone) return GQ_OK;
  std::lock_guard<std::mutex> hold(lock);
  if (guard.used[dev] && guard.last[dev] != stream) {
    // (a stream that no longer exists gives an error code: nothing of it can be pending)
    const hipError_t pending = hipStreamQuery(guard.last[dev]);
    (void)hipGetLastError();  // the query's "not ready" is an answer, not an error of this call
    if (pending == hipErrorNotReady)
      return fail(GQ_ERR_UNSUPPORTED,
                  "%s: the block that the library keeps per device is still in use by work enqueued on another stream; "
                  "calls that share it must be enqueued on one stream (or the other stream's work must have completed) -- "
                  "use the variant that takes a workspace for concurrent streams", who);
  }
  guard.last[dev] = stream;
  guard.used[dev] = true;
  return GQ_OK;
}

namespace {

bool misaligned(const void *p, size_t a) { return ((uintptr_t)p % a) != 0; }

int check_linear_args(const char *who, const uint16_t *x, int64_t m_rows, const uint16_t *packed,
                      const uint16_t *scale, const uint16_t *bias, const uint16_t *out_bias, uint16_t *y,
                      int64_t n_out, int64_t k_in, int64_t group_size) {
  if (m_rows < 0 || n_out < 0 || k_in < 0)
    return fail(GQ_ERR_BAD_SHAPE, "%s: negative size (m_rows=%lld n_out=%lld k_in=%lld)", who,
                (long long)m_rows, (long long)n_out, (long long)k_in);
  if (group_size <= 0 || group_size % 4 != 0)
    return fail(GQ_ERR_BAD_SHAPE, "%s: group_size=%lld must be a positive multiple of 4", who,
                (long long)group_size);
  if (k_in % group_size != 0)
    return fail(GQ_ERR_BAD_SHAPE, "%s: k_in=%lld is not a multiple of group_size=%lld", who, (long long)k_in,
                (long long)group_size);
  if (m_rows == 0 || n_out == 0) return GQ_OK;
  if (!y) return fail(GQ_ERR_NULL_POINTER, "%s: y is NULL", who);
  if (k_in > 0 && (!x || !packed || !scale || !bias))
    return fail(GQ_ERR_NULL_POINTER, "%s: x/packed/scale/bias must not be NULL", who);
  if (misaligned(x, 2) || misaligned(packed, 2) || misaligned(scale, 2) || misaligned(bias, 2) ||
      misaligned(out_bias, 2) || misaligned(y, 2))
    return fail(GQ_ERR_MISALIGNED, "%s: pointers must be 2-byte aligned", who);
  if (m_rows > (int64_t)1 << 30 || n_out > (int64_t)1 << 30 || k_in > (int64_t)1 << 30)
    return fail(GQ_ERR_UNSUPPORTED, "%s: a dimension exceeds 2^30", who);
  return 1;  // proceed
}

int decompress_common(const char *who, const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                      uint16_t *out, int64_t rows, int64_t n_groups, int64_t n_ids, bool transposed,
                      void *stream) {
  if (rows < 0 || n_groups < 0 || n_ids < 0)
    return fail(GQ_ERR_BAD_SHAPE, "%s: negative size (rows=%lld n_groups=%lld n_ids=%lld)", who,
                (long long)rows, (long long)n_groups, (long long)n_ids);
  if (rows == 0 || n_groups == 0 || n_ids == 0) return GQ_OK;
  if (!packed || !scale || !bias || !out) return fail(GQ_ERR_NULL_POINTER, "%s: NULL pointer argument", who);
  if (misaligned(packed, 2) || misaligned(scale, 2) || misaligned(bias, 2) || misaligned(out, 2))
    return fail(GQ_ERR_MISALIGNED, "%s: pointers must be 2-byte aligned", who);
  if (rows > ((int64_t)1 << 40) / n_groups / n_ids)
    return fail(GQ_ERR_UNSUPPORTED, "%s: more than 2^40 packed words", who);
  return launch_decompress(packed, scale, bias, out, rows, n_groups, n_ids, transposed, (hipStream_t)stream);
}

}  // namespace
}  // namespace gq

extern "C" {

int gq_abi_version(void) { return GQ_ABI_VERSION; }

const char *gq_last_error(void) { return gq::g_error; }

int gq_decompress_f16(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, uint16_t *out,
                      int64_t rows, int64_t n_groups, int64_t n_ids, void *stream) {
  return gq::decompress_common("gq_decompress_f16", packed, scale, bias, out, rows, n_groups, n_ids, false,
                               stream);
}

int gq_decompress_f16_transposed(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                                 uint16_t *out_t, int64_t rows, int64_t n_groups, int64_t n_ids,
                                 void *stream) {
  return gq::decompress_common("gq_decompress_f16_transposed", packed, scale, bias, out_t, rows, n_groups,
                               n_ids, true, stream);
}

int gq_gemv_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, void *stream) {
  const int rc = gq::check_linear_args("gq_gemv_f16", x, m_rows, packed, scale, bias, out_bias, y, n_out,
                                       k_in, group_size);
  if (rc <= 0) return rc;
  if (m_rows > 16)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_f16: m_rows=%lld exceeds 16; use gq_gemm_f16",
                    (long long)m_rows);
  return gq::launch_gemv(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, GQ_ACT_NONE,
                         (hipStream_t)stream);
}

int gq_gemm_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, void *stream) {
  const int rc = gq::check_linear_args("gq_gemm_f16", x, m_rows, packed, scale, bias, out_bias, y, n_out,
                                       k_in, group_size);
  if (rc <= 0) return rc;
  return gq::launch_gemm(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, GQ_ACT_NONE, nullptr,
                         (hipStream_t)stream);
}

int gq_linear_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                  const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                  int64_t group_size, void *stream) {
  const int rc = gq::check_linear_args("gq_linear_f16", x, m_rows, packed, scale, bias, out_bias, y, n_out,
                                       k_in, group_size);
  if (rc <= 0) return rc;
  return gq_linear_act_f16(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, GQ_ACT_NONE, stream);
}

int gq_linear_act_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                      const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                      int64_t group_size, int32_t activation, void *stream) {
  return gq_linear_act_ws_f16(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, activation, nullptr, 0,
                              stream);
}

int64_t gq_gemm_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size) {
  if (m_rows <= 16) return 0;  // (the GEMV kernels take none)
  return gq::gemm_workspace_bytes(m_rows, n_out, k_in, group_size);
}

int gq_linear_act_ws_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                         const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                         int64_t group_size, int32_t activation, void *workspace, int64_t workspace_bytes, void *stream) {
  return gq_linear_p_act_f16(x, m_rows, packed, scale, bias, nullptr, out_bias, y, n_out, k_in, group_size, activation, workspace,
                             workspace_bytes, stream);
}

int gq_linear_p_act_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                        const uint16_t *bias, const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                        int64_t k_in, int64_t group_size, int32_t activation, void *workspace, int64_t workspace_bytes,
                        void *stream) {
  // With the copy, packed, scale and bias may all be NULL (a caller that keeps only the copy): every kernel then reads
  // the copy, which takes a 16-byte aligned x.  (The copy stands in for them in the checks shared with the other entry points.)
  const bool only_blob = blob && !packed && !scale && !bias;
  const uint16_t *const stand_in = static_cast<const uint16_t *>(blob);
  const int rc = gq::check_linear_args("gq_linear_act_f16", x, m_rows, only_blob ? stand_in : packed, only_blob ? stand_in : scale,
                                       only_blob ? stand_in : bias, out_bias, y, n_out, k_in, group_size);
  if (rc <= 0) return rc;
  if (activation < GQ_ACT_NONE || activation > GQ_ACT_GELU_TANH)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_linear_act_f16: unknown activation %d", (int)activation);
  if (blob) {
    const int64_t blob_bytes = gq_gemv_prepacked_bytes(n_out, k_in, group_size);
    if (blob_bytes < 0) return (int)blob_bytes;  // (no streaming layout for this shape: the message is set)
    if (gq::misaligned(blob, 16)) return gq::fail(GQ_ERR_MISALIGNED, "gq_linear_p_act_f16: blob must be 16-byte aligned");
    if (only_blob && gq::misaligned(x, 16))
      return gq::fail(GQ_ERR_MISALIGNED, "gq_linear_p_act_f16: without packed, scale and bias, x must be 16-byte aligned");
  }
  // the workspace is an option: one that is missing, misaligned or too small is not used
  if (m_rows <= 16 || !workspace || gq::misaligned(workspace, 16) ||
      workspace_bytes < gq_gemm_workspace_bytes(m_rows, n_out, k_in, group_size))
    workspace = nullptr;
  if (m_rows <= 16)
    return gq::launch_gemv(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, (int)activation,
                           (hipStream_t)stream, blob);
  int passes_rc = GQ_OK;
  if (gq::launch_gemv_passes(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, (int)activation,
                             workspace != nullptr, (hipStream_t)stream, &passes_rc, blob))
    return passes_rc;
  return gq::launch_gemm(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, (int)activation, workspace,
                         (hipStream_t)stream, blob);
}

int gq_linear_p_strided_f16(const uint16_t *x, int64_t x_row_stride, int64_t m_rows, const uint16_t *packed,
                            const uint16_t *scale, const uint16_t *bias, const void *blob, const uint16_t *out_bias,
                            uint16_t *y, int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation,
                            void *stream) {
  const bool only_blob = blob && !packed && !scale && !bias;
  const uint16_t *const stand_in = static_cast<const uint16_t *>(blob);
  const int rc = gq::check_linear_args("gq_linear_p_strided_f16", x, m_rows, only_blob ? stand_in : packed,
                                       only_blob ? stand_in : scale, only_blob ? stand_in : bias, out_bias, y, n_out, k_in,
                                       group_size);
  if (rc <= 0) return rc;
  if (x_row_stride < k_in)
    return gq::fail(GQ_ERR_BAD_SHAPE, "gq_linear_p_strided_f16: x_row_stride=%lld is less than k_in=%lld", (long long)x_row_stride,
                    (long long)k_in);
  if (x_row_stride > (int64_t)1 << 30) return gq::fail(GQ_ERR_UNSUPPORTED, "gq_linear_p_strided_f16: x_row_stride exceeds 2^30");
  if (m_rows > 16)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_linear_p_strided_f16: m_rows=%lld; rows of x apart are taken up to 16 rows "
                    "(gather x, or call per 16 rows)", (long long)m_rows);
  if (activation < GQ_ACT_NONE || activation > GQ_ACT_GELU_TANH)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_linear_p_strided_f16: unknown activation %d", (int)activation);
  if (blob) {
    const int64_t blob_bytes = gq_gemv_prepacked_bytes(n_out, k_in, group_size);
    if (blob_bytes < 0) return (int)blob_bytes;  // (no streaming layout for this shape: the message is set)
    if (gq::misaligned(blob, 16)) return gq::fail(GQ_ERR_MISALIGNED, "gq_linear_p_strided_f16: blob must be 16-byte aligned");
    if (only_blob && (gq::misaligned(x, 16) || x_row_stride % 8 != 0))
      return gq::fail(GQ_ERR_MISALIGNED, "gq_linear_p_strided_f16: without packed, scale and bias, every row of x must be "
                      "16-byte aligned (x, and x_row_stride %% 8 == 0)");
  }
  return gq::launch_gemv(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, (int)activation, (hipStream_t)stream,
                         blob, x_row_stride);
}

int64_t gq_linear_kn_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size) {
  if (m_rows < 0 || n_out < 0 || k_in < 0 || group_size <= 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "gq_linear_kn_workspace_bytes: negative size");
  return gq::linear_kn_workspace_bytes(m_rows, n_out, k_in, group_size);
}

// argument checks shared by the entry points of the [k_in, n_out] layout; 1 = proceed
static int check_linear_kn_args(const char *who, const uint16_t *x, int64_t m_rows, const uint16_t *packed,
                                const uint16_t *scale, const uint16_t *bias, const uint16_t *out_bias, uint16_t *y,
                                int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation) {
  if (m_rows < 0 || n_out < 0 || k_in < 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "%s: negative size (m_rows=%lld n_out=%lld k_in=%lld)", who, (long long)m_rows,
                    (long long)n_out, (long long)k_in);
  if (group_size <= 0 || group_size % 4 != 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "%s: group_size=%lld must be a positive multiple of 4", who, (long long)group_size);
  if (n_out % group_size != 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "%s: n_out=%lld is not a multiple of group_size=%lld", who, (long long)n_out,
                    (long long)group_size);
  if (activation < GQ_ACT_NONE || activation > GQ_ACT_GELU_TANH)
    return gq::fail(GQ_ERR_UNSUPPORTED, "%s: unknown activation %d", who, (int)activation);
  if (m_rows == 0 || n_out == 0) return GQ_OK;
  if (!y) return gq::fail(GQ_ERR_NULL_POINTER, "%s: y is NULL", who);
  if (k_in > 0 && (!x || !packed || !scale || !bias))
    return gq::fail(GQ_ERR_NULL_POINTER, "%s: x/packed/scale/bias must not be NULL", who);
  if (gq::misaligned(x, 2) || gq::misaligned(packed, 2) || gq::misaligned(scale, 2) || gq::misaligned(bias, 2) ||
      gq::misaligned(out_bias, 2) || gq::misaligned(y, 2))
    return gq::fail(GQ_ERR_MISALIGNED, "%s: pointers must be 2-byte aligned", who);
  if (m_rows > (int64_t)1 << 30 || n_out > (int64_t)1 << 30 || k_in > (int64_t)1 << 30)
    return gq::fail(GQ_ERR_UNSUPPORTED, "%s: a dimension exceeds 2^30", who);
  return 1;
}

int gq_linear_kn_act_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                         const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                         int64_t group_size, int32_t activation, void *workspace, int64_t workspace_bytes,
                         void *stream) {
  const int rc = check_linear_kn_args("gq_linear_kn_act_f16", x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in,
                                      group_size, activation);
  if (rc <= 0) return rc;
  const int64_t need = gq::linear_kn_workspace_bytes(m_rows, n_out, k_in, group_size);
  // (more than 16 rows: the workspace is an option -- with one that is large enough the batch may run as
  // passes of the decode kernel, without it the prefill kernel runs)
  if (m_rows > 16 && (!workspace || workspace_bytes < need || gq::misaligned(workspace, 16))) {
    workspace = nullptr;
  } else if (need > 0) {
    if (!workspace) return gq::fail(GQ_ERR_NULL_POINTER, "gq_linear_kn_act_f16: this problem needs a workspace of %lld bytes",
                                    (long long)need);
    if (gq::misaligned(workspace, 16))
      return gq::fail(GQ_ERR_MISALIGNED, "gq_linear_kn_act_f16: workspace must be 16-byte aligned");
    if (workspace_bytes < need)
      return gq::fail(GQ_ERR_BAD_SHAPE, "gq_linear_kn_act_f16: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
                      (long long)need);
  }
  return gq::launch_linear_kn(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size, (int)activation,
                              workspace, (hipStream_t)stream);
}

int gq_linear_kn_act_noalloc_f16(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                                 const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                                 int64_t k_in, int64_t group_size, int32_t activation, void *stream) {
  const int rc = check_linear_kn_args("gq_linear_kn_act_noalloc_f16", x, m_rows, packed, scale, bias, out_bias, y, n_out,
                                      k_in, group_size, activation);
  if (rc <= 0) return rc;
  return gq::launch_linear_kn_noalloc(x, m_rows, packed, scale, bias, out_bias, y, n_out, k_in, group_size,
                                      (int)activation, (hipStream_t)stream);
}

static int gemv_sequence_common(const gq_gemv_desc *descs, const gq_gemv_desc *descs_device, int64_t count,
                                int32_t *status, void *workspace, int64_t spin_limit, void *stream) {
  if (count < 0) return gq::fail(GQ_ERR_BAD_SHAPE, "gq_gemv_sequence_f16: negative count");
  if (count == 0) return GQ_OK;
  if (!descs || !descs_device) return gq::fail(GQ_ERR_NULL_POINTER, "gq_gemv_sequence_f16: descs is NULL");
  if (gq::misaligned(descs_device, 8) || gq::misaligned(status, 4))
    return gq::fail(GQ_ERR_MISALIGNED, "gq_gemv_sequence_f16: misaligned descs_device or status");
  for (int64_t i = 0; i < count; ++i) {
    const gq_gemv_desc &d = descs[i];
    const bool blob = d.scale == nullptr && d.bias == nullptr && d.packed != nullptr;
    if (d.activation & GQ_DESC_KN_LAYOUT) {
      // a weight grouped along the output features, in the kn streaming layout
      const int act = d.activation & ~GQ_DESC_KN_LAYOUT;
      if (!blob)
        return gq::fail(GQ_ERR_UNSUPPORTED,
                        "gq_gemv_sequence_f16: entry %lld is marked GQ_DESC_KN_LAYOUT: `packed` must be the blob written by "
                        "gq_gemv_kn_prepack_f16 and scale, bias NULL", (long long)i);
      if (!gq::gemv_kn_prepack_shape_ok(d.n_out, d.k_in, d.group_size) || d.m_rows < 1 || d.m_rows > 16)
        return gq::fail(GQ_ERR_UNSUPPORTED,
                        "gq_gemv_sequence_f16: entry %lld is in the kn streaming layout, which needs group_size 64, n_out %% 64 == 0, "
                        "k_in %% 512 == 0 and 1 <= m_rows <= 16 (got group_size=%d n_out=%d k_in=%d m_rows=%d)",
                        (long long)i, d.group_size, d.n_out, d.k_in, d.m_rows);
      if (!d.x || !d.y) return gq::fail(GQ_ERR_NULL_POINTER, "gq_gemv_sequence_f16: entry %lld: x or y is NULL", (long long)i);
      if (gq::misaligned(d.packed, 16) || gq::misaligned(d.x, 16) || gq::misaligned(d.y, 8) || gq::misaligned(d.out_bias, 2))
        return gq::fail(GQ_ERR_MISALIGNED, "gq_gemv_sequence_f16: entry %lld: blob and x must be 16-byte aligned, y 8-byte",
                        (long long)i);
      if (act < GQ_ACT_NONE || act > GQ_ACT_GELU_TANH)
        return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_sequence_f16: entry %lld has unknown activation %d", (long long)i, act);
      if (d.wait_entries < 0 || d.wait_entries > i)
        return gq::fail(GQ_ERR_BAD_SHAPE, "gq_gemv_sequence_f16: entry %lld has wait_entries=%d outside [0, %lld]",
                        (long long)i, d.wait_entries, (long long)i);
      continue;
    }
    if (blob) {
      // the weight in the streaming layout (the persistent kernels up to 4 rows, a launch of the one-shot kernel above)
      if (d.group_size != 64 || d.k_in <= 0 || d.k_in % 512 != 0 || d.m_rows < 1 || d.m_rows > 16 || d.n_out < 1)
        return gq::fail(GQ_ERR_UNSUPPORTED,
                        "gq_gemv_sequence_f16: entry %lld is in the streaming layout, which needs group_size 64, "
                        "k_in %% 512 == 0 and 1 <= m_rows <= 16 (got group_size=%d k_in=%d m_rows=%d n_out=%d)",
                        (long long)i, d.group_size, d.k_in, d.m_rows, d.n_out);
      if (gq::misaligned(d.packed, 16) || gq::misaligned(d.x, 16))
        return gq::fail(GQ_ERR_MISALIGNED, "gq_gemv_sequence_f16: entry %lld: blob and x must be 16-byte aligned",
                        (long long)i);
    }
    // (the blob stands in for scale and bias in the checks shared with the other entry points)
    const int rc = gq::check_linear_args("gq_gemv_sequence_f16", d.x, d.m_rows, d.packed, blob ? d.packed : d.scale,
                                         blob ? d.packed : d.bias, d.out_bias, d.y, d.n_out, d.k_in, d.group_size);
    if (rc < 0) return rc;
    if (rc == 0 || d.k_in == 0)
      return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_sequence_f16: entry %lld is empty", (long long)i);
    if (d.m_rows > 16)
      return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_sequence_f16: entry %lld has m_rows=%d > 16", (long long)i,
                      d.m_rows);
    if (d.activation < GQ_ACT_NONE || d.activation > GQ_ACT_GELU_TANH)
      return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_sequence_f16: entry %lld has unknown activation %d", (long long)i,
                      d.activation);
    if (d.wait_entries < 0 || d.wait_entries > i)
      return gq::fail(GQ_ERR_BAD_SHAPE, "gq_gemv_sequence_f16: entry %lld has wait_entries=%d outside [0, %lld]",
                      (long long)i, d.wait_entries, (long long)i);
  }
  return gq::launch_gemv_sequence(descs, descs_device, count, status, workspace, spin_limit, (hipStream_t)stream);
}

int gq_gemv_sequence_f16(const gq_gemv_desc *descs, const gq_gemv_desc *descs_device, int64_t count,
                         int32_t *status, void *stream) {
  return gemv_sequence_common(descs, descs_device, count, status, nullptr, 0, stream);
}

int64_t gq_gemv_sequence_workspace_bytes(void) { return gq::gemv_sequence_workspace_bytes(); }

int gq_gemv_sequence_ws_f16(const gq_gemv_desc *descs, const gq_gemv_desc *descs_device, int64_t count,
                            int32_t *status, void *workspace, int64_t workspace_bytes, int64_t spin_limit,
                            void *stream) {
  if (count > 0) {
    if (!workspace) return gq::fail(GQ_ERR_NULL_POINTER, "gq_gemv_sequence_ws_f16: workspace is NULL");
    if (gq::misaligned(workspace, 256))
      return gq::fail(GQ_ERR_MISALIGNED, "gq_gemv_sequence_ws_f16: workspace must be 256-byte aligned");
    if (workspace_bytes < gq::gemv_sequence_workspace_bytes())
      return gq::fail(GQ_ERR_BAD_SHAPE, "gq_gemv_sequence_ws_f16: workspace of %lld bytes, need %lld",
                      (long long)workspace_bytes, (long long)gq::gemv_sequence_workspace_bytes());
  }
  return gemv_sequence_common(descs, descs_device, count, status, workspace, spin_limit, stream);
}

int64_t gq_gemv_prepacked_bytes(int64_t n_out, int64_t k_in, int64_t group_size) {
  if (n_out < 0 || k_in < 0) return gq::fail(GQ_ERR_BAD_SHAPE, "gq_gemv_prepacked_bytes: negative size");
  if (group_size != 64 || k_in % 512 != 0)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_prepacked_bytes: the streaming layout needs group_size 64 and k_in %% 512 == 0 "
                                        "(got group_size=%lld k_in=%lld)", (long long)group_size, (long long)k_in);
  if (n_out > (1 << 22) || k_in > (1 << 24))
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_gemv_prepacked_bytes: n_out=%lld or k_in=%lld too large", (long long)n_out,
                    (long long)k_in);
  return gq::gemv_prepacked_bytes(n_out, k_in);
}

int gq_gemv_prepack_f16(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob, int64_t n_out,
                        int64_t k_in, int64_t group_size, void *stream) {
  const int64_t bytes = gq_gemv_prepacked_bytes(n_out, k_in, group_size);
  if (bytes < 0) return (int)bytes;
  if (bytes == 0) return GQ_OK;
  if (!packed || !scale || !bias || !blob) return gq::fail(GQ_ERR_NULL_POINTER, "gq_gemv_prepack_f16: NULL pointer argument");
  if (gq::misaligned(packed, 16) || gq::misaligned(scale, 16) || gq::misaligned(bias, 16) || gq::misaligned(blob, 16))
    return gq::fail(GQ_ERR_MISALIGNED, "gq_gemv_prepack_f16: pointers must be 16-byte aligned");
  return gq::launch_gemv_prepack(packed, scale, bias, blob, n_out, k_in, (hipStream_t)stream);
}

int64_t gq_gemv_kn_prepacked_bytes(int64_t n_out, int64_t k_in, int64_t group_size) {
  if (n_out < 0 || k_in < 0) return gq::fail(GQ_ERR_BAD_SHAPE, "gq_gemv_kn_prepacked_bytes: negative size");
  if (n_out == 0 || k_in == 0) return 0;
  if (!gq::gemv_kn_prepack_shape_ok(n_out, k_in, group_size))
    return gq::fail(GQ_ERR_UNSUPPORTED,
                    "gq_gemv_kn_prepacked_bytes: the kn streaming layout needs group_size 64, n_out %% 64 == 0, k_in %% 512 == 0, "
                    "n_out <= 2^22 and k_in <= 2^24 (got group_size=%lld n_out=%lld k_in=%lld)",
                    (long long)group_size, (long long)n_out, (long long)k_in);
  return gq::gemv_kn_prepacked_bytes(n_out, k_in);
}

int gq_gemv_kn_prepack_f16(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob, int64_t n_out,
                           int64_t k_in, int64_t group_size, void *stream) {
  const int64_t bytes = gq_gemv_kn_prepacked_bytes(n_out, k_in, group_size);
  if (bytes < 0) return (int)bytes;
  if (bytes == 0) return GQ_OK;
  if (!packed || !scale || !bias || !blob) return gq::fail(GQ_ERR_NULL_POINTER, "gq_gemv_kn_prepack_f16: NULL pointer argument");
  if (gq::misaligned(packed, 2) || gq::misaligned(scale, 2) || gq::misaligned(bias, 2) || gq::misaligned(blob, 16))
    return gq::fail(GQ_ERR_MISALIGNED, "gq_gemv_kn_prepack_f16: the blob must be 16-byte aligned, the other pointers 2-byte");
  return gq::launch_gemv_kn_prepack(packed, scale, bias, blob, n_out, k_in, (hipStream_t)stream);
}

// argument checks shared by the two entry points on the kn streaming layout; 1 = proceed
static int check_linear_knp_args(const char *who, const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias,
                                 uint16_t *y, int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation) {
  if (m_rows < 0 || n_out < 0 || k_in < 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "%s: negative size (m_rows=%lld n_out=%lld k_in=%lld)", who, (long long)m_rows,
                    (long long)n_out, (long long)k_in);
  if (activation < GQ_ACT_NONE || activation > GQ_ACT_GELU_TANH)
    return gq::fail(GQ_ERR_UNSUPPORTED, "%s: unknown activation %d", who, (int)activation);
  if (m_rows == 0 || n_out == 0) return GQ_OK;
  if (!gq::gemv_kn_prepack_shape_ok(n_out, k_in, group_size))
    return gq::fail(GQ_ERR_UNSUPPORTED,
                    "%s: the kn streaming layout needs group_size 64, n_out %% 64 == 0 and k_in %% 512 == 0 (got "
                    "group_size=%lld n_out=%lld k_in=%lld)", who, (long long)group_size, (long long)n_out, (long long)k_in);
  if (!x || !blob || !y) return gq::fail(GQ_ERR_NULL_POINTER, "%s: x, blob and y must not be NULL", who);
  if (gq::misaligned(x, 16) || gq::misaligned(blob, 16) || gq::misaligned(y, 8) || gq::misaligned(out_bias, 2))
    return gq::fail(GQ_ERR_MISALIGNED, "%s: x and blob must be 16-byte aligned, y 8-byte, out_bias 2-byte", who);
  if (m_rows > (int64_t)1 << 30) return gq::fail(GQ_ERR_UNSUPPORTED, "%s: m_rows exceeds 2^30", who);
  return 1;
}

int gq_linear_knp_strided_f16(const uint16_t *x, int64_t x_row_stride, int64_t m_rows, const void *blob, const uint16_t *out_bias,
                              uint16_t *y, int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation, void *stream) {
  const int rc = check_linear_knp_args("gq_linear_knp_strided_f16", x, m_rows, blob, out_bias, y, n_out, k_in, group_size, activation);
  if (rc <= 0) return rc;
  if (x_row_stride < k_in)
    return gq::fail(GQ_ERR_BAD_SHAPE, "gq_linear_knp_strided_f16: x_row_stride=%lld is less than k_in=%lld", (long long)x_row_stride,
                    (long long)k_in);
  if (x_row_stride > (int64_t)1 << 30) return gq::fail(GQ_ERR_UNSUPPORTED, "gq_linear_knp_strided_f16: x_row_stride exceeds 2^30");
  if (x_row_stride % 8 != 0)
    return gq::fail(GQ_ERR_MISALIGNED, "gq_linear_knp_strided_f16: every row of x must be 16-byte aligned (x_row_stride %% 8 == 0)");
  if (m_rows > 16)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_linear_knp_strided_f16: m_rows=%lld; rows of x apart are taken up to 16 rows "
                    "(gather x, or call per 16 rows)", (long long)m_rows);
  return gq::launch_gemv_knp(x, m_rows, blob, out_bias, y, n_out, k_in, (int)activation, (hipStream_t)stream, x_row_stride);
}

int gq_linear_knp_act_f16(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias, uint16_t *y,
                          int64_t n_out, int64_t k_in, int64_t group_size, int32_t activation, void *stream) {
  const int args_rc = check_linear_knp_args("gq_linear_knp_act_f16", x, m_rows, blob, out_bias, y, n_out, k_in, group_size, activation);
  if (args_rc <= 0) return args_rc;
  if (m_rows <= 16) return gq::launch_gemv_knp(x, m_rows, blob, out_bias, y, n_out, k_in, (int)activation, (hipStream_t)stream);
  // 17 to 32 rows: two passes of the decode kernel over 16 rows each are faster than the prefill kernel's
  // mostly empty tiles (as for the other layout)
  if (m_rows <= 32) {
    const int rc = gq::launch_gemv_knp(x, 16, blob, out_bias, y, n_out, k_in, (int)activation, (hipStream_t)stream);
    if (rc != GQ_OK) return rc;
    return gq::launch_gemv_knp(x + 16 * k_in, m_rows - 16, blob, out_bias, y + 16 * n_out, n_out, k_in, (int)activation,
                               (hipStream_t)stream);
  }
  return gq::launch_gemm_knp(x, m_rows, blob, out_bias, y, n_out, k_in, (int)activation, (hipStream_t)stream);
}

int gq_compress_f16(const uint16_t *t, uint16_t *packed, uint16_t *scale, uint16_t *bias,
                    int32_t *nonfinite_flag, int64_t rows, int64_t n_groups, int64_t group_size,
                    void *stream) {
  if (rows < 0 || n_groups < 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "gq_compress_f16: negative size");
  if (group_size <= 0 || group_size % 4 != 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "gq_compress_f16: group_size=%lld must be a positive multiple of 4",
                    (long long)group_size);
  if (rows == 0 || n_groups == 0) return GQ_OK;
  if (!t || !packed || !scale || !bias) return gq::fail(GQ_ERR_NULL_POINTER, "gq_compress_f16: NULL pointer argument");
  if (gq::misaligned(t, 2) || gq::misaligned(packed, 2) || gq::misaligned(scale, 2) ||
      gq::misaligned(bias, 2) || gq::misaligned(nonfinite_flag, 4))
    return gq::fail(GQ_ERR_MISALIGNED, "gq_compress_f16: misaligned pointer");
  if (rows > ((int64_t)1 << 40) / n_groups / group_size)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_compress_f16: more than 2^40 elements");
  return gq::launch_compress(t, packed, scale, bias, nonfinite_flag, rows, n_groups, group_size,
                             (hipStream_t)stream);
}

int gq_compress_f32(const float *t, uint16_t *packed, uint16_t *scale, uint16_t *bias, int32_t *nonfinite_flag,
                    int64_t rows, int64_t n_groups, int64_t group_size, void *stream) {
  if (rows < 0 || n_groups < 0) return gq::fail(GQ_ERR_BAD_SHAPE, "gq_compress_f32: negative size");
  if (group_size <= 0 || group_size % 4 != 0)
    return gq::fail(GQ_ERR_BAD_SHAPE, "gq_compress_f32: group_size=%lld must be a positive multiple of 4",
                    (long long)group_size);
  if (rows == 0 || n_groups == 0) return GQ_OK;
  if (!t || !packed || !scale || !bias) return gq::fail(GQ_ERR_NULL_POINTER, "gq_compress_f32: NULL pointer argument");
  if (gq::misaligned(t, 4) || gq::misaligned(packed, 2) || gq::misaligned(scale, 2) || gq::misaligned(bias, 2) ||
      gq::misaligned(nonfinite_flag, 4))
    return gq::fail(GQ_ERR_MISALIGNED, "gq_compress_f32: misaligned pointer");
  if (rows > ((int64_t)1 << 40) / n_groups / group_size)
    return gq::fail(GQ_ERR_UNSUPPORTED, "gq_compress_f32: more than 2^40 elements");
  return gq::launch_compress_f32(t, packed, scale, bias, nonfinite_flag, rows, n_groups, group_size,
                                 (hipStream_t)stream);
}

}  // extern "C"
