// Internal helpers shared by the gfx950 kernels and the C-ABI layer of libgq_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gq_hip.h"

namespace gq {

// Records a message for gq_last_error() on the calling thread and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Maps the runtime's last launch error (if any) to a return code, recording its text.
int check_launch(const char *what);

// A block of device memory that the library keeps per GPU and every call on that GPU shares (the
// progress words of gq_gemv_sequence_f16, the scratch of gq_linear_kn_act_noalloc_f16): calls
// that use it are ordered by the stream they are enqueued on.  Remembers the stream of the last
// call per device; a call on ANOTHER stream while that stream still has work pending is refused
// (GQ_ERR_UNSUPPORTED, nothing launched) instead of racing silently.  A stream under capture is
// neither checked nor remembered (replays of a graph are the caller's to order).
struct SharedBlockGuard {
  static constexpr int kMaxDevices = 64;
  hipStream_t last[kMaxDevices];
  bool used[kMaxDevices];
};
int claim_shared_block(SharedBlockGuard &guard, int dev, hipStream_t stream, const char *who);

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

// Epilogue applied to sum + out_bias before the result is rounded to binary16 (GQ_ACT_* of the C ABI).
__device__ __forceinline__ float apply_activation(float v, int act) {
  if (act == GQ_ACT_RELU) return fmaxf(v, 0.f);
  if (act == GQ_ACT_GELU_TANH) {
    const float u = 0.7978845608028654f * (v + 0.044715f * (v * v * v));
    return 0.5f * v * (1.f + tanhf(u));
  }
  return v;
}

// Launchers implemented next to their kernels.
int launch_decompress(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, uint16_t *out,
                      int64_t rows, int64_t n_groups, int64_t n_ids, bool transposed, hipStream_t stream);
// blob: NULL, or the same weight in the streaming layout of gq_gemv_prepack_f16 (packed, scale, bias may then be NULL)
// ldx: elements from a row of x to the next (0: k_in) -- here and in the two launchers below
int launch_gemv(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, int act, hipStream_t stream, const void *blob = nullptr, int64_t ldx = 0);
// One or two batch rows, group 64, k_in % 512 == 0, x / packed (or blob) 16-byte and scale / bias 4-byte aligned:
// scale and bias applied to group sums (gq_gemv_sums.hip).  blob: NULL, or the weight's streaming-layout copy.
int launch_gemv_sums(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                     const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in, int act,
                     hipStream_t stream, int64_t ldx = 0);
// Three to eight batch rows, group 64, x / packed (or blob) / scale / bias 16-byte aligned, a shape that gemv_rows_fits
// (k_in <= 4096, a multiple of 512; rows enough to fill the compute units): the waves of a workgroup share the rows' x
// (gq_gemv_rows.hip).  blob: NULL, or the weight's streaming-layout copy.
bool gemv_rows_fits(int64_t m_rows, int64_t n_out, int64_t k_in);
int launch_gemv_rows(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale, const uint16_t *bias,
                     const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in, int act,
                     hipStream_t stream, int64_t ldx = 0);
// workspace: NULL, or gemm_workspace_bytes() bytes (first 16 KiB zero), with which K may be divided over workgroups
// blob: NULL, or the same weight in the streaming layout of gq_gemv_prepack_f16, which the pipelined kernel then reads
int launch_gemm(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                int64_t group_size, int act, void *workspace, hipStream_t stream, const void *blob = nullptr);
int64_t gemm_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size);
double gemm_expected_us(int64_t m_rows, int64_t n_out, int64_t k_in, bool may_split);
// Batches of 17 to 128 rows as passes of the GEMV kernel over 16 rows each, where that is expected
// to beat the GEMM kernel (whose 128 x 64 tiles are mostly empty there); false: not such a case,
// nothing launched.
bool launch_gemv_passes(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                        const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                        int64_t group_size, int act, bool gemm_may_split, hipStream_t stream, int *rc, const void *blob = nullptr);
int launch_gemv_generic_rows(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                             const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                             int64_t k_in, int64_t group_size, int act, hipStream_t stream);
int launch_gemv_streamed(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                         const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                         int64_t group_size, int act, hipStream_t stream);
// workspace: the sequence's progress words (gemv_sequence_workspace_bytes() zeroed bytes), or
// nullptr for the block the library keeps per device; spin_limit <= 0: the default
int launch_gemv_sequence(const gq_gemv_desc *host, const gq_gemv_desc *device, int64_t count, int *status,
                         void *workspace, int64_t spin_limit, hipStream_t stream);
int64_t gemv_sequence_workspace_bytes();
int64_t linear_kn_workspace_bytes(int64_t m_rows, int64_t n_out, int64_t k_in, int64_t group_size);
int launch_linear_kn(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                     const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                     int64_t group_size, int act, void *workspace, hipStream_t stream);
int launch_linear_kn_noalloc(const uint16_t *x, int64_t m_rows, const uint16_t *packed, const uint16_t *scale,
                             const uint16_t *bias, const uint16_t *out_bias, uint16_t *y, int64_t n_out, int64_t k_in,
                             int64_t group_size, int act, hipStream_t stream);
int64_t gemv_prepacked_bytes(int64_t n_out, int64_t k_in);
int launch_gemv_prepack(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob, int64_t n_out,
                        int64_t k_in, hipStream_t stream);
// the kn streaming layout (weights grouped along the output features) and the GEMV that reads it
bool gemv_kn_prepack_shape_ok(int64_t n_out, int64_t k_in, int64_t group_size);
int64_t gemv_kn_prepacked_bytes(int64_t n_out, int64_t k_in);
int launch_gemv_kn_prepack(const uint16_t *packed, const uint16_t *scale, const uint16_t *bias, void *blob, int64_t n_out,
                           int64_t k_in, hipStream_t stream);
int launch_gemv_knp(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                    int64_t k_in, int act, hipStream_t stream, int64_t ldx = 0);
int launch_gemm_knp(const uint16_t *x, int64_t m_rows, const void *blob, const uint16_t *out_bias, uint16_t *y, int64_t n_out,
                    int64_t k_in, int act, hipStream_t stream);
int launch_compress(const uint16_t *t, uint16_t *packed, uint16_t *scale, uint16_t *bias, int32_t *flag,
                    int64_t rows, int64_t n_groups, int64_t group_size, hipStream_t stream);
int launch_compress_f32(const float *t, uint16_t *packed, uint16_t *scale, uint16_t *bias, int32_t *flag,
                        int64_t rows, int64_t n_groups, int64_t group_size, hipStream_t stream);

}  // namespace gq
