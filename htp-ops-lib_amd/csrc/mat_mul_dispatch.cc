// Chooses between the decode (GEMV), small-batch (skinny MFMA) and prefill (MFMA GEMM) kernels of the quantized matmul.
#include "kernels.h"

namespace htpops {

size_t mat_mul_workspace_bytes(int m, int k, int n) {
  const size_t a = gemm_workspace_bytes(m, k), b = matmul_skinny_workspace_bytes(m, k, n);
  return a > b ? a : b;
}

hipError_t launch_mat_mul_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                   int n, WeightType wt, void *workspace, unsigned *tickets, int ticket_slots) {
  // One activation row: pure weight streaming. More rows: the MFMA kernel reads the weights once for all rows.
  static const int gemm_min_m   = env_int("HTPOPS_GEMM_MIN_M", 2);
  static const int skinny_max_m = env_int("HTPOPS_SKINNY_MAX_M", 63);
  if (m < gemm_min_m) {
    return launch_gemv_q8_0_act(stream, out, act, weight, m, k, n, wt);
  }
  // A handful of rows: still weight streaming, with the block dots on the matrix core; 32 rows per pass.
  if (m <= skinny_max_m && k % 64 == 0) {
    const size_t act_row = (size_t) (k / 32) * 34;
    for (int m0 = 0; m0 < m; m0 += 32) {
      const int  rows = m - m0 < 32 ? m - m0 : 32;
      hipError_t e    = launch_matmul_skinny(stream, out + (size_t) m0 * n,
                                             static_cast<const uint8_t *>(act) + (size_t) m0 * act_row, weight, rows, k, n,
                                             wt, workspace, tickets, ticket_slots);
      if (e != hipSuccess) {
        return e;
      }
    }
    return hipSuccess;
  }
  hipError_t e = launch_gemm_q8_0_act(stream, out, act, weight, m, k, n, wt, workspace);
  if (e == hipErrorNotSupported) {
    return launch_gemv_q8_0_act(stream, out, act, weight, m, k, n, wt);
  }
  return e;
}

}  // namespace htpops
