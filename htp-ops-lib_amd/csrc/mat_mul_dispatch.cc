// Chooses between the one-row (GEMV) and small-batch (skinny MFMA) kernels of the quantized matmul. Many rows
// (prefill) go through launch_gemm_i8_fragments, which needs converted weights and is therefore routed by the
// caller that owns the conversion cache.
#include "kernels.h"

namespace htpops {

size_t mat_mul_workspace_bytes(int m, int k, int n) {
  return matmul_skinny_workspace_bytes(m, k, n);
}

hipError_t launch_mat_mul_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                   int n, WeightType wt, void *workspace, unsigned *tickets, int ticket_slots) {
  // One activation row: pure weight streaming, one lane group per weight row.
  if (m == 1) {
    return launch_gemv_q8_0_act(stream, out, act, weight, m, k, n, wt);
  }
  // A handful of rows: still weight streaming, with the block dots on the matrix core; 32 rows per pass.
  if (k % 64 == 0) {
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
  // rows that are not dword multiples (k = 32 * odd): the generic kernel, row by row
  return launch_gemv_q8_0_act(stream, out, act, weight, m, k, n, wt);
}

}  // namespace htpops
