// Chooses between the decode (GEMV) and prefill (MFMA GEMM) kernels of the quantized matmul.
#include "kernels.h"

namespace htpops {

size_t mat_mul_workspace_bytes(int m, int k) {
  return gemm_workspace_bytes(m, k);
}

hipError_t launch_mat_mul_q8_0_act(hipStream_t stream, float *out, const void *act, const void *weight, int m, int k,
                                   int n, WeightType wt, void *workspace) {
  // One activation row: pure weight streaming. More rows: the MFMA kernel reads the weights once for all rows.
  static const int gemm_min_m = env_int("HTPOPS_GEMM_MIN_M", 2);
  if (m < gemm_min_m) {
    return launch_gemv_q8_0_act(stream, out, act, weight, m, k, n, wt);
  }
  hipError_t e = launch_gemm_q8_0_act(stream, out, act, weight, m, k, n, wt, workspace);
  if (e == hipErrorNotSupported) {
    return launch_gemv_q8_0_act(stream, out, act, weight, m, k, n, wt);
  }
  return e;
}

}  // namespace htpops
