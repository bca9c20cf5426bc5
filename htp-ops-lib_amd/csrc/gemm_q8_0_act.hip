#include "kernels.h"
namespace htpops {
hipError_t launch_gemm_q8_0_act(hipStream_t, float *, const void *, const void *, int, int, int, WeightType) {
  return hipErrorNotSupported;
}
}  // namespace htpops
