// placeholder until the fused GEMM lands
#include "device_utils.h"
extern "C" int actnn_linear_grad_weight_q2(const void*, const int8_t*, const void*, const void*, void*,
                                           int64_t, int64_t, int64_t, int, int, int, void*) {
  return ACTNN_EINVAL;
}
