// bfloat16 matrix products on the matrix cores (MFMA).  Only in the bfloat16 build.
#include "api.h"
#include "common.h"

#if AXON_BF16
int launch_gemm_mfma(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                     int out_stride, int m, int n, int k, int mode, hipStream_t stream, bool* handled) {
  *handled = false;
  return 0;
}
#endif
