// The toy recurrent mixer's own kernel (a test's, not the engine's): for each request's tokens
// in the step, in order, s = decay * s + u[t]; out[t] = s; the request's state is s afterwards.
// One block a span, a thread a state element.  Built by the engine from this file alone
// (register_kernel_source), with the engine's headers on the include path.
#include "api.h"
#include "common.h"

__global__ void toy_decay_scan_kernel(const float* __restrict__ u, float* __restrict__ state, int state_stride,
                                      const int32_t* __restrict__ spans, float decay, elem_t* __restrict__ out, int width) {
  const int slot = spans[3 * blockIdx.x], first = spans[3 * blockIdx.x + 1], count = spans[3 * blockIdx.x + 2];
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    float s = state[(size_t)slot * state_stride + j];
    for (int t = first; t < first + count; ++t) {
      s = __fadd_rn(__fmul_rn(decay, s), u[(size_t)t * width + j]);
      out[(size_t)t * width + j] = from_float(s);
    }
    state[(size_t)slot * state_stride + j] = s;
  }
}

// spans [n_spans][3] = (state slot, first token, tokens), on the device; out [tokens, width] in the compute dtype
extern "C" int toy_decay_scan(const float* u, float* state, int state_stride, const int32_t* spans, int n_spans, float decay,
                              void* out, int width, void* stream) {
  AXK_REQUIRE(n_spans >= 0 && width > 0 && state_stride >= width, "toy_decay_scan: %d spans, width %d, state stride %d",
              n_spans, width, state_stride);
  if (n_spans == 0) return 0;
  toy_decay_scan_kernel<<<n_spans, 64, 0, (hipStream_t)stream>>>(u, state, state_stride, spans, decay, (elem_t*)out, width);
  AXK_LAUNCH_CHECK("toy_decay_scan");
  return 0;
}
