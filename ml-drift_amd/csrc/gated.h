// dst = activation(gate) * up: the elementwise step after the gate and up projections of a
// decoder layer, in fp32 and in the operation order of the LLM sample's kernels
// (samples/llm/gemma3_model_builder.cc:1054-1090 CreateGeluTanhMulOp,
// samples/llm/qwen3_model_builder.cc:850-883 CreateSiluMulOp).  Device code only.
#ifndef MLDHIP_CSRC_GATED_H_
#define MLDHIP_CSRC_GATED_H_

#include <hip/hip_runtime.h>

#include "../../include/mldhip.h"

namespace mldhip {

__device__ __forceinline__ float GatedActivation(int act, float g, float u) {
  if (act == MLDHIP_GATE_GELU_TANH) {
    const float gate_sq = g * g;
    const float tanh_in = g * (0.7978845608f + 0.03567740813f * gate_sq);
    const float clamped = fminf(fmaxf(tanh_in, -10.0f), 10.0f);
    // tanh(x) = 1 - 2 / (exp(2x) + 1) on the hardware exponential and reciprocal (|x| <= 10, so
    // exp(2x) stays finite): a few fp32 ulp, far below the fp16 rounding of the result, and a
    // handful of instructions where the library routine takes a hundred at the tail of a GEMM tile
    const float tanh_val = 1.0f - 2.0f * __frcp_rn(__expf(2.0f * clamped) + 1.0f);
    const float gate_up_half = 0.5f * g * u;
    return fminf(fmaxf(gate_up_half * (1.0f + tanh_val), -65504.0f), 65504.0f);
  }
  const float sig = __frcp_rn(1.0f + __expf(-g));  // exp(-g) = inf for very negative g: sig = 0
  const float silu = g * sig;
  return fminf(fmaxf(silu * u, -65504.0f), 65504.0f);
}

}  // namespace mldhip

#endif  // MLDHIP_CSRC_GATED_H_
