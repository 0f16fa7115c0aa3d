// Gate activation shared by the KDA kernels.
// fla/ops/ascendc/kda/kda_gate_cumsum/op_kernel/kda_gate_cumsum_kernel.h:374-419:
//   raw = g + dt_bias;  safe gate: lower_bound * sigmoid(e^{A_log} raw);  otherwise -e^{A_log} softplus(raw).
#pragma once

#include "device_utils.h"

namespace fla {

constexpr float kRcpLn2 = 1.4426950408889634f;

__device__ __forceinline__ float kda_activate(float x, float bias, float eig, int safe, float lower_bound) {
    const float raw = x + bias;
    if (safe) return lower_bound * __builtin_amdgcn_rcpf(1.f + __expf(-eig * raw));  // 1-ulp reciprocal
    const float sp = fmaxf(raw, 0.f) + __logf(1.f + __expf(-fabsf(raw)));
    return -eig * sp;
}

}  // namespace fla
