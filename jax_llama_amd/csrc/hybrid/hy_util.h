// Small device helpers shared by the hybrid-mixer kernels.
#pragma once
#include "../kernels/common.h"

namespace jla {

// 8 consecutive elements of a row (zero beyond the `n` valid ones) as floats; 16-byte loads where aligned
JLA_DEV void hy_load8(const float* p, int n, float* f) {
  if (n >= 8 && ((uintptr_t)p & 15) == 0) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = i < n ? p[i] : 0.f;
  }
}
JLA_DEV void hy_load8(const bf16_t* p, int n, float* f) {
  if (n >= 8 && ((uintptr_t)p & 15) == 0) {
    unpack8(*reinterpret_cast<const u32x4*>(p), f);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = i < n ? bf2f(p[i]) : 0.f;
  }
}

JLA_DEV float hy_silu(float x) { return x / (1.f + expf(-x)); }
JLA_DEV float hy_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
JLA_DEV float hy_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

}  // namespace jla
