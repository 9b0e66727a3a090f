// Row kernels of the hybrid stack: embedding-slice gather, the norm on a sublayer's OUTPUT fused with the residual add
// (x += rms_norm(sum of the chosen experts' outputs) * w, w one number or a vector), and the per-layer token-side gate
// (gelu_tanh(gate projection) * a slice of a second embedding table). fp32 statistics and residual.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

JLA_DEV float ns_ld(const float* p) { return *p; }
JLA_DEV float ns_ld(const bf16_t* p) { return bf2f(*p); }

template <typename WT>
__global__ void __launch_bounds__(256) embed_rows_kernel(const int32_t* ids, const WT* table, int V, int ld, int col0,
                                                         float* out, int D) {
  const int m = blockIdx.x;
  int id = ids[m];
  id = id < 0 || id >= V ? 0 : id;
  const WT* row = table + (size_t)id * ld + col0;
  for (int d = threadIdx.x; d < D; d += 256) out[(size_t)m * D + d] = ns_ld(row + d);
}

int hy_embed_rows(const int32_t* ids, const void* table, int wbf16, int V, int ld, int col0, float* out, int M, int D,
                  hipStream_t s) {
  if (M < 0 || D < 1 || V < 1 || col0 < 0 || col0 + D > ld) return -1;
  if (M == 0) return 0;
  if (wbf16) embed_rows_kernel<bf16_t><<<M, 256, 0, s>>>(ids, reinterpret_cast<const bf16_t*>(table), V, ld, col0, out, D);
  else embed_rows_kernel<float><<<M, 256, 0, s>>>(ids, reinterpret_cast<const float*>(table), V, ld, col0, out, D);
  JLA_CHECK_LAUNCH();
  return 0;
}

// one workgroup per row; rows of up to 4096 columns are held in registers (y, x and the gain loaded in one round trip)
constexpr int NR_REGS = 16;

__global__ void __launch_bounds__(256) norm_residual_kernel(const float* y, int nsum, float ysc, const float* w,
                                                            int w_vec, float eps, float* x, float* out, int D) {
  __shared__ float red[16];
  const int m = blockIdx.x;
  const float* yr = y + (size_t)m * nsum * D;
  if (D <= 256 * NR_REGS) {
    float v[NR_REGS], xv[NR_REGS], wv[NR_REGS];
    const float w0 = w_vec ? 0.f : w[0];
#pragma unroll
    for (int u = 0; u < NR_REGS; ++u) {
      v[u] = xv[u] = wv[u] = 0.f;
      if (256 * u < D) {  // (uniform)
        const int d = min(threadIdx.x + 256 * u, D - 1);
        float a = 0.f;
        for (int c = 0; c < nsum; ++c) a += yr[(size_t)c * D + d];
        v[u] = a * ysc;
        xv[u] = x ? x[(size_t)m * D + d] : 0.f;
        wv[u] = w_vec ? w[d] : w0;
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NR_REGS; ++u)
      if (threadIdx.x + 256 * u < D) ss = fmaf(v[u], v[u], ss);
    ss = block_sum(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int u = 0; u < NR_REGS; ++u) {
      const int d = threadIdx.x + 256 * u;
      if (d < D) (x ? x : out)[(size_t)m * D + d] = xv[u] + v[u] * sc * wv[u];
    }
    return;
  }
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {
    float v = 0.f;
    for (int c = 0; c < nsum; ++c) v += yr[(size_t)c * D + d];
    v *= ysc;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float sc = 1.f / sqrtf(ss / (float)D + eps);
  const float w0 = w_vec ? 0.f : w[0];
  for (int d = threadIdx.x; d < D; d += 256) {
    float v = 0.f;
    for (int c = 0; c < nsum; ++c) v += yr[(size_t)c * D + d];
    v = v * ysc * sc * (w_vec ? w[d] : w0);
    if (x) x[(size_t)m * D + d] += v;
    else out[(size_t)m * D + d] = v;
  }
}

int hy_norm_residual(const float* y, int nsum, float ysc, const float* w, int w_vec, float eps, float* x, float* out,
                     int M, int D, hipStream_t s) {
  if (M < 0 || D < 1 || nsum < 1 || (!x && !out)) return -1;
  if (M == 0) return 0;
  norm_residual_kernel<<<M, 256, 0, s>>>(y, nsum, ysc, w, w_vec, eps, x, out, D);
  JLA_CHECK_LAUNCH();
  return 0;
}

// bf16 copy of an fp32 activation (the A operand of the packed MFMA GEMMs), 8 elements per thread
__global__ void __launch_bounds__(256) cast_bf16_kernel(const float* __restrict__ x, bf16_t* __restrict__ y, long long n8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  float f[8];
  hy_load8(x + 8 * i, 8, f);
  *reinterpret_cast<u32x4*>(y + 8 * i) = pack8(f);
}

int hy_cast_bf16(const float* x, bf16_t* y, long long n, hipStream_t s) {
  if (n < 0 || n % 8) return -1;
  if (n == 0) return 0;
  const long long n8 = n / 8;
  cast_bf16_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, s>>>(x, y, n8);
  JLA_CHECK_LAUNCH();
  return 0;
}

JLA_DEV float ns_gelu_tanh(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename WT>
__global__ void __launch_bounds__(256) gelu_gate_rows_kernel(const float* gp, const int32_t* ids, const WT* table, int V,
                                                             int ld, int col0, float* g, int D) {
  const int m = blockIdx.x;
  int id = ids[m];
  id = id < 0 || id >= V ? 0 : id;
  const WT* row = table + (size_t)id * ld + col0;
  for (int d = threadIdx.x; d < D; d += 256) g[(size_t)m * D + d] = ns_gelu_tanh(gp[(size_t)m * D + d]) * ns_ld(row + d);
}

int hy_gelu_gate_rows(const float* gp, const int32_t* ids, const void* table, int wbf16, int V, int ld, int col0,
                      float* g, int M, int D, hipStream_t s) {
  if (M < 0 || D < 1 || V < 1 || col0 < 0 || col0 + D > ld) return -1;
  if (M == 0) return 0;
  if (wbf16)
    gelu_gate_rows_kernel<bf16_t><<<M, 256, 0, s>>>(gp, ids, reinterpret_cast<const bf16_t*>(table), V, ld, col0, g, D);
  else
    gelu_gate_rows_kernel<float><<<M, 256, 0, s>>>(gp, ids, reinterpret_cast<const float*>(table), V, ld, col0, g, D);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
