// Gated delta rule (a linear-attention recurrence with a per-head decay and a delta-rule write), fp32 throughout.
//
// Per head, with state S [dim, vdim] (key rows, value columns), decay g, write strength beta:
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q        (the read-out sees this token's write)
//
//   hy_delta_prep        : from the fused projection output, per (token, head): the short causal convolution over
//                          time of the q / k / v channels (taps weights per channel, the last tap on the current token;
//                          inputs before this call come from the carried tail, zeros at a sequence start), SiLU, then
//                          q and k scaled to unit length (q also by dim^-1/2); beta = sigmoid(.), and the decay
//                          g = exp(-exp(A_log) softplus(a + dt_bias)).
//   hy_conv_state_update : the carried tail <- the last taps - 1 inputs of every channel (after hy_delta_prep).
//   hy_delta_scan        : the recurrence, token by token. A thread owns 32 key rows of one value column in registers;
//                          the lanes sharing a column (dim / 32 of them, adjacent) combine their partial S^T k and
//                          S^T q by lane exchange. k, q, v, g, beta of a token are wave-uniform or per-column loads.
//   hy_gated_rmsnorm     : o / rms(o) * w * silu(gate) per head.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

// conv input of channel c at sequence offset t (t < 0: the carried tail)
JLA_DEV float dp_input(const DeltaPrep& p, int b, int t, int c, int col) {
  if (t >= 0) return p.proj[((size_t)b * p.S + t) * p.ld + col];
  const int C = 2 * p.G * p.dim + p.H * p.vdim;
  return p.conv_state[((size_t)b * C + c) * (p.taps - 1) + (p.taps - 1 + t)];
}

// grid (M, ceil((2G + H + 1) / 4)), 4 waves; item: [0, G) q heads, [G, 2G) k heads, [2G, 2G + H) v heads, then the gates
__global__ void __launch_bounds__(256) delta_prep_kernel(DeltaPrep p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.x, item = blockIdx.y * 4 + wave;
  const int items = 2 * p.G + p.H + 1;
  if (item >= items) return;
  const int b = m / p.S, t = m - b * p.S;
  const int QK = p.G * p.dim, VV = p.H * p.vdim;
  if (item == items - 1) {  // gates: beta, decay
    const float* row = p.proj + (size_t)m * p.ld + 2 * QK + 2 * VV;
    for (int h = lane; h < p.H; h += 64) {
      p.beta[(size_t)m * p.H + h] = hy_sigmoid(row[h]);
      p.decay[(size_t)m * p.H + h] = expf(-expf(p.a_log[h]) * hy_softplus(row[p.H + h] + p.dt_bias[h]));
    }
    return;
  }
  int kind, head, len, c0;  // c0: first channel (= projection column) of the head
  if (item < p.G) { kind = 0; head = item; len = p.dim; c0 = head * p.dim; }
  else if (item < 2 * p.G) { kind = 1; head = item - p.G; len = p.dim; c0 = QK + head * p.dim; }
  else { kind = 2; head = item - 2 * p.G; len = p.vdim; c0 = 2 * QK + head * p.vdim; }
  float* dst = kind == 0 ? p.qn + ((size_t)m * p.G + head) * p.dim
             : kind == 1 ? p.kn + ((size_t)m * p.G + head) * p.dim
                         : p.vc + ((size_t)m * p.H + head) * p.vdim;
  float ss = 0.f;
  for (int d = lane; d < len; d += 64) {
    const int c = c0 + d;
    float y = 0.f;
    for (int tap = 0; tap < p.taps; ++tap)
      y = fmaf(p.conv_w[(size_t)c * p.taps + tap], dp_input(p, b, t - (p.taps - 1) + tap, c, c), y);
    y = hy_silu(y);
    dst[d] = y;
    ss = fmaf(y, y, ss);
  }
  if (kind == 2) return;
  ss = wave_sum(ss);
  float sc = 1.f / sqrtf(ss + 1e-6f);
  if (kind == 0) sc *= 1.f / sqrtf((float)p.dim);
  for (int d = lane; d < len; d += 64) dst[d] *= sc;  // (each lane rescales what it wrote)
}

// one thread per (row, channel): tail <- last taps - 1 of [tail, this call's inputs]
__global__ void __launch_bounds__(256) conv_state_update_kernel(DeltaPrep p) {
  const int C = 2 * p.G * p.dim + p.H * p.vdim;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.B * C) return;
  const int b = idx / C, c = idx - b * C;
  const int n = p.taps - 1;
  float* st = p.conv_state + (size_t)idx * n;
  // new[i] = input at sequence offset S - n + i
  if (p.S >= n) {
    for (int i = 0; i < n; ++i) st[i] = p.proj[((size_t)b * p.S + (p.S - n + i)) * p.ld + c];
  } else {
    for (int i = 0; i < n - p.S; ++i) st[i] = st[i + p.S];  // ascending: reads run ahead of writes
    for (int i = n - p.S; i < n; ++i) st[i] = p.proj[((size_t)b * p.S + (p.S - n + i)) * p.ld + c];
  }
}

static int dp_check(const DeltaPrep& p) {
  if (p.B < 0 || p.S < 1 || p.H < 1 || p.G < 1 || p.H % p.G || p.dim < 1 || p.vdim < 1 || p.taps < 1) return -1;
  if (p.ld < 2 * p.G * p.dim + 2 * p.H * p.vdim + 2 * p.H) return -2;
  return 0;
}

int hy_delta_prep(const DeltaPrep& p, hipStream_t s) {
  if (int r = dp_check(p)) return r;
  const int M = p.B * p.S;
  if (M == 0) return 0;
  const int items = 2 * p.G + p.H + 1;
  if ((items + 3) / 4 > 65535) return -3;
  delta_prep_kernel<<<dim3(M, (items + 3) / 4), 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

int hy_conv_state_update(const DeltaPrep& p, hipStream_t s) {
  if (int r = dp_check(p)) return r;
  if (p.B == 0 || p.taps == 1) return 0;
  const long long n = (long long)p.B * (2 * p.G * p.dim + p.H * p.vdim);
  conv_state_update_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

constexpr int DS_SLICE = 32;  // key rows per thread

// grid (ceil(vdim * R / 256), H, B); thread -> (column j = t / R, slice r = t % R), R = lanes per column (power of 2)
__global__ void __launch_bounds__(256) delta_scan_kernel(DeltaScan p, int R) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int j = t / R, r = t - j * R;
  const bool live = j < p.vdim;  // (dead threads still join the lane exchanges)
  const int jc = live ? j : 0;
  const int kh = h / (p.H / p.G);
  const int i0 = r * DS_SLICE;
  float S[DS_SLICE];
  float* sp = p.state + (((size_t)b * p.H + h) * p.dim) * p.vdim + jc;
#pragma unroll
  for (int i = 0; i < DS_SLICE; ++i) S[i] = (live && i0 + i < p.dim) ? sp[(size_t)(i0 + i) * p.vdim] : 0.f;
  for (int s = 0; s < p.S; ++s) {
    const size_t m = (size_t)b * p.S + s;
    const float* k = p.kn + (m * p.G + kh) * p.dim + i0;
    const float* q = p.qn + (m * p.G + kh) * p.dim + i0;
    const float g = p.decay[m * p.H + h], beta = p.beta[m * p.H + h];
    const float v = p.v[(m * p.H + h) * p.vdim + jc];
    float kv[DS_SLICE], sk = 0.f;
#pragma unroll
    for (int i = 0; i < DS_SLICE; ++i) {
      kv[i] = i0 + i < p.dim ? k[i] : 0.f;
      S[i] *= g;
      sk = fmaf(S[i], kv[i], sk);
    }
    for (int o = 1; o < R; o <<= 1) sk += __shfl_xor(sk, o, 64);
    const float u = beta * (v - sk);
    float oq = 0.f;
#pragma unroll
    for (int i = 0; i < DS_SLICE; ++i) {
      S[i] = fmaf(kv[i], u, S[i]);
      oq = fmaf(S[i], i0 + i < p.dim ? q[i] : 0.f, oq);
    }
    for (int o = 1; o < R; o <<= 1) oq += __shfl_xor(oq, o, 64);
    if (live && r == 0) p.o[(m * p.H + h) * p.vdim + j] = oq;
  }
#pragma unroll
  for (int i = 0; i < DS_SLICE; ++i)
    if (live && i0 + i < p.dim) sp[(size_t)(i0 + i) * p.vdim] = S[i];
}

int hy_delta_scan(const DeltaScan& p, hipStream_t s) {
  if (p.B < 0 || p.S < 1 || p.H < 1 || p.G < 1 || p.H % p.G || p.dim < 1 || p.vdim < 1) return -1;
  if (p.dim > 64 * DS_SLICE) return -2;
  if (p.B == 0) return 0;
  if (p.H > 65535 || p.B > 65535) return -3;
  int R = 1;
  while (R * DS_SLICE < p.dim) R <<= 1;
  const long long threads = (long long)p.vdim * R;
  delta_scan_kernel<<<dim3((unsigned)((threads + 255) / 256), p.H, p.B), 256, 0, s>>>(p, R);
  JLA_CHECK_LAUNCH();
  return 0;
}

// grid (M, ceil(H / 4)), one wave per (token, head)
__global__ void __launch_bounds__(256) gated_rmsnorm_kernel(const float* o, const float* gate, int ldg, const float* w,
                                                            float eps, float* out, int M, int H, int vdim) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.x, h = blockIdx.y * 4 + wave;
  if (h >= H) return;
  const float* x = o + ((size_t)m * H + h) * vdim;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += 64) ss = fmaf(x[d], x[d], ss);
  ss = wave_sum(ss);
  const float sc = 1.f / sqrtf(ss / (float)vdim + eps);
  const float* gr = gate + (size_t)m * ldg + (size_t)h * vdim;
  float* dst = out + ((size_t)m * H + h) * vdim;
  for (int d = lane; d < vdim; d += 64) dst[d] = x[d] * sc * w[d] * hy_silu(gr[d]);
}

int hy_gated_rmsnorm(const float* o, const float* gate, int ldg, const float* w, float eps, float* out, int M, int H,
                     int vdim, hipStream_t s) {
  if (M < 0 || H < 1 || vdim < 1 || ldg < H * vdim) return -1;
  if (M == 0) return 0;
  if ((H + 3) / 4 > 65535) return -2;
  gated_rmsnorm_kernel<<<dim3(M, (H + 3) / 4), 256, 0, s>>>(o, gate, ldg, w, eps, out, M, H, vdim);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
