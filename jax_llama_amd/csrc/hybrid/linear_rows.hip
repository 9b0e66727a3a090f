// Row-gathered, expert-grouped linear on row-major weights of any shape (no N % 16 / K % 32 packing constraint):
//   out[dst(r), :] = act(A[src(r), :] @ W[expert(r)]^T)
// A is fp32 in memory. With bf16 weights the A tile is rounded to bf16 while it is staged (v_mfma_f32_32x32x16_bf16,
// fp32 accumulation); with fp32 weights everything stays fp32 on the exact-f32 MFMA (v_mfma_f32_32x32x2_f32).
//
//  * tiles: 64 x 64 or (with rows to fill them) 128 x 64 outputs per 256-thread workgroup, four waves of 32 x 32 /
//    64 x 32, K staged 32 deep through LDS (several workgroups per CU hide each other's staging; a 128 x 128 tile with
//    register prefetch and a 64-deep K stage measured slower). The activations may be a bf16 copy and the output bf16
//    (the expert pair of a prompt: x -> bf16 once, hidden kept bf16), which halves the activation traffic. With an
//    expert offset table the m-tiles of the launch are dealt to the experts in order (a workgroup finds its expert by
//    walking the table; surplus workgroups exit), so one launch covers every expert of a token-sorted batch.
//  * few rows (decode): a wave streams one or four weight rows once and dots them with up to 8 activation rows.
//  * swiglu epilogue: the gate and the up rows of a column are accumulated side by side, out = silu(g) * u.
// The table router's counting sort is here too.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

using f32x16 = __attribute__((ext_vector_type(16))) float;

constexpr int LR_BM = 64, LR_BN = 64, LR_BK = 32, LR_THREADS = 256;

template <typename WT>
struct LrTile;
template <>
struct LrTile<bf16_t> {
  static constexpr int LD = LR_BK + 8;  // 80-byte rows: 16-byte aligned fragment reads, rows spread over the banks
};
template <>
struct LrTile<float> {
  static constexpr int LD = LR_BK + 1;
};

JLA_DEV void lr_store8(bf16_t* dst, const float* f) { *reinterpret_cast<u32x4*>(dst) = pack8(f); }
JLA_DEV void lr_store8(float* dst, const float* f) {
#pragma unroll
  for (int i = 0; i < 8; ++i) dst[i] = f[i];
}

JLA_DEV void lr_mma(const bf16_t* a_row, const bf16_t* b_row, int hi, f32x16& acc) {
#pragma unroll
  for (int kk = 0; kk < LR_BK / 16; ++kk) {
    const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(a_row + 16 * kk + 8 * hi);
    const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(b_row + 16 * kk + 8 * hi);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
  }
}
JLA_DEV void lr_mma(const float* a_row, const float* b_row, int hi, f32x16& acc) {
#pragma unroll
  for (int kk = 0; kk < LR_BK / 2; ++kk)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_row[2 * kk + hi], b_row[2 * kk + hi], acc, 0, 0, 0);
}

// 8 consecutive k of a row into the LDS tile (zeros past `left`); a bf16 source going to a bf16 tile is copied as is
JLA_DEV void lr_stage8(const float* src, int left, bf16_t* dst) {
  float f[8];
  hy_load8(src, left, f);
  lr_store8(dst, f);
}
JLA_DEV void lr_stage8(const float* src, int left, float* dst) {
  float f[8];
  hy_load8(src, left, f);
  lr_store8(dst, f);
}
JLA_DEV void lr_stage8(const bf16_t* src, int left, bf16_t* dst) {
  if (left >= 8 && ((uintptr_t)src & 15) == 0) {
    *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
  } else {
    float f[8];
    hy_load8(src, left, f);
    lr_store8(dst, f);
  }
}
JLA_DEV void lr_stage8(const bf16_t* src, int left, float* dst) {
  float f[8];
  hy_load8(src, left, f);
  lr_store8(dst, f);
}
template <typename T>
JLA_DEV void lr_zero8(T* dst) {
  const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  lr_store8(dst, z);
}
JLA_DEV void lr_out(float* p, float v) { *p = v; }
JLA_DEV void lr_out(bf16_t* p, float v) { *p = f2bf(v); }

// WT: weight / tile type; AT: activation type in memory (fp32, or a bf16 copy); OT: output type; TMM: 32-row tiles per
// wave along M (workgroup tile 64 TMM x 64: the 128-row form halves the weight traffic per output row).
template <typename WT, int SWIGLU, typename AT, typename OT, int TMM>
__global__ void __launch_bounds__(LR_THREADS) lr_gemm_kernel(RowLinear p) {
  constexpr int LD = LrTile<WT>::LD;
  constexpr int BM = LR_BM * TMM;
  __shared__ __attribute__((aligned(16))) WT As[BM * LD];
  __shared__ __attribute__((aligned(16))) WT Bs[(SWIGLU ? 2 : 1) * LR_BN * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, hi = lane >> 5;
  // which expert and which rows
  int e = 0, r0 = blockIdx.y * BM, rend = p.R;
  if (p.offs) {
    int tile = blockIdx.y;
    bool found = false;
    for (e = 0; e < p.E; ++e) {
      const int b = p.offs[e], cnt = p.offs[e + 1] - b, nt = (cnt + BM - 1) / BM;
      if (tile < nt) {
        r0 = b + tile * BM;
        rend = b + cnt;
        found = true;
        break;
      }
      tile -= nt;
    }
    if (!found) return;
  } else if (r0 >= rend) {
    return;
  }
  const int n0 = blockIdx.x * LR_BN;
  const WT* W = reinterpret_cast<const WT*>(p.w) + (size_t)e * p.w_stride;
  const int K = p.K, N = p.N;

  // staging role: 8 consecutive k of row (tid >> 2) (+ 64 for the second half of a 128-row tile)
  const int srow = tid >> 2, skq = (tid & 3) * 8;
  const AT* a_ptr[TMM];
#pragma unroll
  for (int t = 0; t < TMM; ++t) {
    const int ar = r0 + srow + 64 * t;
    a_ptr[t] = ar < rend ? reinterpret_cast<const AT*>(p.a) + (size_t)(p.a_idx ? p.a_idx[ar] : ar) * p.lda : nullptr;
  }
  const int wr = n0 + srow;
  const WT* w_ptr = wr < N ? W + (size_t)wr * K : nullptr;
  const WT* w2_ptr = (SWIGLU && wr < N) ? W + (size_t)(N + wr) * K : nullptr;

  f32x16 acc[TMM], acc2[TMM];
#pragma unroll
  for (int t = 0; t < TMM; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = acc2[t][r] = 0.f;

  for (int k0 = 0; k0 < K; k0 += LR_BK) {
    const int gk = k0 + skq, left = K - gk;
#pragma unroll
    for (int t = 0; t < TMM; ++t) {
      if (a_ptr[t] && left > 0) lr_stage8(a_ptr[t] + gk, left, &As[(srow + 64 * t) * LD + skq]);
      else lr_zero8(&As[(srow + 64 * t) * LD + skq]);
    }
    if (w_ptr && left > 0) lr_stage8(w_ptr + gk, left, &Bs[srow * LD + skq]);
    else lr_zero8(&Bs[srow * LD + skq]);
    if (SWIGLU) {
      if (w2_ptr && left > 0) lr_stage8(w2_ptr + gk, left, &Bs[(LR_BN + srow) * LD + skq]);
      else lr_zero8(&Bs[(LR_BN + srow) * LD + skq]);
    }
    __syncthreads();
    const WT* b_row = &Bs[(wn * 32 + (lane & 31)) * LD];
#pragma unroll
    for (int t = 0; t < TMM; ++t) {
      const WT* a_row = &As[(wm * 32 * TMM + 32 * t + (lane & 31)) * LD];
      lr_mma(a_row, b_row, hi, acc[t]);
      if (SWIGLU) lr_mma(a_row, b_row + LR_BN * LD, hi, acc2[t]);
    }
    __syncthreads();
  }
  // C/D map of the 32 x 32 shapes: col = lane & 31, row = (r & 3) + 8 (r >> 2) + 4 (lane >> 5)
  const int col = n0 + wn * 32 + (lane & 31);
  if (col >= N) return;
  OT* out = reinterpret_cast<OT*>(p.out);
#pragma unroll
  for (int t = 0; t < TMM; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = r0 + wm * 32 * TMM + 32 * t + (r & 3) + 8 * (r >> 2) + 4 * hi;
      if (row < rend) {
        const int drow = p.dst_idx ? p.dst_idx[row] : row;
        lr_out(out + (size_t)drow * p.ldo + col, SWIGLU ? hy_silu(acc[t][r]) * acc2[t][r] : acc[t][r]);
      }
    }
}

JLA_DEV float lr_round(float v, const bf16_t*) { return bf2f(f2bf(v)); }
JLA_DEV float lr_round(float v, const float*) { return v; }

// A wave owns LR_CPW consecutive output columns (4 for wide outputs such as a vocabulary head, 1 where that would
// leave too few workgroups): their weight rows are streamed once (16-byte loads, LR_CPW rows in flight per lane) and
// dotted with the rows of group blockIdx.y: a fixed count of rows, one row with its own expert (row_expert), or every
// row of one expert of an expert-sorted batch (offs).
template <typename WT, int SWIGLU, int LR_CPW>
__global__ void __launch_bounds__(LR_THREADS) lr_gemv_kernel(RowLinear p, int rows_per_group) {
  constexpr int MAXR = HY_GEMV_MAX_R;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * (LR_THREADS / 64) + wave) * LR_CPW;
  if (n0 >= p.N) return;
  // rows of this group: a fixed count, one row with its own expert, or (offs) every row of expert blockIdx.y
  int g0 = blockIdx.y * rows_per_group, g1 = min(g0 + rows_per_group, p.R), e = 0;
  if (p.offs) {
    e = blockIdx.y;
    g0 = p.offs[e];
    g1 = p.offs[e + 1];
  } else if (p.row_expert) {
    e = p.row_expert[g0];
  }
  const int K = p.K;
  for (int r0 = g0; r0 < g1; r0 += MAXR) {  // (more than MAXR rows: the weights are streamed again per 8 rows)
  const int nr = min(MAXR, g1 - r0);
  const WT* wbase = reinterpret_cast<const WT*>(p.w) + (size_t)e * p.w_stride;
  const WT* w[LR_CPW];
#pragma unroll
  for (int c = 0; c < LR_CPW; ++c) w[c] = wbase + (size_t)min(n0 + c, p.N - 1) * K;  // (surplus columns re-read the last)
  const size_t up = (size_t)p.N * K;
  const float* a[MAXR];
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    const int rr = r0 + min(r, nr - 1);
    a[r] = reinterpret_cast<const float*>(p.a) + (size_t)(p.a_idx ? p.a_idx[rr] : rr) * p.lda;
  }
  float acc[MAXR][LR_CPW], acc2[MAXR][LR_CPW];
#pragma unroll
  for (int r = 0; r < MAXR; ++r)
#pragma unroll
    for (int c = 0; c < LR_CPW; ++c) acc[r][c] = acc2[r][c] = 0.f;
#pragma unroll 4
  for (int k = lane * 8; k < K; k += 64 * 8) {
    const int left = K - k;
    float wf[LR_CPW][8], uf[LR_CPW][8];
#pragma unroll
    for (int c = 0; c < LR_CPW; ++c) {
      hy_load8(w[c] + k, left, wf[c]);
      if (SWIGLU) hy_load8(w[c] + up + k, left, uf[c]);
    }
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      if (r < nr) {
        float xf[8];
        hy_load8(a[r] + k, left, xf);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float xv = lr_round(xf[i], wbase);
#pragma unroll
          for (int c = 0; c < LR_CPW; ++c) {
            acc[r][c] = fmaf(xv, wf[c][i], acc[r][c]);
            if (SWIGLU) acc2[r][c] = fmaf(xv, uf[c][i], acc2[r][c]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < nr) {  // (wave-uniform)
      const int row = r0 + r, drow = p.dst_idx ? p.dst_idx[row] : row;
#pragma unroll
      for (int c = 0; c < LR_CPW; ++c) {
        const float g = wave_sum(acc[r][c]);
        const float u = SWIGLU ? wave_sum(acc2[r][c]) : 0.f;
        if (lane == 0 && n0 + c < p.N)
          reinterpret_cast<float*>(p.out)[(size_t)drow * p.ldo + n0 + c] = SWIGLU ? hy_silu(g) * u : g;
      }
    }
  }
  }
}

// rows at or below which an expert-sorted batch runs the expert-grouped GEMV (each expert's weights streamed once)
constexpr int HY_GROUPED_GEMV_MAX_R = 64;

int hy_linear_rows(const RowLinear& p, hipStream_t s) {
  if (p.R < 0 || p.N <= 0 || p.K <= 0 || p.lda < p.K || p.ldo < p.N || p.E < 1) return -1;
  if (p.R == 0) return 0;
  if (p.offs && p.E > 65535) return -2;
  const bool grouped = p.offs && p.R <= HY_GROUPED_GEMV_MAX_R;
  const bool small = grouped || (p.R <= HY_GEMV_MAX_R && (!p.offs || p.row_expert));
  if (small) {
    if (p.a_bf16 || p.out_bf16) return -7;  // (the GEMV reads and writes fp32)
    const int rpg = p.row_expert && !grouped ? 1 : HY_GEMV_MAX_R;
    const int cpw = p.N >= 8192 ? 4 : 1;
    dim3 grid((p.N + 4 * cpw - 1) / (4 * cpw), grouped ? p.E : (p.R + rpg - 1) / rpg);
    RowLinear q = p;
    if (!grouped) q.offs = nullptr;
#define LR_GEMV(WT, SW)                                                              \
  do {                                                                               \
    if (cpw == 4) lr_gemv_kernel<WT, SW, 4><<<grid, LR_THREADS, 0, s>>>(q, rpg);     \
    else lr_gemv_kernel<WT, SW, 1><<<grid, LR_THREADS, 0, s>>>(q, rpg);              \
  } while (0)
    if (p.wbf16) {
      if (p.swiglu) LR_GEMV(bf16_t, 1);
      else LR_GEMV(bf16_t, 0);
    } else {
      if (p.swiglu) LR_GEMV(float, 1);
      else LR_GEMV(float, 0);
    }
#undef LR_GEMV
    JLA_CHECK_LAUNCH();
    return 0;
  }
  if (!p.offs && p.E != 1) return -3;
  if ((p.a_bf16 || p.out_bf16) && !p.wbf16) return -5;
  // 128-row tiles once every expert (or the whole batch) has rows to fill them; the SwiGLU form (two accumulator sets)
  // only with many such tiles per expert (measured: 512 rows per expert run faster on 64-row tiles, 4096 on 128-row)
  const long long per_e = p.R / (p.offs ? p.E : 1);
  const int tmm = per_e >= (p.swiglu ? 1024 : (p.offs ? 128 : 256)) ? 2 : 1;
  const int bm = LR_BM * tmm;
  const long long mt = (p.R + bm - 1) / bm + (p.offs ? p.E : 0);
  if (mt > 65535) return -4;
  dim3 grid((p.N + LR_BN - 1) / LR_BN, (unsigned)mt);
  RowLinear q = p;
  q.row_expert = nullptr;
#define LR_GEMM(WT, SW, AT, OT)                                                           \
  do {                                                                                    \
    if (tmm == 2) lr_gemm_kernel<WT, SW, AT, OT, 2><<<grid, LR_THREADS, 0, s>>>(q);       \
    else lr_gemm_kernel<WT, SW, AT, OT, 1><<<grid, LR_THREADS, 0, s>>>(q);                \
  } while (0)
  if (p.wbf16) {
    if (p.a_bf16 && p.out_bf16 && p.swiglu) LR_GEMM(bf16_t, 1, bf16_t, bf16_t);
    else if (p.a_bf16 && !p.out_bf16 && !p.swiglu) LR_GEMM(bf16_t, 0, bf16_t, float);
    else if (p.a_bf16 || p.out_bf16) return -6;  // (combinations nothing uses)
    else if (p.swiglu) LR_GEMM(bf16_t, 1, float, float);
    else LR_GEMM(bf16_t, 0, float, float);
  } else {
    if (p.swiglu) LR_GEMM(float, 1, float, float);
    else LR_GEMM(float, 0, float, float);
  }
#undef LR_GEMM
  JLA_CHECK_LAUNCH();
  return 0;
}

// ---- table router: counting sort of the (token, choice) rows by expert (one workgroup) -------------------------------
constexpr int RT_MAX_E = 1024;

__global__ void __launch_bounds__(256) route_table_kernel(const int32_t* ids, const int32_t* table, int V, int M, int top,
                                                          int E, int32_t* row_expert, int32_t* row_tok,
                                                          int32_t* sort_tok, int32_t* sort_dst, int32_t* offs) {
  __shared__ int cnt[RT_MAX_E + 1];
  __shared__ int cur[RT_MAX_E];
  const int R = M * top;
  for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += blockDim.x) {
    const int m = r / top, c = r - m * top;
    int id = ids[m];
    id = id < 0 || id >= V ? 0 : id;
    int e = table[(size_t)id * top + c];
    e = e < 0 || e >= E ? 0 : e;
    row_expert[r] = e;
    row_tok[r] = m;
    atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cnt[e];
      cur[e] = run;
      offs[e] = run;
      run += c;
    }
    offs[E] = run;
  }
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += blockDim.x) {
    const int e = row_expert[r];
    const int pos = atomicAdd(&cur[e], 1);
    sort_tok[pos] = r / top;
    sort_dst[pos] = r;
  }
}

int hy_route_table(const int32_t* ids, const int32_t* table, int V, int M, int top, int E, int32_t* row_expert,
                   int32_t* row_tok, int32_t* sort_tok, int32_t* sort_dst, int32_t* offs, hipStream_t s) {
  if (M < 0 || top < 1 || E < 1 || E > RT_MAX_E || V < 1) return -1;
  if (M == 0) return 0;
  route_table_kernel<<<1, 256, 0, s>>>(ids, table, V, M, top, E, row_expert, row_tok, sort_tok, sort_dst, offs);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
