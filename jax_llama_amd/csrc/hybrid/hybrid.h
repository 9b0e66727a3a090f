// Host launchers of the hybrid-sequence-mixer kernels (module jax_llama_amd._C_hybrid): row-gathered / expert-grouped
// linears on row-major weights of any shape, attention with a distance-bias table and a score soft cap, the gated
// delta rule with its short convolutions, and the output-side norms. Pure HIP translation units (no torch headers).
// Every launcher returns 0 on success, <0 on a shape/argument error, >0 for a hipError_t.
//
// Activations between kernels are fp32 in both number formats. "wbf16" selects the weight / cache element type: bf16
// (matrix operands rounded to bf16, fp32 accumulation) or fp32 (exact-f32 MFMA, fp32 caches).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace jla {

// out[M, D] (fp32) = table[ids[m], col0 : col0 + D]; table rows are `ld` elements apart. Ids outside [0, V) read row 0.
int hy_embed_rows(const int32_t* ids, const void* table, int wbf16, int V, int ld, int col0, float* out, int M, int D,
                  hipStream_t s);

struct RowLinear {
  const void* a;         // [*, lda] activations: fp32, or (a_bf16, tile path with bf16 weights only) bf16
  int a_bf16;
  int lda;
  const int32_t* a_idx;  // optional: activation row of linear row r (else r)
  const void* w;         // [E][Nw][K] row-major; Nw = N (store) or 2N (swiglu: gate rows [0, N), up rows [N, 2N))
  long long w_stride;    // elements between experts
  int wbf16;
  int N, K;
  void* out;             // [*, ldo] fp32, or (out_bf16, tile path with bf16 weights only) bf16
  int out_bf16;
  int ldo;
  const int32_t* dst_idx;     // optional: output row of linear row r (else r)
  const int32_t* offs;        // optional [E + 1]: rows [offs[e], offs[e + 1]) use expert e (rows sorted by expert)
  const int32_t* row_expert;  // optional [R]: expert of each row (the small-R path)
  int E;
  int R;                 // linear rows
  int swiglu;            // 0: out = a W^T; 1: out = silu(a Wg^T) * (a Wu^T)
};
// R <= HY_GEMV_MAX_R and (offs == nullptr or row_expert != nullptr): one wave per output column (weights streamed once
// per row group); else the 64 x 64 MFMA tiles (offs: expert-grouped).
constexpr int HY_GEMV_MAX_R = 8;
int hy_linear_rows(const RowLinear& p, hipStream_t s);

// Table routing: expert of (token m, choice c) = table[ids[m], c]. Writes row_expert[R] and row_tok[R] in (m, c) order
// (R = M * top), and the expert-sorted order: sort_tok[p] (token of sorted row p), sort_dst[p] (its (m, c) row),
// offs[E + 1]. One workgroup; E <= 1024.
int hy_route_table(const int32_t* ids, const int32_t* table, int V, int M, int top, int E, int32_t* row_expert,
                   int32_t* row_tok, int32_t* sort_tok, int32_t* sort_dst, int32_t* offs, hipStream_t s);

// x[m, :] += (sum_{c < nsum} y[m * nsum + c, :]) * ysc / sqrt(mean(.^2) + eps) * w   (w: one number, or D numbers).
// x == nullptr: out-of-place into `out` without the add (a plain RMS norm).
int hy_norm_residual(const float* y, int nsum, float ysc, const float* w, int w_vec, float eps, float* x, float* out,
                     int M, int D, hipStream_t s);

// y (bf16) = x (fp32), n a multiple of 8
typedef uint16_t bf16_t;
int hy_cast_bf16(const float* x, bf16_t* y, long long n, hipStream_t s);

// g[m, c] = gelu_tanh(gp[m, c]) * table[ids[m], col0 + c]
int hy_gelu_gate_rows(const float* gp, const int32_t* ids, const void* table, int wbf16, int V, int ld, int col0,
                      float* g, int M, int D, hipStream_t s);

struct AttnPrep {
  const float* proj;  // [M, ld]: q heads at column 0, then (if has_kv) k heads, then v heads
  int ld;
  const int32_t* positions;  // [M]
  const int32_t* slot;       // device int32[1]: cache slot of this call's first token
  int B, S, H, G, dim, vdim, T;
  int has_kv;
  void* kc;  // [B, G, T, dim]
  void* vc;  // [B, G, T, vdim]
  int cbf16;
  float* q;  // [M, H, dim]
  float eps;
  float temp_coef;  // 0: no query temperature
  int temp_every;
};
// Per head: q, k divided by their RMS over dim (v over vdim); q times 1 + coef * ln(floor((p + 1) / every) + 1);
// k, v written to the cache at slot + s.
int hy_attn_prep(const AttnPrep& p, hipStream_t s);

struct AttnBias {
  const float* q;  // [B, S, H, dim]
  const void* kc;
  const void* vc;
  int cbf16;
  const int32_t* slot;
  int B, S, H, G, dim, vdim, T;
  float scale, softcap;  // softcap <= 0: none
  const float* bias;     // optional [nbias, H]: added to the score of distance n at row min(n, nbias - 1)
  int nbias;
  float* out;  // [B * S, H * vdim]
  int t_cap;   // keys the launch may have to cover (decode split sizing); <= T
  float* ws;   // decode split partials: B * H * splits * (vdim + 2) floats
  int splits;
  void* vt_ws;  // prefill: hy_attn_prefill_ws_bytes(...) bytes for the transposed values (nullptr: the plain kernel)
};
int hy_attn_bias(const AttnBias& p, hipStream_t s);
long long hy_attn_prefill_ws_bytes(int B, int S, int G, int dim, int vdim, int T, int cbf16);
int hy_attn_decode_splits(int B, int H, int t_cap);

struct DeltaPrep {
  const float* proj;  // [M, ld]: q (G * dim), k (G * dim), v (H * vdim), gate (H * vdim), b (H), a (H)
  int ld;
  int B, S, H, G, dim, vdim, taps;
  const float* conv_w;  // [2 G dim + H vdim, taps] fp32, channel order q, k, v
  float* conv_state;    // [B, C, taps - 1]: the last inputs of every channel, oldest first
  const float* a_log;   // [H]
  const float* dt_bias; // [H]
  float* qn;  // [M, G, dim]   unit vectors times dim^-1/2
  float* kn;  // [M, G, dim]   unit vectors
  float* vc;  // [M, H, vdim]
  float* beta;   // [M, H]
  float* decay;  // [M, H]
};
int hy_delta_prep(const DeltaPrep& p, hipStream_t s);
int hy_conv_state_update(const DeltaPrep& p, hipStream_t s);

struct DeltaScan {
  const float* qn;
  const float* kn;
  const float* v;
  const float* beta;
  const float* decay;
  float* state;  // [B, H, dim, vdim] fp32, read and written
  float* o;      // [M, H, vdim]
  int B, S, H, G, dim, vdim;
};
int hy_delta_scan(const DeltaScan& p, hipStream_t s);

// out[m, h * vdim + j] = o[m, h, j] / sqrt(mean_j(o^2) + eps) * w[j] * silu(gate[m * ldg + h * vdim + j])
int hy_gated_rmsnorm(const float* o, const float* gate, int ldg, const float* w, float eps, float* out, int M, int H,
                     int vdim, hipStream_t s);

}  // namespace jla
