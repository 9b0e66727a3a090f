// Python bindings of the hybrid-mixer kernels (module jax_llama_amd._C_hybrid). Thin: validate dtypes, shapes and
// contiguity on the host (a wrong shape must never reach a kernel), take raw pointers and launch on torch's current HIP
// stream, so hipGraph capture through torch.cuda.graph records these launches.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include "hybrid.h"

namespace {

using torch::Tensor;
using OptT = c10::optional<Tensor>;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

void check(bool cond, const char* msg) { TORCH_CHECK(cond, "jax_llama_amd._C_hybrid: ", msg); }

void rc(int r, const char* what) { TORCH_CHECK(r == 0, "jax_llama_amd._C_hybrid: ", what, " failed (code ", r, ")"); }

void gpu(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), "jax_llama_amd._C_hybrid: ", name, " must be a GPU tensor");
  TORCH_CHECK(t.is_contiguous(), "jax_llama_amd._C_hybrid: ", name, " must be contiguous");
}

const float* f32(const Tensor& t, const char* name) {
  gpu(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kFloat32, "jax_llama_amd._C_hybrid: ", name, " must be float32");
  return reinterpret_cast<const float*>(t.data_ptr());
}
float* f32w(const Tensor& t, const char* name) { return const_cast<float*>(f32(t, name)); }

const int32_t* i32(const Tensor& t, const char* name, int64_t min_numel) {
  gpu(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kInt32 && t.numel() >= min_numel, "jax_llama_amd._C_hybrid: ", name,
              " must be int32 with at least ", min_numel, " elements");
  return reinterpret_cast<const int32_t*>(t.data_ptr());
}
int32_t* i32w(const Tensor& t, const char* name, int64_t n) { return const_cast<int32_t*>(i32(t, name, n)); }

// weight / cache element type: 1 = bf16, 0 = fp32
int wtype(const Tensor& t, const char* name) {
  gpu(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16 || t.scalar_type() == torch::kFloat32, "jax_llama_amd._C_hybrid: ",
              name, " must be bfloat16 or float32");
  return t.scalar_type() == torch::kBFloat16;
}

// a 2-d fp32 or bf16 view with unit inner stride (rows may be strided); *bf = 1 for bf16
void* rows2d_any(const Tensor& t, const char* name, int64_t cols, int* ld, int* bf) {
  TORCH_CHECK(t.is_cuda() && (t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kBFloat16) &&
                  t.dim() == 2 && t.stride(1) == 1 && t.size(1) == cols && t.stride(0) >= cols,
              "jax_llama_amd._C_hybrid: ", name, " must be a float32 / bfloat16 [rows, ", cols,
              "] GPU view with unit inner stride");
  *ld = (int)t.stride(0);
  *bf = t.scalar_type() == torch::kBFloat16;
  return t.data_ptr();
}

// a 2-d fp32 view with unit inner stride (rows may be strided)
const float* rows2d(const Tensor& t, const char* name, int64_t cols, int* ld) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 && t.dim() == 2 && t.stride(1) == 1 &&
                  t.size(1) == cols && t.stride(0) >= cols,
              "jax_llama_amd._C_hybrid: ", name, " must be a float32 [rows, ", cols, "] GPU view with unit inner stride");
  *ld = (int)t.stride(0);
  return reinterpret_cast<const float*>(t.data_ptr());
}

void embed_rows(Tensor ids, Tensor table, int64_t col0, Tensor out) {
  const int wb = wtype(table, "table");
  check(table.dim() == 2 && out.dim() == 2, "embed_rows: 2-d table and out");
  const int M = out.size(0), D = out.size(1);
  rc(jla::hy_embed_rows(i32(ids, "ids", M), table.data_ptr(), wb, table.size(0), table.size(1), col0,
                        f32w(out, "out"), M, D, stream()),
     "embed_rows");
}

void linear_rows(Tensor a, OptT a_idx, Tensor w, Tensor out, OptT dst_idx, OptT offs, OptT row_expert, int64_t R,
                 bool swiglu) {
  jla::RowLinear p{};
  p.wbf16 = wtype(w, "w");
  check(w.dim() == 2 || w.dim() == 3, "linear_rows: w is [Nw, K] or [E, Nw, K]");
  p.E = w.dim() == 3 ? w.size(0) : 1;
  const int64_t Nw = w.size(-2);
  p.K = w.size(-1);
  check(!swiglu || Nw % 2 == 0, "linear_rows: swiglu needs gate and up rows");
  p.N = swiglu ? Nw / 2 : Nw;
  p.w = w.data_ptr();
  p.w_stride = Nw * (int64_t)p.K;
  p.a = rows2d_any(a, "a", p.K, &p.lda, &p.a_bf16);
  p.out = rows2d_any(out, "out", p.N, &p.ldo, &p.out_bf16);
  p.R = R;
  p.swiglu = swiglu;
  check(R >= 0, "linear_rows: R");
  if (a_idx.has_value()) p.a_idx = i32(*a_idx, "a_idx", R);
  else check(a.size(0) >= R, "linear_rows: a has fewer rows than R");
  if (dst_idx.has_value()) p.dst_idx = i32(*dst_idx, "dst_idx", R);
  else check(out.size(0) >= R, "linear_rows: out has fewer rows than R");
  if (offs.has_value()) p.offs = i32(*offs, "offs", p.E + 1);
  if (row_expert.has_value()) p.row_expert = i32(*row_expert, "row_expert", R);
  check(p.E == 1 || p.offs || p.row_expert, "linear_rows: stacked experts need offs or row_expert");
  rc(jla::hy_linear_rows(p, stream()), "linear_rows");
}

void route_table(Tensor ids, Tensor table, int64_t E, Tensor row_expert, Tensor row_tok, Tensor sort_tok, Tensor sort_dst,
                 Tensor offs) {
  check(table.dim() == 2, "route_table: table is [vocab, top]");
  const int M = ids.numel(), top = table.size(1);
  const int64_t R = (int64_t)M * top;
  rc(jla::hy_route_table(i32(ids, "ids", M), i32(table, "table", table.numel()), table.size(0), M, top, E,
                         i32w(row_expert, "row_expert", R), i32w(row_tok, "row_tok", R), i32w(sort_tok, "sort_tok", R),
                         i32w(sort_dst, "sort_dst", R), i32w(offs, "offs", E + 1), stream()),
     "route_table");
}

void norm_residual(Tensor y, int64_t nsum, double ysc, Tensor w, double eps, OptT x, OptT out) {
  check(y.dim() == 2 && nsum >= 1 && y.size(0) % nsum == 0, "norm_residual: y is [M * nsum, D]");
  const int M = y.size(0) / nsum, D = y.size(1);
  check(w.numel() == 1 || w.numel() == D, "norm_residual: w has 1 or D elements");
  float* xp = nullptr;
  float* op = nullptr;
  if (x.has_value()) {
    check(x->numel() == (int64_t)M * D, "norm_residual: x shape");
    xp = f32w(*x, "x");
  }
  if (out.has_value()) {
    check(out->numel() == (int64_t)M * D, "norm_residual: out shape");
    op = f32w(*out, "out");
  }
  check(xp || op, "norm_residual: x or out");
  rc(jla::hy_norm_residual(f32(y, "y"), nsum, (float)ysc, f32(w, "w"), w.numel() > 1 || D == 1, (float)eps, xp, op, M,
                           D, stream()),
     "norm_residual");
}

void cast_bf16(Tensor x, Tensor y) {
  gpu(y, "y");
  check(y.scalar_type() == torch::kBFloat16 && y.numel() == x.numel() && x.numel() % 8 == 0, "cast_bf16 shapes");
  rc(jla::hy_cast_bf16(f32(x, "x"), reinterpret_cast<jla::bf16_t*>(y.data_ptr()), x.numel(), stream()), "cast_bf16");
}

void gelu_gate_rows(Tensor gp, Tensor ids, Tensor table, int64_t col0, Tensor g) {
  const int wb = wtype(table, "table");
  check(gp.dim() == 2 && table.dim() == 2 && g.sizes() == gp.sizes(), "gelu_gate_rows shapes");
  const int M = gp.size(0), D = gp.size(1);
  rc(jla::hy_gelu_gate_rows(f32(gp, "gp"), i32(ids, "ids", M), table.data_ptr(), wb, table.size(0), table.size(1), col0,
                            f32w(g, "g"), M, D, stream()),
     "gelu_gate_rows");
}

void attn_prep(Tensor proj, Tensor positions, Tensor slot, int64_t B, int64_t S, int64_t H, int64_t G, int64_t dim,
               int64_t vdim, OptT kc, OptT vc, Tensor q, double eps, double temp_coef, int64_t temp_every) {
  jla::AttnPrep p{};
  p.has_kv = kc.has_value();
  check(kc.has_value() == vc.has_value(), "attn_prep: k and v caches together");
  const int64_t cols = H * dim + (p.has_kv ? G * (dim + vdim) : 0);
  check(proj.dim() == 2 && proj.size(0) == B * S, "attn_prep: proj rows");
  p.proj = rows2d(proj, "proj", cols, &p.ld);
  p.positions = i32(positions, "positions", B * S);
  p.slot = i32(slot, "slot", 1);
  p.B = B; p.S = S; p.H = H; p.G = G; p.dim = dim; p.vdim = vdim;
  p.T = 1;
  if (p.has_kv) {
    p.cbf16 = wtype(*kc, "k cache");
    check(wtype(*vc, "v cache") == p.cbf16, "attn_prep: cache dtypes differ");
    check(kc->dim() == 4 && kc->size(0) == B && kc->size(1) == G && kc->size(3) == dim, "attn_prep: k cache shape");
    p.T = kc->size(2);
    check(vc->dim() == 4 && vc->size(0) == B && vc->size(1) == G && vc->size(2) == p.T && vc->size(3) == vdim,
          "attn_prep: v cache shape");
    p.kc = kc->data_ptr();
    p.vc = vc->data_ptr();
  }
  check(q.numel() == B * S * H * dim, "attn_prep: q shape");
  p.q = f32w(q, "q");
  p.eps = eps;
  p.temp_coef = temp_coef;
  p.temp_every = temp_every;
  rc(jla::hy_attn_prep(p, stream()), "attn_prep");
}

int64_t attn_decode_splits(int64_t B, int64_t H, int64_t t_cap) { return jla::hy_attn_decode_splits(B, H, t_cap); }

int64_t attn_prefill_ws_bytes(int64_t B, int64_t S, int64_t G, int64_t dim, int64_t vdim, int64_t T, bool cbf16) {
  return jla::hy_attn_prefill_ws_bytes(B, S, G, dim, vdim, T, cbf16);
}

void attn_bias(Tensor q, Tensor kc, Tensor vc, Tensor slot, double scale, double softcap, OptT bias, Tensor out,
               int64_t t_cap, OptT ws, int64_t splits, OptT vt_ws) {
  jla::AttnBias p{};
  check(q.dim() == 4, "attn_bias: q is [B, S, H, dim]");
  p.B = q.size(0); p.S = q.size(1); p.H = q.size(2); p.dim = q.size(3);
  p.q = f32(q, "q");
  p.cbf16 = wtype(kc, "k cache");
  check(wtype(vc, "v cache") == p.cbf16, "attn_bias: cache dtypes differ");
  check(kc.dim() == 4 && vc.dim() == 4 && kc.size(0) == p.B && vc.size(0) == p.B && kc.size(3) == p.dim &&
            kc.size(1) == vc.size(1) && kc.size(2) == vc.size(2),
        "attn_bias: cache shapes");
  p.G = kc.size(1); p.T = kc.size(2); p.vdim = vc.size(3);
  p.kc = kc.data_ptr();
  p.vc = vc.data_ptr();
  p.slot = i32(slot, "slot", 1);
  p.scale = scale;
  p.softcap = softcap;
  if (bias.has_value()) {
    check(bias->dim() == 2 && bias->size(1) == p.H, "attn_bias: bias is [distances, H]");
    p.bias = f32(*bias, "bias");
    p.nbias = bias->size(0);
  }
  check(out.numel() == (int64_t)p.B * p.S * p.H * p.vdim, "attn_bias: out shape");
  p.out = f32w(out, "out");
  p.t_cap = std::min<int64_t>(t_cap, p.T);
  p.splits = splits;
  if (p.S == 1) {
    check(ws.has_value() && splits >= 1 && ws->numel() >= (int64_t)p.B * p.H * splits * (p.vdim + 2),
          "attn_bias: decode workspace");
    p.ws = f32w(*ws, "ws");
  }
  if (vt_ws.has_value()) {
    gpu(*vt_ws, "vt_ws");
    check((int64_t)(vt_ws->numel() * vt_ws->element_size()) >=
              jla::hy_attn_prefill_ws_bytes(p.B, p.S, p.G, p.dim, p.vdim, p.T, p.cbf16),
          "attn_bias: transposed-value workspace too small");
    p.vt_ws = vt_ws->data_ptr();
  }
  rc(jla::hy_attn_bias(p, stream()), "attn_bias");
}

jla::DeltaPrep delta_args(const Tensor& proj, int64_t B, int64_t S, int64_t H, int64_t G, int64_t dim, int64_t vdim,
                          const Tensor& conv_w, const Tensor& conv_state) {
  jla::DeltaPrep p{};
  const int64_t C = 2 * G * dim + H * vdim;
  check(proj.dim() == 2 && proj.size(0) == B * S, "delta: proj rows");
  p.proj = rows2d(proj, "proj", C + H * vdim + 2 * H, &p.ld);
  p.B = B; p.S = S; p.H = H; p.G = G; p.dim = dim; p.vdim = vdim;
  check(conv_w.dim() == 2 && conv_w.size(0) == C, "delta: conv_w is [channels, taps]");
  p.taps = conv_w.size(1);
  p.conv_w = f32(conv_w, "conv_w");
  check(conv_state.numel() == B * C * (p.taps - 1), "delta: conv_state is [B, channels, taps - 1]");
  p.conv_state = f32w(conv_state, "conv_state");
  return p;
}

void delta_prep(Tensor proj, int64_t B, int64_t S, int64_t H, int64_t G, int64_t dim, int64_t vdim, Tensor conv_w,
                Tensor conv_state, Tensor a_log, Tensor dt_bias, Tensor qn, Tensor kn, Tensor vcv, Tensor beta,
                Tensor decay) {
  jla::DeltaPrep p = delta_args(proj, B, S, H, G, dim, vdim, conv_w, conv_state);
  const int64_t M = B * S;
  check(a_log.numel() == H && dt_bias.numel() == H, "delta_prep: per-head constants");
  p.a_log = f32(a_log, "a_log");
  p.dt_bias = f32(dt_bias, "dt_bias");
  check(qn.numel() == M * G * dim && kn.numel() == M * G * dim && vcv.numel() == M * H * vdim &&
            beta.numel() == M * H && decay.numel() == M * H,
        "delta_prep: output shapes");
  p.qn = f32w(qn, "qn");
  p.kn = f32w(kn, "kn");
  p.vc = f32w(vcv, "v");
  p.beta = f32w(beta, "beta");
  p.decay = f32w(decay, "decay");
  rc(jla::hy_delta_prep(p, stream()), "delta_prep");
}

void conv_state_update(Tensor proj, int64_t B, int64_t S, int64_t H, int64_t G, int64_t dim, int64_t vdim, Tensor conv_w,
                       Tensor conv_state) {
  jla::DeltaPrep p = delta_args(proj, B, S, H, G, dim, vdim, conv_w, conv_state);
  rc(jla::hy_conv_state_update(p, stream()), "conv_state_update");
}

void delta_scan(Tensor qn, Tensor kn, Tensor v, Tensor beta, Tensor decay, Tensor state, Tensor o, int64_t B, int64_t S,
                int64_t H, int64_t G, int64_t dim, int64_t vdim) {
  jla::DeltaScan p{};
  const int64_t M = B * S;
  check(qn.numel() == M * G * dim && kn.numel() == M * G * dim && v.numel() == M * H * vdim && beta.numel() == M * H &&
            decay.numel() == M * H && o.numel() == M * H * vdim && state.numel() == B * H * dim * vdim,
        "delta_scan shapes");
  p.qn = f32(qn, "qn");
  p.kn = f32(kn, "kn");
  p.v = f32(v, "v");
  p.beta = f32(beta, "beta");
  p.decay = f32(decay, "decay");
  p.state = f32w(state, "state");
  p.o = f32w(o, "o");
  p.B = B; p.S = S; p.H = H; p.G = G; p.dim = dim; p.vdim = vdim;
  rc(jla::hy_delta_scan(p, stream()), "delta_scan");
}

void gated_rmsnorm(Tensor o, Tensor gate, Tensor w, double eps, Tensor out, int64_t H, int64_t vdim) {
  const int64_t M = o.numel() / (H * vdim);
  check(o.numel() == M * H * vdim && out.numel() == o.numel() && w.numel() == vdim, "gated_rmsnorm shapes");
  int ldg = 0;
  check(gate.dim() == 2 && gate.size(0) == M, "gated_rmsnorm: gate rows");
  const float* g = rows2d(gate, "gate", H * vdim, &ldg);
  rc(jla::hy_gated_rmsnorm(f32(o, "o"), g, ldg, f32(w, "w"), (float)eps, f32w(out, "out"), M, H, vdim, stream()),
     "gated_rmsnorm");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.attr("GEMV_MAX_R") = jla::HY_GEMV_MAX_R;
  m.def("embed_rows", &embed_rows);
  m.def("linear_rows", &linear_rows);
  m.def("route_table", &route_table);
  m.def("norm_residual", &norm_residual);
  m.def("gelu_gate_rows", &gelu_gate_rows);
  m.def("cast_bf16", &cast_bf16);
  m.def("attn_prep", &attn_prep);
  m.def("attn_decode_splits", &attn_decode_splits);
  m.def("attn_bias", &attn_bias);
  m.def("attn_prefill_ws_bytes", &attn_prefill_ws_bytes);
  m.def("delta_prep", &delta_prep);
  m.def("conv_state_update", &conv_state_update);
  m.def("delta_scan", &delta_scan);
  m.def("gated_rmsnorm", &gated_rmsnorm);
}
