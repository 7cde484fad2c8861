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

void embed_rows(Tensor ids, Tensor table, int64_t col0, Tensor out, double scale, int64_t copies) {
  const int wb = wtype(table, "table");
  check(table.dim() == 2 && out.dim() == 2 && copies >= 1 && out.size(0) % copies == 0,
        "embed_rows: 2-d table, out is [copies * M, D]");
  const int M = out.size(0) / copies, D = out.size(1);
  rc(jla::hy_embed_rows(i32(ids, "ids", M), table.data_ptr(), wb, table.size(0), table.size(1), col0,
                        (float)scale, f32w(out, "out"), M, D, copies, stream()),
     "embed_rows");
}

void linear_rows(Tensor a, OptT a_idx, Tensor w, Tensor out, OptT dst_idx, OptT offs, OptT row_expert, int64_t R,
                 int64_t act, double act_limit, double act_alpha, OptT a_scale, OptT a_norm_w, double a_norm_eps,
                 int64_t even_rows, bool add_out) {
  jla::RowLinear p{};
  p.even_rows = even_rows;
  p.add_out = add_out;
  p.wbf16 = wtype(w, "w");
  check(w.dim() == 2 || w.dim() == 3, "linear_rows: w is [Nw, K] or [E, Nw, K]");
  p.E = w.dim() == 3 ? w.size(0) : 1;
  const int64_t Nw = w.size(-2);
  p.K = w.size(-1);
  check(act >= jla::HY_ACT_NONE && act <= jla::HY_ACT_SOFTCAP, "linear_rows: unknown activation");
  const bool gated = jla::hy_act_gated(act);
  check(!gated || Nw % 2 == 0, "linear_rows: a gated activation needs gate and up rows");
  p.N = gated ? Nw / 2 : Nw;
  p.w = w.data_ptr();
  p.w_stride = Nw * (int64_t)p.K;
  p.a = rows2d_any(a, "a", p.K, &p.lda, &p.a_bf16);
  p.out = rows2d_any(out, "out", p.N, &p.ldo, &p.out_bf16);
  p.R = R;
  p.act = act;
  p.act_limit = act_limit;
  p.act_alpha = act_alpha;
  check(R >= 0, "linear_rows: R");
  if (a_idx.has_value()) p.a_idx = i32(*a_idx, "a_idx", R);
  else check(a.size(0) >= R, "linear_rows: a has fewer rows than R");
  if (dst_idx.has_value()) p.dst_idx = i32(*dst_idx, "dst_idx", R);
  else check(out.size(0) >= R, "linear_rows: out has fewer rows than R");
  if (offs.has_value()) p.offs = i32(*offs, "offs", p.E + 1);
  if (row_expert.has_value()) p.row_expert = i32(*row_expert, "row_expert", R);
  if (a_scale.has_value()) {
    check(a_scale->numel() >= R && !p.a_bf16, "linear_rows: a_scale is [R] and needs float32 activations");
    p.a_scale = f32(*a_scale, "a_scale");
  }
  if (a_norm_w.has_value()) {
    check(a_norm_w->numel() == p.K && !p.a_bf16, "linear_rows: a_norm_w is [K] and needs float32 activations");
    p.a_norm_w = f32(*a_norm_w, "a_norm_w");
    p.a_norm_eps = a_norm_eps;
  }
  check(p.E == 1 || p.offs || p.row_expert, "linear_rows: stacked experts need offs or row_expert");
  rc(jla::hy_linear_rows(p, stream()), "linear_rows");
}

// whether a dense linear of `rows` rows with `n` output columns runs the GEMV (where an input norm can be fused)
bool dense_is_gemv(int64_t rows, int64_t n) {
  jla::RowLinear p{};
  p.R = rows; p.N = n; p.E = 1;
  return jla::hy_linear_rows_is_gemv(p);
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

void route_topk(Tensor z, int64_t E, int64_t top, Tensor row_expert, Tensor row_tok, Tensor row_w, OptT sort_tok,
                OptT sort_dst, OptT sort_w, OptT offs) {
  check(z.dim() == 2 && z.size(1) >= E && top >= 1 && top <= E, "route_topk: z is [M, >= E], 1 <= top <= E");
  int ldz = 0;
  const float* zp = rows2d(z, "z", z.size(1), &ldz);
  const int M = z.size(0);
  const int64_t R = (int64_t)M * top;
  check(row_w.numel() >= R, "route_topk: weight outputs hold R numbers");
  const bool sorted = sort_tok.has_value();
  check(sorted == sort_dst.has_value() && sorted == sort_w.has_value() && sorted == offs.has_value(),
        "route_topk: the sorted outputs come together");
  check(!sorted || sort_w->numel() >= R, "route_topk: weight outputs hold R numbers");
  rc(jla::hy_route_topk(zp, ldz, M, top, E, i32w(row_expert, "row_expert", R), i32w(row_tok, "row_tok", R),
                        f32w(row_w, "row_w"), sorted ? i32w(*sort_tok, "sort_tok", R) : nullptr,
                        sorted ? i32w(*sort_dst, "sort_dst", R) : nullptr,
                        sorted ? f32w(*sort_w, "sort_w") : nullptr, sorted ? i32w(*offs, "offs", E + 1) : nullptr,
                        stream()),
     "route_topk");
}

void route_grouped(Tensor z, OptT correction, int64_t E, int64_t top, int64_t groups, int64_t keep, Tensor row_expert,
                   Tensor row_tok, Tensor row_w, OptT sort_tok, OptT sort_dst, OptT sort_w, OptT offs) {
  check(z.dim() == 2 && z.size(1) >= E && top >= 1 && top <= E, "route_grouped: z is [M, >= E], 1 <= top <= E");
  int ldz = 0;
  const float* zp = rows2d(z, "z", z.size(1), &ldz);
  const int M = z.size(0);
  const int64_t R = (int64_t)M * top;
  check(row_w.numel() >= R, "route_grouped: weight outputs hold R numbers");
  check(!correction.has_value() || correction->numel() == E, "route_grouped: correction is [E]");
  const bool sorted = sort_tok.has_value();
  check(sorted == sort_dst.has_value() && sorted == sort_w.has_value() && sorted == offs.has_value(),
        "route_grouped: the sorted outputs come together");
  check(!sorted || sort_w->numel() >= R, "route_grouped: weight outputs hold R numbers");
  rc(jla::hy_route_grouped(zp, ldz, correction.has_value() ? f32(*correction, "correction") : nullptr, M, top, E, groups,
                           keep, i32w(row_expert, "row_expert", R), i32w(row_tok, "row_tok", R), f32w(row_w, "row_w"),
                           sorted ? i32w(*sort_tok, "sort_tok", R) : nullptr,
                           sorted ? i32w(*sort_dst, "sort_dst", R) : nullptr, sorted ? f32w(*sort_w, "sort_w") : nullptr,
                           sorted ? i32w(*offs, "offs", E + 1) : nullptr, stream()),
     "route_grouped");
}

void hc_update(Tensor xs, OptT mix, OptT out_w, OptT y, int64_t nsum, OptT row_w, OptT row_expert, int64_t n_real,
               OptT ident, OptT extra, OptT next_in, OptT u) {
  jla::HyperUpdate p{};
  check(xs.dim() == 3, "hc_update: xs is [S, M, D]");
  p.S = xs.size(0); p.M = xs.size(1); p.D = xs.size(2);
  p.xs = f32w(xs, "xs");
  const int64_t md = (int64_t)p.M * p.D;
  check(mix.has_value() == out_w.has_value() && mix.has_value() == y.has_value(), "hc_update: mix, out_w and y together");
  if (mix.has_value()) {
    check(mix->numel() == (int64_t)p.S * p.S && out_w->numel() == p.S, "hc_update: mix is [S, S], out_w [S]");
    p.mix = f32(*mix, "mix");
    p.out_w = f32(*out_w, "out_w");
    check(nsum >= 1 && y->numel() == md * nsum, "hc_update: y is [M * nsum, D]");
    p.y = f32(*y, "y");
    p.nsum = nsum;
    const int64_t R = (int64_t)p.M * nsum;
    if (row_w.has_value()) {
      check(row_w->numel() >= R, "hc_update: row_w is [M * nsum]");
      p.row_w = f32(*row_w, "row_w");
    }
    if (row_expert.has_value()) {
      check(row_w.has_value() && ident.has_value() && ident->numel() == md, "hc_update: row_expert needs row_w and ident [M, D]");
      p.row_expert = i32(*row_expert, "row_expert", R);
      p.ident = f32(*ident, "ident");
      p.n_real = n_real;
    }
    if (extra.has_value()) {
      check(extra->numel() == md, "hc_update: extra is [M, D]");
      p.extra = f32(*extra, "extra");
    }
  }
  check(next_in.has_value() == u.has_value(), "hc_update: next_in and u together");
  if (next_in.has_value()) {
    check(next_in->numel() == p.S && u->numel() == md, "hc_update: next_in is [S], u [M, D]");
    p.next_in = f32(*next_in, "next_in");
    p.u = f32w(*u, "u");
  }
  rc(jla::hy_hc_update(p, stream()), "hc_update");
}

void norm_residual(Tensor y, int64_t nsum, double ysc, Tensor w, double eps, OptT x, OptT out, OptT extra,
                   OptT extra_gate) {
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
  const float* ep = nullptr;
  const float* gp = nullptr;
  int ldg = 0;
  if (extra.has_value()) {
    check(extra->numel() == (int64_t)M * D, "norm_residual: extra shape");
    ep = f32(*extra, "extra");
  }
  if (extra_gate.has_value()) {
    check(ep && extra_gate->dim() == 2 && extra_gate->size(0) == M, "norm_residual: extra_gate is [M, 1] beside extra");
    gp = rows2d(*extra_gate, "extra_gate", 1, &ldg);
  }
  rc(jla::hy_norm_residual(f32(y, "y"), nsum, (float)ysc, f32(w, "w"), w.numel() > 1 || D == 1, (float)eps, xp, op, M,
                           D, ep, gp, ldg, stream()),
     "norm_residual");
}

void cast_bf16(Tensor x, Tensor y, int64_t act) {
  gpu(y, "y");
  check(y.scalar_type() == torch::kBFloat16 && y.numel() == x.numel() && x.numel() % 8 == 0, "cast_bf16 shapes");
  rc(jla::hy_cast_bf16(f32(x, "x"), reinterpret_cast<jla::bf16_t*>(y.data_ptr()), x.numel(), act, stream()), "cast_bf16");
}

void softcap(Tensor x, double cap) {
  rc(jla::hy_softcap(f32w(x, "x"), x.numel(), (float)cap, stream()), "softcap");
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
               int64_t vdim, OptT kc, OptT vc, Tensor q, double eps, double temp_coef, int64_t temp_every, OptT q_w, OptT k_w,
               bool norm_v) {
  jla::AttnPrep p{};
  p.norm_v = norm_v;
  if (q_w.has_value()) {
    check(q_w->numel() == dim, "attn_prep: q_w is [dim]");
    p.q_w = f32(*q_w, "q_w");
  }
  if (k_w.has_value()) {
    check(k_w->numel() == dim, "attn_prep: k_w is [dim]");
    p.k_w = f32(*k_w, "k_w");
  }
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

const double* f64(const Tensor& t, const char* name);

void latent_prep(Tensor proj, int64_t col0, Tensor w, Tensor slot, int64_t B, int64_t S, Tensor cache, double eps,
                 OptT q, int64_t q_col0, OptT q_norm_w, OptT rot_freq, OptT positions) {
  jla::LatentPrep p{};
  check(proj.dim() == 2 && proj.size(0) == B * S && proj.scalar_type() == torch::kFloat32 && proj.is_cuda() &&
            proj.stride(1) == 1,
        "latent_prep: proj is a float32 [B * S, cols] GPU view with unit inner stride");
  p.proj = reinterpret_cast<const float*>(proj.data_ptr());
  p.ld = proj.stride(0);
  p.col0 = col0;
  p.cbf16 = wtype(cache, "latent cache");
  check(cache.dim() == 4 && cache.size(0) == B && cache.size(1) == 1, "latent_prep: cache is [B, 1, T, row]");
  p.T = cache.size(2);
  p.row = cache.size(3);
  p.rank = w.numel();
  check(col0 >= 0 && p.rank >= 1 && p.rank <= p.row && col0 + p.row <= proj.size(1), "latent_prep: latent columns / gain");
  if (rot_freq.has_value() && rot_freq->numel() > 0) {
    p.rot_half = rot_freq->numel();
    check(2 * p.rot_half <= p.row - p.rank && positions.has_value(), "latent_prep: rotated numbers / positions");
    p.rot_freq = f64(*rot_freq, "rot_freq");
    p.positions = i32(*positions, "positions", B * S);
  }
  p.w = f32(w, "w");
  p.slot = i32(slot, "slot", 1);
  p.B = B; p.S = S;
  p.cache = cache.data_ptr();
  p.eps = eps;
  if (q.has_value()) {
    check(q->dim() == 2 && q->size(0) == B * S && q_col0 >= 0 && q_col0 + q->size(1) <= proj.size(1),
          "latent_prep: q is [B * S, q_cols]");
    p.q = f32w(*q, "q");
    p.q_cols = q->size(1);
    p.q_col0 = q_col0;
    if (q_norm_w.has_value()) {
      check(q_norm_w->numel() == p.q_cols, "latent_prep: q_norm_w is [q_cols]");
      p.q_norm_w = f32(*q_norm_w, "q_norm_w");
    }
  }
  rc(jla::hy_latent_prep(p, stream()), "latent_prep");
}

int64_t attn_decode_splits(int64_t B, int64_t H, int64_t t_cap) { return jla::hy_attn_decode_splits(B, H, t_cap); }

int64_t attn_prefill_ws_bytes(int64_t B, int64_t S, int64_t G, int64_t dim, int64_t vdim, int64_t T, bool cbf16) {
  return jla::hy_attn_prefill_ws_bytes(B, S, G, dim, vdim, T, cbf16);
}

void attn_bias(Tensor q, Tensor kc, Tensor vc, Tensor slot, double scale, double softcap, OptT bias, Tensor out,
               int64_t t_cap, OptT ws, int64_t splits, OptT vt_ws, OptT sink, int64_t chunk, OptT head_scale, int64_t window,
               int64_t keep_first, OptT gate, c10::optional<int64_t> vdim) {
  jla::AttnBias p{};
  check(q.dim() == 4, "attn_bias: q is [B, S, H, dim]");
  p.B = q.size(0); p.S = q.size(1); p.H = q.size(2); p.dim = q.size(3);
  p.q = f32(q, "q");
  p.cbf16 = wtype(kc, "k cache");
  check(wtype(vc, "v cache") == p.cbf16, "attn_bias: cache dtypes differ");
  check(kc.dim() == 4 && vc.dim() == 4 && kc.size(0) == p.B && vc.size(0) == p.B && kc.size(3) == p.dim &&
            kc.size(1) == vc.size(1) && kc.size(2) == vc.size(2),
        "attn_bias: cache shapes");
  p.G = kc.size(1); p.T = kc.size(2);
  p.ldv = vc.size(3);
  p.vdim = vdim.has_value() ? *vdim : vc.size(3);
  check(p.vdim >= 1 && p.vdim <= p.ldv, "attn_bias: vdim is at most the width of a value row");
  check(window >= 0 && window <= INT32_MAX && keep_first >= 0 && keep_first <= INT32_MAX, "attn_bias: window / keep_first");
  p.window = window;
  p.keep_first = keep_first;
  if (gate.has_value()) {
    check(gate->dim() == 2 && gate->size(0) == (int64_t)p.B * p.S && gate->size(1) >= p.H, "attn_bias: gate is [B * S, >= H]");
    p.gate = rows2d(*gate, "gate", gate->size(1), &p.ldg);
  }
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
  if (sink.has_value()) {
    check(sink->numel() == p.H, "attn_bias: sink is [H]");
    p.sink = f32(*sink, "sink");
  }
  check(chunk >= 0 && chunk <= INT32_MAX, "attn_bias: chunk");
  p.chunk = chunk;
  if (head_scale.has_value()) {
    check(head_scale->numel() == p.H, "attn_bias: head_scale is [H]");
    p.head_scale = f32(*head_scale, "head_scale");
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

// a 2-d float32 view with unit inner stride whose rows hold at least `cols` numbers
float* slice2d(const Tensor& t, const char* name, int64_t rows, int64_t cols, int* ld) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 && t.dim() == 2 && t.stride(1) == 1 &&
                  t.size(0) == rows && t.size(1) == cols && (rows <= 1 || t.stride(0) >= cols),
              "jax_llama_amd._C_hybrid: ", name, " must be a float32 [", rows, ", ", cols,
              "] GPU view with unit inner stride");
  *ld = rows > 1 ? (int)t.stride(0) : (int)cols;
  return reinterpret_cast<float*>(t.data_ptr());
}

// a [M, H, n] float32 view whose heads are adjacent (stride(1) == n, unit inner stride): rows may be strided
const float* heads3d(const Tensor& t, const char* name, int64_t M, int64_t H, int64_t n, int* ld) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 && t.dim() == 3 && t.size(0) == M && t.size(1) == H &&
                  t.size(2) == n && t.stride(2) == 1 && (H == 1 || t.stride(1) == n) && (M <= 1 || t.stride(0) >= H * n),
              "jax_llama_amd._C_hybrid: ", name, " must be a float32 [", M, ", ", H, ", ", n,
              "] GPU view with adjacent heads");
  *ld = M > 1 ? (int)t.stride(0) : (int)(H * n);
  return reinterpret_cast<const float*>(t.data_ptr());
}

const double* f64(const Tensor& t, const char* name) {
  gpu(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kFloat64, "jax_llama_amd._C_hybrid: ", name, " must be float64");
  return reinterpret_cast<const double*>(t.data_ptr());
}

void gated_rmsnorm(Tensor o, Tensor gate, Tensor w, double eps, Tensor out, int64_t H, int64_t vdim, int64_t gate_act,
                   OptT denom_floor, double gain) {
  jla::GatedNorm p{};
  const int64_t ov = denom_floor.has_value() ? vdim + 1 : vdim;
  const int64_t M = o.numel() / (H * ov);
  check(o.numel() == M * H * ov && (w.numel() == vdim || w.numel() == H * vdim), "gated_rmsnorm shapes");
  check(gate.dim() == 2 && gate.size(0) == M, "gated_rmsnorm: gate rows");
  p.o = f32(o, "o");
  p.gate = rows2d(gate, "gate", H * vdim, &p.ldg);
  p.w = f32(w, "w");
  p.w_heads = w.numel() != vdim || H == 1;
  p.eps = eps;
  p.out = slice2d(out, "out", M, H * vdim, &p.ldo);
  p.M = M; p.H = H; p.vdim = vdim;
  p.gate_act = gate_act;
  if (denom_floor.has_value()) {
    check(denom_floor->numel() == M * H, "gated_rmsnorm: denom_floor is [M, H]");
    p.denom_floor = f32(*denom_floor, "denom_floor");
  }
  p.gain = gain;
  rc(jla::hy_gated_rmsnorm(p, stream()), "gated_rmsnorm");
}

void rope_prep(Tensor proj, OptT bias, Tensor positions, Tensor slot, int64_t B, int64_t S, int64_t H, int64_t G,
               int64_t dim, int64_t vdim, Tensor kc, Tensor vc, Tensor q, Tensor qk_freq, OptT v_freq) {
  jla::RopePrep p{};
  const int64_t cols = (H + G) * dim + G * vdim;
  check(proj.dim() == 2 && proj.size(0) == B * S, "rope_prep: proj rows");
  p.proj = rows2d(proj, "proj", cols, &p.ld);
  if (bias.has_value()) {
    check(bias->numel() == cols, "rope_prep: one bias per projection column");
    p.bias = f32(*bias, "bias");
  }
  p.positions = i32(positions, "positions", B * S);
  p.slot = i32(slot, "slot", 1);
  p.B = B; p.S = S; p.H = H; p.G = G; p.dim = dim; p.vdim = vdim;
  p.cbf16 = wtype(kc, "k cache");
  check(wtype(vc, "v cache") == p.cbf16, "rope_prep: cache dtypes differ");
  check(kc.dim() == 4 && kc.size(0) == B && kc.size(1) == G && kc.size(3) == dim, "rope_prep: k cache shape");
  p.T = kc.size(2);
  check(vc.dim() == 4 && vc.size(0) == B && vc.size(1) == G && vc.size(2) == p.T && vc.size(3) == vdim,
        "rope_prep: v cache shape");
  p.kc = kc.data_ptr();
  p.vc = vc.data_ptr();
  check(q.numel() == B * S * H * dim, "rope_prep: q shape");
  p.q = f32w(q, "q");
  p.qk_half = qk_freq.numel();
  check(2 * p.qk_half <= dim, "rope_prep: more rotated numbers than a head holds");
  p.qk_freq = p.qk_half ? f64(qk_freq, "qk_freq") : nullptr;
  if (v_freq.has_value() && v_freq->numel() > 0) {
    p.v_half = v_freq->numel();
    check(2 * p.v_half <= vdim, "rope_prep: more rotated numbers than a value head holds");
    p.v_freq = f64(*v_freq, "v_freq");
  }
  rc(jla::hy_rope_prep(p, stream()), "rope_prep");
}

void rotate_heads(Tensor a, Tensor positions, OptT freq, int64_t H, double sign, double gain, Tensor out, int64_t offset,
                  bool interleaved) {
  check(a.dim() == 2 && a.size(1) % H == 0, "rotate_heads: a is [M, H * n]");
  const int64_t M = a.size(0), n = a.size(1) / H;
  int lda = 0, ldo = 0;
  const float* ap = slice2d(a, "a", M, H * n, &lda);
  float* op = slice2d(out, "out", M, H * n, &ldo);
  const int half = freq.has_value() ? (int)freq->numel() : 0;
  check(offset >= 0 && offset + 2 * half <= n, "rotate_heads: more rotated numbers than a head holds");
  rc(jla::hy_rotate_heads(ap, lda, i32(positions, "positions", M), half ? f64(*freq, "freq") : nullptr, half, M, H, n,
                          (float)sign, (float)gain, op, ldo, offset, interleaved, stream()),
     "rotate_heads");
}

void token_shift(Tensor h, Tensor prev, Tensor mu, Tensor out, int64_t B, int64_t S) {
  check(mu.dim() == 2, "token_shift: mu is [n, D]");
  const int64_t n = mu.size(0), D = mu.size(1);
  check(h.numel() == B * S * D && prev.numel() == B * D && out.numel() == n * B * S * D, "token_shift shapes");
  rc(jla::hy_token_shift(f32(h, "h"), f32w(prev, "prev"), f32(mu, "mu"), n, f32w(out, "out"), B, S, D, stream()),
     "token_shift");
}

void mlstm_prep(Tensor proj, int64_t col_i, int64_t col_f, Tensor gate_bias, double cap, Tensor mstate, Tensor out,
                int64_t B, int64_t S, int64_t H) {
  jla::MlstmPrep p{};
  check(proj.dim() == 2 && proj.size(0) == B * S, "mlstm_prep: proj rows");
  p.proj = rows2d(proj, "proj", proj.size(1), &p.ld);
  check(col_i >= 0 && col_f >= 0 && col_i + H <= proj.size(1) && col_f + H <= proj.size(1), "mlstm_prep: gate columns");
  p.col_i = col_i; p.col_f = col_f;
  check(gate_bias.numel() == 2 * H && mstate.numel() == B * H && out.numel() == 3 * B * S * H, "mlstm_prep shapes");
  p.gate_bias = f32(gate_bias, "gate_bias");
  p.cap = cap;
  p.mstate = f32w(mstate, "mstate");
  float* o = f32w(out, "out");
  p.keep = o; p.write = o + B * S * H; p.floor = o + 2 * B * S * H;
  p.B = B; p.S = S; p.H = H;
  rc(jla::hy_mlstm_prep(p, stream()), "mlstm_prep");
}

void lin_scan(int64_t mode, Tensor q, Tensor k, Tensor v, Tensor decay, OptT write, OptT w0, OptT u, Tensor state,
              Tensor o, int64_t B, int64_t S, double q_scale, int64_t nseg, int64_t seg_len, OptT seg_ws) {
  jla::LinScan p{};
  check(mode == 0 || mode == 1, "lin_scan: mode");
  check(q.dim() == 3 && v.dim() == 3, "lin_scan: q, k are [M, H, dim], v is [M, H, vdim]");
  const int64_t M = B * S, H = q.size(1), dim = q.size(2), vdim = v.size(2);
  const int64_t cols = mode == 0 ? vdim + 1 : vdim;
  p.mode = mode;
  p.q = heads3d(q, "q", M, H, dim, &p.ldq);
  p.k = heads3d(k, "k", M, H, dim, &p.ldk);
  p.v = heads3d(v, "v", M, H, vdim, &p.ldv);
  if (mode == 0) {
    check(decay.numel() == M * H && write.has_value() && write->numel() == M * H, "lin_scan: keep, write are [M, H]");
    p.decay = f32(decay, "keep");
    p.write = f32(*write, "write");
  } else {
    p.decay = heads3d(decay, "decay", M, H, dim, &p.ldd);
    check(w0.has_value() && u.has_value() && w0->numel() == H * dim && u->numel() == H * dim, "lin_scan: w0, u are [H, dim]");
    p.w0 = f32(*w0, "w0");
    p.u = f32(*u, "u");
  }
  check(state.numel() == B * H * dim * cols && o.numel() == M * H * cols, "lin_scan: state / output shapes");
  p.state = f32w(state, "state");
  p.o = f32w(o, "o");
  p.B = B; p.S = S; p.H = H; p.dim = dim; p.vdim = vdim;
  p.q_scale = q_scale;
  check(nseg >= 1 && seg_len >= 1 && nseg * seg_len >= S && (nseg - 1) * seg_len < S, "lin_scan: segments cover the tokens");
  p.nseg = nseg;
  p.seg_len = seg_len;
  if (nseg > 1) {
    const int64_t ns = B * nseg * H * dim * cols, nd = B * nseg * H * (mode == 1 ? dim : 1);
    check(seg_ws.has_value() && seg_ws->numel() >= ns + nd, "lin_scan: segment workspace");
    p.seg_state = f32w(*seg_ws, "seg_ws");
    p.seg_decay = p.seg_state + ns;
  }
  rc(jla::hy_lin_scan(p, stream()), "lin_scan");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.attr("GEMV_MAX_R") = jla::HY_GEMV_MAX_R;
  m.def("embed_rows", &embed_rows, py::arg("ids"), py::arg("table"), py::arg("col0"), py::arg("out"), py::arg("scale"),
        py::arg("copies") = 1);
  m.def("route_grouped", &route_grouped);
  m.def("hc_update", &hc_update);
  m.def("linear_rows", &linear_rows, py::arg("a"), py::arg("a_idx"), py::arg("w"), py::arg("out"), py::arg("dst_idx"),
        py::arg("offs"), py::arg("row_expert"), py::arg("R"), py::arg("act"), py::arg("act_limit"), py::arg("act_alpha"),
        py::arg("a_scale"), py::arg("a_norm_w"), py::arg("a_norm_eps"), py::arg("even_rows") = 0,
        py::arg("add_out") = false);
  m.def("route_table", &route_table);
  m.def("route_topk", &route_topk);
  m.def("dense_is_gemv", &dense_is_gemv);
  m.def("latent_prep", &latent_prep, py::arg("proj"), py::arg("col0"), py::arg("w"), py::arg("slot"), py::arg("B"),
        py::arg("S"), py::arg("cache"), py::arg("eps"), py::arg("q"), py::arg("q_col0") = 0,
        py::arg("q_norm_w") = py::none(), py::arg("rot_freq") = py::none(), py::arg("positions") = py::none());
  m.attr("ACT_NONE") = (int)jla::HY_ACT_NONE;
  m.attr("ACT_RELU2") = (int)jla::HY_ACT_RELU2;
  m.attr("ACT_SWIGLU") = (int)jla::HY_ACT_SWIGLU;
  m.attr("ACT_CLAMP_GLU") = (int)jla::HY_ACT_CLAMP_GLU;
  m.def("norm_residual", &norm_residual);
  m.def("gelu_gate_rows", &gelu_gate_rows);
  m.def("cast_bf16", &cast_bf16, py::arg("x"), py::arg("y"), py::arg("act") = 0);
  m.def("softcap", &softcap);
  m.def("attn_prep", &attn_prep, py::arg("proj"), py::arg("positions"), py::arg("slot"), py::arg("B"), py::arg("S"),
        py::arg("H"), py::arg("G"), py::arg("dim"), py::arg("vdim"), py::arg("kc"), py::arg("vc"), py::arg("q"),
        py::arg("eps"), py::arg("temp_coef"), py::arg("temp_every"), py::arg("q_w") = py::none(),
        py::arg("k_w") = py::none(), py::arg("norm_v") = true);
  m.def("attn_decode_splits", &attn_decode_splits);
  m.def("attn_bias", &attn_bias, py::arg("q"), py::arg("kc"), py::arg("vc"), py::arg("slot"), py::arg("scale"),
        py::arg("softcap"), py::arg("bias"), py::arg("out"), py::arg("t_cap"), py::arg("ws"), py::arg("splits"),
        py::arg("vt_ws"), py::arg("sink"), py::arg("chunk") = 0, py::arg("head_scale") = py::none(),
        py::arg("window") = 0, py::arg("keep_first") = 0, py::arg("gate") = py::none(), py::arg("vdim") = py::none());
  m.def("attn_prefill_ws_bytes", &attn_prefill_ws_bytes);
  m.def("delta_prep", &delta_prep);
  m.def("conv_state_update", &conv_state_update);
  m.def("delta_scan", &delta_scan);
  m.def("gated_rmsnorm", &gated_rmsnorm, py::arg("o"), py::arg("gate"), py::arg("w"), py::arg("eps"), py::arg("out"),
        py::arg("H"), py::arg("vdim"), py::arg("gate_act") = 0, py::arg("denom_floor") = py::none(),
        py::arg("gain") = 1.0);
  m.attr("ACT_SOFTCAP") = (int)jla::HY_ACT_SOFTCAP;
  m.def("rope_prep", &rope_prep);
  m.def("rotate_heads", &rotate_heads, py::arg("a"), py::arg("positions"), py::arg("freq"), py::arg("H"), py::arg("sign"),
        py::arg("gain"), py::arg("out"), py::arg("offset") = 0, py::arg("interleaved") = false);
  m.def("token_shift", &token_shift);
  m.def("mlstm_prep", &mlstm_prep);
  m.def("lin_scan", &lin_scan, py::arg("mode"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("decay"),
        py::arg("write"), py::arg("w0"), py::arg("u"), py::arg("state"), py::arg("o"), py::arg("B"), py::arg("S"),
        py::arg("q_scale"), py::arg("nseg") = 1, py::arg("seg_len") = (int64_t)1 << 40, py::arg("seg_ws") = py::none());
}
