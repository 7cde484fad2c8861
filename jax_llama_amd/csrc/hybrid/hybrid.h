// Host launchers of the hybrid-sequence-mixer kernels (module jax_llama_amd._C_hybrid): row-gathered / expert-grouped
// linears on row-major weights of any shape, attention with a distance-bias table and a score soft cap (and block-local
// masks, sinks, per-head factors), rotary positions, the gated delta rule with its short convolutions, two matrix-memory
// recurrences with their gates, and the output-side norms. Pure HIP translation units (no torch headers).
// Every launcher returns 0 on success, <0 on a shape/argument error, >0 for a hipError_t.
//
// Activations between kernels are fp32 in both number formats. "wbf16" selects the weight / cache element type: bf16
// (matrix operands rounded to bf16, fp32 accumulation) or fp32 (exact-f32 MFMA, fp32 caches).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace jla {

// out[c][M, D] (fp32) = table[ids[m], col0 : col0 + D] * scale for c < copies (the same rows `copies` times: the residual
// streams of a hyper-connected stack); table rows are `ld` elements apart. Ids outside [0, V) read row 0.
int hy_embed_rows(const int32_t* ids, const void* table, int wbf16, int V, int ld, int col0, float scale, float* out,
                  int M, int D, int copies, hipStream_t s);

// Epilogue of a row linear. Plain forms take one accumulator, gated forms two (gate rows [0, N), up rows [N, 2N)).
enum RowAct {
  HY_ACT_NONE = 0,        // out = y
  HY_ACT_RELU2 = 1,       // out = max(y, 0)^2
  HY_ACT_SWIGLU = 2,      // out = silu(g) * u
  HY_ACT_CLAMP_GLU = 3,   // g = min(g, limit), u = clamp(u, -limit, limit): out = g * sigmoid(alpha g) * (u + 1)
  HY_ACT_SOFTCAP = 4,     // out = limit * tanh(y / limit)   (limit = 1: tanh)
};

struct RowLinear {
  const void* a;         // [*, lda] activations: fp32, or (a_bf16, tile path with bf16 weights only) bf16
  int a_bf16;
  int lda;
  const int32_t* a_idx;  // optional: activation row of linear row r (else r)
  const float* a_scale;  // optional [R]: linear row r reads a_scale[r] * A[src(r)] (fp32 activations; scaled before
                         // the operand is rounded)
  const float* a_norm_w; // optional [K] (GEMV path only): the row is RMS-normed first, a[k] / sqrt(mean(a^2) + a_norm_eps) *
  float a_norm_eps;      // a_norm_w[k] -- a sublayer's input norm computed by the linear that reads it
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
  int even_rows;         // with offs: every expert has exactly this many rows (a per-head linear); 0 = unknown
  int R;                 // linear rows
  int act;               // RowAct; the gated forms read W as [2N, K]
  float act_limit;       // HY_ACT_CLAMP_GLU
  float act_alpha;
  int add_out;           // out += act(...) instead of out = (fp32 outputs): a residual add in the epilogue
};
inline bool hy_act_gated(int act) { return act == HY_ACT_SWIGLU || act == HY_ACT_CLAMP_GLU; }
// R <= HY_GEMV_MAX_R and (offs == nullptr or row_expert != nullptr): one wave per output column (weights streamed once
// per row group); else the 64 x 64 MFMA tiles (offs: expert-grouped).
constexpr int HY_GEMV_MAX_R = 8;
int hy_linear_rows(const RowLinear& p, hipStream_t s);

// Table routing: expert of (token m, choice c) = table[ids[m], c]. Writes row_expert[R] and row_tok[R] in (m, c) order
// (R = M * top), and the expert-sorted order: sort_tok[p] (token of sorted row p), sort_dst[p] (its (m, c) row),
// offs[E + 1]. One workgroup; E <= 1024.
int hy_route_table(const int32_t* ids, const int32_t* table, int V, int M, int top, int E, int32_t* row_expert,
                   int32_t* row_tok, int32_t* sort_tok, int32_t* sort_dst, int32_t* offs, hipStream_t s);

// rows at or below which a dense linear runs the GEMV; output columns at or below which it does so for any row count
// (hy_linear_rows_is_gemv tells which path a call takes: an input norm can only be fused there)
bool hy_linear_rows_is_gemv(const RowLinear& p);

// Score routing: expert c of token m = the c-th largest of z[m, 0 : E] (rows `ldz` apart; ties go to the lower index),
// weight = sigmoid(z) of the chosen expert (not renormalised). Writes the same index sets as hy_route_table plus the
// weights in (m, c) order (row_w[R]) and in expert-sorted order (sort_w[R]). E <= 1024, top <= E.
// sort_tok == nullptr: the selection only (a few rows that run per-row GEMVs need no sorted order).
int hy_route_topk(const float* z, int ldz, int M, int top, int E, int32_t* row_expert, int32_t* row_tok, float* row_w,
                  int32_t* sort_tok, int32_t* sort_dst, float* sort_w, int32_t* offs, hipStream_t s);

// Grouped softmax routing: scores = softmax(z[m, 0 : E]); the choice is made on score + correction[e] (correction
// optional); the E experts form `groups` equal groups of neighbours, a group's score is its largest choice score, and
// only experts of the `keep` best groups can be chosen; the `top` largest are taken (ties to the lower index
// everywhere), weight = the chosen expert's score (not renormalised). Same outputs as hy_route_topk. E <= 1024,
// E % groups == 0, groups <= 64, top <= keep * (E / groups).
int hy_route_grouped(const float* z, int ldz, const float* correction, int M, int top, int E, int groups, int keep,
                     int32_t* row_expert, int32_t* row_tok, float* row_w, int32_t* sort_tok, int32_t* sort_dst,
                     float* sort_w, int32_t* offs, hipStream_t s);

// Hyper-connections: S residual streams xs[S][M, D] (fp32). With mix != nullptr the streams are replaced in place, all
// at once from the old ones:   xs[t][m] <- sum_s mix[s * S + t] xs[s][m] + out_w[t] * v[m],
//   v[m] = sum_{c < nsum} w_c y[m * nsum + c] (+ extra[m]),  w_c = row_w ? row_w[m * nsum + c] : 1;
// with row_expert, a row whose expert is >= n_real is an identity expert: it adds w_c * ident[m] and its y row is not read.
// With next_in != nullptr: u[m] = sum_t next_in[t] xs[t][m] of the (new) streams. mix == nullptr: only u. S <= 16.
struct HyperUpdate {
  float* xs;
  int S, M, D;
  const float* mix;    // [S, S] indexed [from, to]
  const float* out_w;  // [S]
  const float* y;      // [M * nsum, D]
  int nsum;
  const float* row_w;        // optional [M * nsum]
  const int32_t* row_expert; // optional [M * nsum]
  int n_real;
  const float* ident;  // [M, D], with row_expert
  const float* extra;  // optional [M, D]
  const float* next_in;  // optional [S]
  float* u;              // [M, D], with next_in
};
int hy_hc_update(const HyperUpdate& p, hipStream_t s);

// x[m, :] += (sum_{c < nsum} y[m * nsum + c, :]) * ysc / sqrt(mean(.^2) + eps) * w   (w: one number, or D numbers).
// x == nullptr: out-of-place into `out` without the add (a plain RMS norm).
// extra (optional, [M, D]): sigmoid(extra_gate[m * ldg]) * extra[m, :] joins the sum before the norm (extra_gate ==
// nullptr: weight 1).
int hy_norm_residual(const float* y, int nsum, float ysc, const float* w, int w_vec, float eps, float* x, float* out,
                     int M, int D, const float* extra, const float* extra_gate, int ldg, hipStream_t s);

// y (bf16) = act(x (fp32)), n a multiple of 8; act: HY_ACT_NONE or HY_ACT_RELU2 (the activation of a feed-forward whose two
// products run on the packed GEMM, applied while the hidden activation is rounded for the second)
typedef uint16_t bf16_t;
int hy_cast_bf16(const float* x, bf16_t* y, long long n, int act, hipStream_t s);

// x <- cap * tanh(x / cap) in place (cap = 1: tanh), n elements
int hy_softcap(float* x, long long n, float cap, hipStream_t s);

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
  const float* q_w;  // optional [dim]: gain of the q norm (shared by all heads)
  const float* k_w;  // optional [dim]: gain of the k norm
  int norm_v;        // 0: values are cached as projected
};
// Per head: q, k divided by their RMS over dim (v over vdim); q times 1 + coef * ln(floor((p + 1) / every) + 1);
// k, v written to the cache at slot + s.
int hy_attn_prep(const AttnPrep& p, hipStream_t s);

struct LatentPrep {
  const float* proj;  // [M, ld]: the down-projected latent at columns [col0, col0 + rank)
  int ld, col0;
  const float* w;     // [rank] plain gain
  const int32_t* slot;
  int B, S, rank, T;
  void* cache;        // [B, 1, T, rank]
  int cbf16;
  float eps;
  float* q;           // optional [M, q_cols]: dense copy of proj's columns [q_col0, q_col0 + q_cols) (the queries of the
  int q_cols;         // same fused projection), for the linear that follows
  int q_col0;
  const float* q_norm_w;  // optional [q_cols]: the copy is RMS-normed with this plain gain (a query latent)
  int row;                // width of a cache row, >= rank: the columns behind the latent, proj[col0 + rank, col0 + row), are
                          // cached as they are behind it, their first 2 rot_half numbers rotated by the token's position
  const double* rot_freq; // optional [rot_half]: pair (2i, 2i + 1) turns by position * rot_freq[i]
  int rot_half;
  const int32_t* positions;  // [M], with rot_freq
};
// cache[b, 0, slot + s, :] = proj_latent / sqrt(mean(.^2) + eps) * w: the one vector per token that latent attention
// keeps (keys and values of every head are linear maps of it).
int hy_latent_prep(const LatentPrep& p, hipStream_t s);

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
  const float* sink;     // optional [H]: exp(sink[h]) joins the softmax denominator (no key, no value, not scaled)
  float* out;  // [B * S, H * vdim]
  int t_cap;   // keys the launch may have to cover (decode split sizing); <= T
  float* ws;   // decode split partials: B * H * splits * (vdim + 2) floats
  int splits;
  void* vt_ws;  // prefill: hy_attn_prefill_ws_bytes(...) bytes for the transposed values (nullptr: the plain kernel)
  int chunk;    // > 0: query at slot i sees only keys j <= i with floor(j / chunk) == floor(i / chunk)
  const float* head_scale;  // optional [H]: head h's scores are (q . k * scale) * head_scale[h]
  int window;      // > 0 (chunk == 0): query at slot i sees key j <= i only if i - j < window or j < keep_first
  int keep_first;
  const float* gate;  // optional: head h's output of token m is multiplied by sigmoid(gate[m * ldg + h])
  int ldg;
  int ldv;         // elements between value rows (>= vdim; the values are the first vdim numbers of each row)
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

// out[m * ldo + h * vdim + j] = x[m, h, j] / sqrt(mean_j(x^2) + eps) * w[w_heads ? h * vdim + j : j] *
// act(gate[m * ldg + h * vdim + j]) * gain, act = silu (gate_act 0) or sigmoid (1). x = o, or with denom_floor [M, H]:
// o is [M, H, vdim + 1] and x[m, h, j] = o[m, h, j] / (max(|o[m, h, vdim]|, denom_floor[m, h]) + 1e-6).
struct GatedNorm {
  const float* o;
  const float* gate;
  int ldg;
  const float* w;
  int w_heads;
  float eps;
  float* out;
  int ldo;
  int M, H, vdim;
  int gate_act;
  const float* denom_floor;
  float gain;
};
int hy_gated_rmsnorm(const GatedNorm& p, hipStream_t s);

// Rotary positions for a fused q | k | v projection (+ bias per column): q and k heads rotated on their first 2 qk_half
// numbers (number i with i + qk_half, angle position * qk_freq[i]), v heads on their first 2 v_half numbers when v_freq
// is given; q to a dense buffer, k / v into the caches at slot + s. Angles are formed in 64-bit.
struct RopePrep {
  const float* proj;  // [M, ld]: q heads, k heads, v heads
  int ld;
  const float* bias;  // optional [H dim + G dim + G vdim]
  const int32_t* positions;  // [M]
  const int32_t* slot;
  int B, S, H, G, dim, vdim, T;
  void* kc;  // [B, G, T, dim]
  void* vc;  // [B, G, T, vdim]
  int cbf16;
  float* q;  // [M, H, dim]
  const double* qk_freq;
  int qk_half;
  const double* v_freq;  // optional
  int v_half;
};
int hy_rope_prep(const RopePrep& p, hipStream_t s);

// out[m * ldo + h * n + d] = gain * turn(a[m * lda + h * n + .], sign * positions[m])[d]: the first 2 half numbers of
// every head rotated (freq == nullptr: none, a scaled copy)
// offset: the rotated numbers start there within each head; interleaved: number 2i pairs with 2i + 1 instead. out may be a.
int hy_rotate_heads(const float* a, int lda, const int32_t* positions, const double* freq, int half, int M, int H, int n,
                    float sign, float gain, float* out, int ldo, int offset, int interleaved, hipStream_t s);

// out[i][m][:] = h[m] + (h[m - 1] - h[m]) * mu[i] for i < n; the row before a sequence's first is prev[b] (then set to
// the sequence's last row)
int hy_token_shift(const float* h, float* prev, const float* mu, int n, float* out, int B, int S, int D, hipStream_t s);

struct MlstmPrep {
  const float* proj;  // [M, ld]: input-gate pre-activations at columns [col_i, col_i + H), forget-gate at [col_f, col_f + H)
  int ld, col_i, col_f;
  const float* gate_bias;  // [2 H]
  float cap;
  float* mstate;  // [B, H] running maximum, read and advanced
  float* keep;    // [M, H] exp(f + m' - m)
  float* write;   // [M, H] exp(a - m)
  float* floor;   // [M, H] exp(-m)
  int B, S, H;
};
int hy_mlstm_prep(const MlstmPrep& p, hipStream_t s);

// Linear recurrences over a matrix state [B, H, dim, cols] (fp32), token by token.
//   mode 0 (scalar gates, read after the write; cols = vdim + 1, the last column's value is 1):
//       S <- keep S + write k [v, 1]^T;   o = S^T (q_scale q)
//   mode 1 (a decay per key channel, bonus u for the current token, read before the write; cols = vdim):
//       d = exp(-exp(decay + w0));   o = (S + diag(u) k v^T)^T q;   S <- diag(d) S + k v^T
struct LinScan {
  int mode;
  const float* q;  // token m, head h at q + m * ldq + h * dim
  int ldq;
  const float* k;
  int ldk;
  const float* v;  // token m, head h at v + m * ldv + h * vdim
  int ldv;
  const float* decay;  // mode 0: keep [M, H]; mode 1: pre-activations, token m, head h at decay + m * ldd + h * dim
  int ldd;
  const float* write;  // mode 0: [M, H]
  const float* w0;     // mode 1: [H, dim]
  const float* u;      // mode 1: [H, dim]
  float* state;
  float* o;  // [M, H, cols]
  int B, S, H, dim, vdim;
  float q_scale;
  // nseg > 1: the sequence runs as nseg segments of seg_len tokens side by side (every segment non-empty), in three
  // launches (each segment's own final state and decay product, their combination, the scan proper from each segment's
  // incoming state); seg_state holds B * nseg * H * dim * cols floats, seg_decay B * nseg * H (* dim in mode 1).
  // nseg == 1 (seg_len >= S): one launch.
  int nseg, seg_len;
  float* seg_state;
  float* seg_decay;
};
int hy_lin_scan(const LinScan& p, hipStream_t s);

}  // namespace jla
