// Row kernels of the hybrid stack: embedding-slice gather, the norm on a sublayer's OUTPUT fused with the residual add
// (x += rms_norm(sum of the chosen experts' outputs) * w, w one number or a vector), the per-layer token-side gate
// (gelu_tanh(gate projection) * a slice of a second embedding table), the latent-attention prep (normed latent, normed
// query latent, rotated shared key part, cache write) and the hyper-connection update of several residual streams.
// fp32 statistics and residual.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

JLA_DEV float ns_ld(const float* p) { return *p; }
JLA_DEV float ns_ld(const bf16_t* p) { return bf2f(*p); }

template <typename WT>
__global__ void __launch_bounds__(256) embed_rows_kernel(const int32_t* ids, const WT* table, int V, int ld, int col0,
                                                         float scale, float* out, int D, int copies) {
  const int m = blockIdx.x, M = gridDim.x;
  int id = ids[m];
  id = id < 0 || id >= V ? 0 : id;
  const WT* row = table + (size_t)id * ld + col0;
  for (int d = threadIdx.x; d < D; d += 256) {
    const float v = ns_ld(row + d) * scale;
    for (int c = 0; c < copies; ++c) out[((size_t)c * M + m) * D + d] = v;
  }
}

int hy_embed_rows(const int32_t* ids, const void* table, int wbf16, int V, int ld, int col0, float scale, float* out,
                  int M, int D, int copies, hipStream_t s) {
  if (M < 0 || D < 1 || V < 1 || col0 < 0 || col0 + D > ld || copies < 1) return -1;
  if (M == 0) return 0;
  if (wbf16)
    embed_rows_kernel<bf16_t><<<M, 256, 0, s>>>(ids, reinterpret_cast<const bf16_t*>(table), V, ld, col0, scale, out, D,
                                                copies);
  else
    embed_rows_kernel<float><<<M, 256, 0, s>>>(ids, reinterpret_cast<const float*>(table), V, ld, col0, scale, out, D,
                                               copies);
  JLA_CHECK_LAUNCH();
  return 0;
}

// one workgroup per row; rows of up to 4096 columns are held in registers: NU values per thread (a template
// parameter, so the loads are branch-free and all in flight together: y's rows, x, the gain and the extra summand in
// one round trip; surplus threads re-read the last column). NU = 0: any width, two passes over y.
template <int NU>
__global__ void __launch_bounds__(256) norm_residual_kernel(const float* y, int nsum, float ysc, const float* w,
                                                            int w_vec, float eps, float* x, float* out, int D,
                                                            const float* extra, const float* extra_gate, int ldg) {
  __shared__ float red[16];
  const int m = blockIdx.x;
  const float* yr = y + (size_t)m * nsum * D;
  const float* er = extra ? extra + (size_t)m * D : nullptr;
  const float eg = er ? (extra_gate ? hy_sigmoid(extra_gate[(size_t)m * ldg]) : 1.f) : 0.f;
  if constexpr (NU > 0) {
    float v[NU], xv[NU], wv[NU], ev[NU];
    int dd[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      dd[u] = min((int)threadIdx.x + 256 * u, D - 1);
      xv[u] = x ? x[(size_t)m * D + dd[u]] : 0.f;
      wv[u] = w[w_vec ? dd[u] : 0];
      ev[u] = er ? er[dd[u]] : 0.f;
      v[u] = 0.f;
    }
    for (int c = 0; c < nsum; ++c) {
#pragma unroll
      for (int u = 0; u < NU; ++u) v[u] += yr[(size_t)c * D + dd[u]];
    }
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      v[u] = fmaf(eg, ev[u], v[u] * ysc);
      if ((int)threadIdx.x + 256 * u < D) ss = fmaf(v[u], v[u], ss);
    }
    ss = block_sum(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int u = 0; u < NU; ++u) {
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
    if (er) v = fmaf(eg, er[d], v);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float sc = 1.f / sqrtf(ss / (float)D + eps);
  const float w0 = w_vec ? 0.f : w[0];
  for (int d = threadIdx.x; d < D; d += 256) {
    float v = 0.f;
    for (int c = 0; c < nsum; ++c) v += yr[(size_t)c * D + d];
    v *= ysc;
    if (er) v = fmaf(eg, er[d], v);
    v = v * sc * (w_vec ? w[d] : w0);
    if (x) x[(size_t)m * D + d] += v;
    else out[(size_t)m * D + d] = v;
  }
}

int hy_norm_residual(const float* y, int nsum, float ysc, const float* w, int w_vec, float eps, float* x, float* out,
                     int M, int D, const float* extra, const float* extra_gate, int ldg, hipStream_t s) {
  if (M < 0 || D < 1 || nsum < 1 || (!x && !out) || (extra_gate && (!extra || ldg < 1))) return -1;
  if (M == 0) return 0;
#define NR_LAUNCH(NU) \
  norm_residual_kernel<NU><<<M, 256, 0, s>>>(y, nsum, ysc, w, w_vec, eps, x, out, D, extra, extra_gate, ldg)
  const int nu = (D + 255) / 256;
  if (nu <= 1) NR_LAUNCH(1);
  else if (nu <= 2) NR_LAUNCH(2);
  else if (nu <= 4) NR_LAUNCH(4);
  else if (nu <= 8) NR_LAUNCH(8);
  else if (nu <= 16) NR_LAUNCH(16);
  else NR_LAUNCH(0);
#undef NR_LAUNCH
  JLA_CHECK_LAUNCH();
  return 0;
}

// bf16 copy of an fp32 activation (the A operand of the packed MFMA GEMMs), 8 elements per thread
template <int RELU2>
__global__ void __launch_bounds__(256) cast_bf16_kernel(const float* __restrict__ x, bf16_t* __restrict__ y, long long n8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  float f[8];
  hy_load8(x + 8 * i, 8, f);
  if (RELU2) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float r = fmaxf(f[k], 0.f);
      f[k] = r * r;
    }
  }
  *reinterpret_cast<u32x4*>(y + 8 * i) = pack8(f);
}

int hy_cast_bf16(const float* x, bf16_t* y, long long n, int act, hipStream_t s) {
  if (n < 0 || n % 8 || (act != HY_ACT_NONE && act != HY_ACT_RELU2)) return -1;
  if (n == 0) return 0;
  const long long n8 = n / 8;
  if (act == HY_ACT_RELU2) cast_bf16_kernel<1><<<(unsigned)((n8 + 255) / 256), 256, 0, s>>>(x, y, n8);
  else cast_bf16_kernel<0><<<(unsigned)((n8 + 255) / 256), 256, 0, s>>>(x, y, n8);
  JLA_CHECK_LAUNCH();
  return 0;
}

// x <- cap * tanh(x / cap), one thread per element
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ x, long long n, float cap, float inv_cap) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] * inv_cap);
}

int hy_softcap(float* x, long long n, float cap, hipStream_t s) {
  if (n < 0 || !(cap > 0.f)) return -1;
  if (n == 0) return 0;
  if ((n + 255) / 256 > 0x7fffffffLL) return -2;
  softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(x, n, cap, 1.f / cap);
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

JLA_DEV void lp_st(float* p, float v) { *p = v; }
JLA_DEV void lp_st(bf16_t* p, float v) { *p = f2bf(v); }
// sine and cosine of position * freq, the angle formed and reduced to [-pi, pi] in 64-bit
JLA_DEV void lp_sincos(int pos, double freq, float* s, float* c) {
  const double a = (double)pos * freq;
  const double r = a - 6.283185307179586476925 * rint(a * 0.159154943091895335769);
  sincosf((float)r, s, c);
}

// one workgroup per token: RMS norm of the down-projected latent with its gain, written to the cache row of slot + s,
// and the dense copy of the queries (four loads in flight per thread: a decode step is one token, so the copy's
// latency, not its bandwidth, is what shows)
template <typename CT>
__global__ void __launch_bounds__(256) latent_prep_kernel(LatentPrep p) {
  __shared__ float red[16];
  const int tid = threadIdx.x, m = blockIdx.x;
  if (p.q) {
    const float* src = p.proj + (size_t)m * p.ld + p.q_col0;
    float* dst = p.q + (size_t)m * p.q_cols;
    float qsc = 1.f;
    if (p.q_norm_w) {  // a query latent: RMS over the copied columns
      float qs = 0.f;
      for (int d0 = 0; d0 < p.q_cols; d0 += 1024) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = src[min(d0 + tid + 256 * u, p.q_cols - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (d0 + tid + 256 * u < p.q_cols) qs = fmaf(v[u], v[u], qs);
      }
      qs = block_sum(qs, red);
      qsc = 1.f / sqrtf(qs / (float)p.q_cols + p.eps);
    }
    for (int d0 = 0; d0 < p.q_cols; d0 += 1024) {
      float v[4], g[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int d = min(d0 + tid + 256 * u, p.q_cols - 1);
        v[u] = src[d];
        g[u] = p.q_norm_w ? p.q_norm_w[d] : 1.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (d0 + tid + 256 * u < p.q_cols) dst[d0 + tid + 256 * u] = p.q_norm_w ? v[u] * qsc * g[u] : v[u];
    }
  }
  const float* row = p.proj + (size_t)m * p.ld + p.col0;
  constexpr int LP_REGS = 4;  // ranks up to 1024 stay in registers
  float rv[LP_REGS], wv[LP_REGS];
  float ss = 0.f;
  if (p.rank <= 256 * LP_REGS) {
#pragma unroll
    for (int u = 0; u < LP_REGS; ++u) {
      const int d = min(tid + 256 * u, p.rank - 1);
      rv[u] = row[d];
      wv[u] = p.w[d];
    }
#pragma unroll
    for (int u = 0; u < LP_REGS; ++u)
      if (tid + 256 * u < p.rank) ss = fmaf(rv[u], rv[u], ss);
  } else {
    for (int d = tid; d < p.rank; d += 256) ss = fmaf(row[d], row[d], ss);
  }
  ss = block_sum(ss, red);
  const float sc = 1.f / sqrtf(ss / (float)p.rank + p.eps);
  const int b = m / p.S, t = *p.slot + (m - b * p.S);
  if (t < 0 || t >= p.T) return;  // cache full: the write is dropped
  CT* dst = reinterpret_cast<CT*>(p.cache) + ((size_t)b * p.T + t) * p.row;
  // behind the latent: the shared key part, rotated in pairs (2i, 2i + 1) by the token's position
  const int tail = p.row - p.rank;
  if (tail > 0) {
    const float* tr = row + p.rank;
    const int pos = p.rot_freq ? p.positions[m] : 0;
    for (int i = tid; i < p.rot_half; i += 256) {
      float sn, cs;
      lp_sincos(pos, p.rot_freq[i], &sn, &cs);
      const float a = tr[2 * i], c = tr[2 * i + 1];
      lp_st(dst + p.rank + 2 * i, a * cs - c * sn);
      lp_st(dst + p.rank + 2 * i + 1, c * cs + a * sn);
    }
    for (int d = 2 * p.rot_half + tid; d < tail; d += 256) lp_st(dst + p.rank + d, tr[d]);
  }
  if (p.rank <= 256 * LP_REGS) {
#pragma unroll
    for (int u = 0; u < LP_REGS; ++u) {
      const int d = tid + 256 * u;
      if (d < p.rank) {
        const float v = rv[u] * sc * wv[u];
        if constexpr (sizeof(CT) == 2) dst[d] = f2bf(v);
        else dst[d] = v;
      }
    }
  } else {
    for (int d = tid; d < p.rank; d += 256) {
      const float v = row[d] * sc * p.w[d];
      if constexpr (sizeof(CT) == 2) dst[d] = f2bf(v);
      else dst[d] = v;
    }
  }
}

int hy_latent_prep(const LatentPrep& p, hipStream_t s) {
  if (p.B < 0 || p.S < 1 || p.rank < 1 || p.T < 1 || p.col0 < 0 || p.row < p.rank || p.col0 + p.row > p.ld) return -1;
  if (p.q && (p.q_cols < 1 || p.q_col0 < 0 || p.q_col0 + p.q_cols > p.ld)) return -2;
  if (p.q_norm_w && !p.q) return -2;
  if (p.rot_half < 0 || 2 * p.rot_half > p.row - p.rank || (p.rot_half > 0 && (!p.rot_freq || !p.positions))) return -4;
  const long long M = (long long)p.B * p.S;
  if (M == 0) return 0;
  if (M > 0x7fffffff) return -3;
  if (p.cbf16) latent_prep_kernel<bf16_t><<<(unsigned)M, 256, 0, s>>>(p);
  else latent_prep_kernel<float><<<(unsigned)M, 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

// one workgroup per token; a thread owns NU columns 256 apart (a template parameter, so that every load of the step --
// all streams, the extra summand, the identity input, then the sublayer's rows -- is issued without a branch and in
// flight together; surplus threads re-read the last column and store nothing). Every stream's old value of a column is
// read before any is written, so the replacement is in place. NU = 0: any width, one column at a time.
template <int S, int NU>
__global__ void __launch_bounds__(256) hc_update_kernel(HyperUpdate p) {
  constexpr int NC = NU > 0 ? NU : 1;
  const int m = blockIdx.x;
  float mixv[S][S], outw[S], inw[S];
#pragma unroll
  for (int a = 0; a < S; ++a) {
    outw[a] = p.mix ? p.out_w[a] : 0.f;
    inw[a] = p.next_in ? p.next_in[a] : 0.f;
#pragma unroll
    for (int t = 0; t < S; ++t) mixv[a][t] = p.mix ? p.mix[a * S + t] : (a == t ? 1.f : 0.f);
  }
  const int nsum = p.mix ? p.nsum : 0;
  const size_t plane = (size_t)p.M * p.D, row = (size_t)m * p.D;
  for (int d0 = threadIdx.x; d0 < (NU > 0 ? 256 : p.D); d0 += 256) {
    int dd[NC];
    float xv[S][NC], v[NC], ev[NC], iv[NC];
#pragma unroll
    for (int u = 0; u < NC; ++u) {
      dd[u] = min(d0 + 256 * u, p.D - 1);
#pragma unroll
      for (int a = 0; a < S; ++a) xv[a][u] = p.xs[a * plane + row + dd[u]];
      ev[u] = p.extra ? p.extra[row + dd[u]] : 0.f;
      iv[u] = p.ident ? p.ident[row + dd[u]] : 0.f;
      v[u] = 0.f;
    }
    float wid = 0.f;  // identity experts pool into one weight on `ident`
#pragma unroll 4
    for (int c = 0; c < nsum; ++c) {
      const size_t r = (size_t)m * nsum + c;
      const float w = p.row_w ? p.row_w[r] : 1.f;
      const bool real = !p.row_expert || p.row_expert[r] < p.n_real;
      float yv[NC];
#pragma unroll
      for (int u = 0; u < NC; ++u) yv[u] = p.y[r * p.D + dd[u]];
#pragma unroll
      for (int u = 0; u < NC; ++u) v[u] += real ? w * yv[u] : 0.f;  // (an identity row's y holds nothing: selected away)
      wid += real ? 0.f : w;
    }
#pragma unroll
    for (int u = 0; u < NC; ++u) {
      const float val = fmaf(wid, iv[u], v[u]) + ev[u];
      float un = 0.f;
#pragma unroll
      for (int t = 0; t < S; ++t) {
        float nv = xv[t][u];
        if (p.mix) {
          nv = outw[t] * val;
#pragma unroll
          for (int a = 0; a < S; ++a) nv = fmaf(mixv[a][t], xv[a][u], nv);
        }
        un = fmaf(inw[t], nv, un);
        if (p.mix && d0 + 256 * u < p.D) p.xs[t * plane + row + dd[u]] = nv;
      }
      if (p.next_in && d0 + 256 * u < p.D) p.u[row + dd[u]] = un;
    }
  }
}

int hy_hc_update(const HyperUpdate& p, hipStream_t s) {
  if (p.S < 1 || p.S > 16 || p.M < 0 || p.D < 1 || !p.xs) return -1;
  if (p.mix && (!p.out_w || !p.y || p.nsum < 1)) return -2;
  if (p.mix && p.row_expert && (!p.row_w || !p.ident)) return -3;
  if ((p.next_in != nullptr) != (p.u != nullptr) || (!p.mix && !p.next_in)) return -4;
  if (p.M == 0) return 0;
  const int nu = (p.D + 255) / 256;
  switch (p.S) {
#define HC_CASE(N)                                                                \
  case N:                                                                         \
    if (nu <= 1) hc_update_kernel<N, 1><<<p.M, 256, 0, s>>>(p);                   \
    else if (nu <= 2) hc_update_kernel<N, 2><<<p.M, 256, 0, s>>>(p);              \
    else if (nu <= 4) hc_update_kernel<N, 4><<<p.M, 256, 0, s>>>(p);              \
    else if (nu <= 8 && N <= 4) hc_update_kernel<N, 8><<<p.M, 256, 0, s>>>(p);    \
    else hc_update_kernel<N, 0><<<p.M, 256, 0, s>>>(p);                           \
    break
    HC_CASE(1); HC_CASE(2); HC_CASE(3); HC_CASE(4); HC_CASE(5); HC_CASE(6); HC_CASE(7); HC_CASE(8);
#undef HC_CASE
#define HC_WIDE(N) case N: hc_update_kernel<N, 0><<<p.M, 256, 0, s>>>(p); break  // (many streams: a column at a time)
    HC_WIDE(9); HC_WIDE(10); HC_WIDE(11); HC_WIDE(12); HC_WIDE(13); HC_WIDE(14); HC_WIDE(15); HC_WIDE(16);
#undef HC_WIDE
  }
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
