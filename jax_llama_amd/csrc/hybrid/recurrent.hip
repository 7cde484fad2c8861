// Linear recurrences over a carried fp32 matrix state, and what feeds them. fp32 throughout.
//
//   hy_token_shift : blends of every token's row with the row before it, one blend vector per consumer; the row before
//                    a call's first token is carried per sequence.
//   hy_mlstm_prep  : capped exponential gates and their running maximum m_t = max(f_t + m_(t-1), a_t) (exactly that
//                    chain, in order: the stabiliser enters the read-out through a floor, so it is not re-associated),
//                    giving per (token, head) the state's keep factor, the write factor and the floor exp(-m_t). One
//                    wave per (row, head): 64 tokens' gates are computed lane-parallel, the chain runs over their
//                    values as wave-uniform scalars.
//   hy_lin_scan    : S <- D_t S + b_t k_t v_t^T with the read-out after the write (scalar D, b: the exponential-gate
//                    memory; its normaliser is one more value column whose value is 1) or before it with a bonus for the
//                    current token (per-channel D from a double exponential: the time-mix memory). Thread layout of the
//                    delta-rule scan: a thread owns 16 key rows of one state column in registers, the lanes of a column
//                    combine their partial read-outs by lane exchange, tokens are staged through LDS a chunk at a time
//                    with the next chunk's loads in flight.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

// grid (M), 256 threads
__global__ void __launch_bounds__(256) token_shift_kernel(const float* __restrict__ h, float* prev,
                                                          const float* __restrict__ mu, int n, float* __restrict__ out,
                                                          int S, int D, size_t MD) {
  const int m = blockIdx.x;
  const int b = m / S, s = m - b * S;
  const float* cur = h + (size_t)m * D;
  const float* before = s == 0 ? prev + (size_t)b * D : cur - D;
  const float* last = h + ((size_t)b * S + S - 1) * D;
  for (int d = threadIdx.x; d < D; d += 256) {
    const float c = cur[d], diff = before[d] - c;
    for (int i = 0; i < n; ++i) out[(size_t)i * MD + (size_t)m * D + d] = fmaf(diff, mu[(size_t)i * D + d], c);
    if (s == 0) prev[(size_t)b * D + d] = last[d];  // (this thread was the only reader of prev[b, d])
  }
}

int hy_token_shift(const float* h, float* prev, const float* mu, int n, float* out, int B, int S, int D, hipStream_t s) {
  if (B < 0 || S < 1 || D < 1 || n < 1) return -1;
  if (B == 0) return 0;
  const long long M = (long long)B * S;
  if (M > 0x7fffffffLL) return -2;
  token_shift_kernel<<<(unsigned)M, 256, 0, s>>>(h, prev, mu, n, out, S, D, (size_t)M * D);
  JLA_CHECK_LAUNCH();
  return 0;
}

JLA_DEV float rc_uniform(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
JLA_DEV float rc_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// grid (H, B), one wave
__global__ void __launch_bounds__(64) mlstm_prep_kernel(MlstmPrep p) {
  const int lane = threadIdx.x, h = blockIdx.x, b = blockIdx.y;
  const float bi = p.gate_bias[h], bf = p.gate_bias[p.H + h];
  const float inv_cap = 1.f / p.cap;
  float m = p.mstate[(size_t)b * p.H + h];
  for (int t0 = 0; t0 < p.S; t0 += 64) {
    const int t = t0 + lane;
    const bool on = t < p.S;
    const size_t row = (size_t)b * p.S + (on ? t : p.S - 1);
    const float xi = p.proj[row * p.ld + p.col_i + h], xf = p.proj[row * p.ld + p.col_f + h];
    // (a token past the end keeps m: f = 0, a = -inf)
    const float a = on ? p.cap * tanhf((xi + bi) * inv_cap) : -INFINITY;
    const float f = on ? rc_logsigmoid(p.cap * tanhf((xf + bf) * inv_cap)) : 0.f;
    float m_before = 0.f, m_after = 0.f;
#pragma unroll
    for (int l = 0; l < 64; ++l) {
      const float mn = fmaxf(rc_uniform(f, l) + m, rc_uniform(a, l));
      if (lane == l) {
        m_before = m;
        m_after = mn;
      }
      m = mn;
    }
    if (on) {
      const size_t o = row * p.H + h;
      p.keep[o] = expf(f + m_before - m_after);
      p.write[o] = expf(a - m_after);
      p.floor[o] = expf(-m_after);
    }
  }
  if (lane == 0) p.mstate[(size_t)b * p.H + h] = m;
}

int hy_mlstm_prep(const MlstmPrep& p, hipStream_t s) {
  if (p.B < 0 || p.S < 1 || p.H < 1 || !(p.cap > 0.f)) return -1;
  if (p.col_i < 0 || p.col_f < 0 || p.col_i + p.H > p.ld || p.col_f + p.H > p.ld) return -2;
  if (p.B == 0) return 0;
  if (p.B > 65535) return -3;
  mlstm_prep_kernel<<<dim3(p.H, p.B), 64, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

constexpr int LS_SLICE = 16;    // key rows per thread
constexpr int LS_PITCH = 20;    // floats between the staged slices: the lanes' 16-byte reads fall on distinct banks
constexpr int LS_STAGE = 4096;  // floats of one staged chunk of tokens in LDS
constexpr int LS_PF = LS_STAGE / 256;

// Staged element i of the chunk starting at token s0. Per token: [k (dimp) | q (dimp) | MODE 1: decay (dimp) |
// v (cols) | MODE 0: keep, write | pad]; dimp = R slices of LS_PITCH floats (16 values + 4 pad; zeros past dim), cols =
// the block's state columns [j0, j0 + cols).
template <int MODE>
JLA_DEV float ls_src(const LinScan& p, int b, int h, int s0, int j0, int cols, int dimp, int per, unsigned per_magic,
                     int i) {
  const int t = (int)__umulhi((unsigned)i, per_magic), e = i - t * per;  // i / per (exact for i < 2^16)
  const size_t m = (size_t)b * p.S + s0 + t;
  constexpr int NV = MODE == 1 ? 3 : 2;  // staged vectors over the key rows
  if (e < NV * dimp) {
    const int which = e / dimp, ee = e - which * dimp;
    const int sl = ee / LS_PITCH, w = ee - sl * LS_PITCH, d = sl * LS_SLICE + w;
    if (w >= LS_SLICE || d >= p.dim) return 0.f;
    if (which == 0) return p.k[m * p.ldk + (size_t)h * p.dim + d];
    if (which == 1) return p.q[m * p.ldq + (size_t)h * p.dim + d] * p.q_scale;
    return expf(-expf(p.decay[m * p.ldd + (size_t)h * p.dim + d] + p.w0[(size_t)h * p.dim + d]));
  }
  const int c = e - NV * dimp;
  if (c < cols) {
    const int j = j0 + c;
    if (MODE == 0 && j >= p.vdim) return 1.f;  // the normaliser's column (and surplus columns, never stored)
    return p.v[m * p.ldv + (size_t)h * p.vdim + min(j, p.vdim - 1)];
  }
  if (MODE == 0 && c == cols) return p.decay[m * p.H + h];
  if (MODE == 0 && c == cols + 1) return p.write[m * p.H + h];
  return 0.f;
}

// Sum over the R adjacent lanes that share a column (R a power of two); DPP moves up to 16 lanes.
JLA_DEV float ls_group_sum(float v, int R) {
  if (R >= 2) v += dppf<0xB1>(v);
  if (R >= 4) v += dppf<0x4E>(v);
  if (R >= 8) v += dppf<0x141>(v);
  if (R >= 16) v += dppf<0x140>(v);
  if (R >= 32) v += __shfl_xor(v, 16, 64);
  if (R >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// grid (ceil(ncols * R / 256), H, B); thread -> (column j = t / R, slice r = t % R), R = lanes per column (power of 2)
template <int MODE>
__global__ void __launch_bounds__(256) lin_scan_kernel(LinScan p, int R, int ct, int per, unsigned per_magic) {
  __shared__ __attribute__((aligned(16))) float stage[LS_STAGE];
  const int ncols = MODE == 0 ? p.vdim + 1 : p.vdim;
  const int tid = threadIdx.x;
  const int t = blockIdx.x * 256 + tid;
  const int h = blockIdx.y, b = blockIdx.z;
  const int j = t / R, r = t - j * R;
  const bool live = j < ncols;  // (dead threads still join the lane exchanges)
  const int jc = live ? j : 0;
  const int i0 = r * LS_SLICE;
  const int j0 = blockIdx.x * (256 / R), cols = 256 / R, jl = j - j0;
  const int dimp = R * LS_PITCH;
  constexpr int NV = MODE == 1 ? 3 : 2;
  float S[LS_SLICE], uu[LS_SLICE];
  float* sp = p.state + (((size_t)b * p.H + h) * p.dim) * ncols + jc;
#pragma unroll
  for (int i = 0; i < LS_SLICE; ++i) {
    const bool in = i0 + i < p.dim;
    S[i] = (live && in) ? sp[(size_t)(i0 + i) * ncols] : 0.f;
    uu[i] = (MODE == 1 && in) ? p.u[(size_t)h * p.dim + i0 + i] : 0.f;
  }
  float pf[LS_PF];
  {
    const int n = min(ct, p.S) * per;  // first chunk
#pragma unroll
    for (int u = 0; u < LS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < n) stage[i] = ls_src<MODE>(p, b, h, 0, j0, cols, dimp, per, per_magic, i);
    }
  }
  __syncthreads();
  for (int s0 = 0; s0 < p.S; s0 += ct) {
    const int nt = min(ct, p.S - s0);
    const int nn = min(ct, max(p.S - s0 - ct, 0)) * per;  // next chunk's floats
#pragma unroll
    for (int u = 0; u < LS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < nn) pf[u] = ls_src<MODE>(p, b, h, s0 + ct, j0, cols, dimp, per, per_magic, i);
    }
    for (int tt = 0; tt < nt; ++tt) {
      const float* row = stage + tt * per;
      const float4* k4 = reinterpret_cast<const float4*>(row + r * LS_PITCH);
      const float4* q4 = reinterpret_cast<const float4*>(row + dimp + r * LS_PITCH);
      const float v = row[NV * dimp + jl];
      float kv[LS_SLICE], qv[LS_SLICE];
#pragma unroll
      for (int i = 0; i < LS_SLICE; i += 4) {
        const float4 a = k4[i >> 2], c = q4[i >> 2];
        kv[i] = a.x; kv[i + 1] = a.y; kv[i + 2] = a.z; kv[i + 3] = a.w;
        qv[i] = c.x; qv[i + 1] = c.y; qv[i + 2] = c.z; qv[i + 3] = c.w;
      }
      float o0 = 0.f, o1 = 0.f;
      if (MODE == 0) {
        const float keep = row[NV * dimp + cols], wv = row[NV * dimp + cols + 1] * v;
#pragma unroll
        for (int i = 0; i < LS_SLICE; i += 2) {
          S[i] = fmaf(keep, S[i], kv[i] * wv);
          S[i + 1] = fmaf(keep, S[i + 1], kv[i + 1] * wv);
          o0 = fmaf(S[i], qv[i], o0);
          o1 = fmaf(S[i + 1], qv[i + 1], o1);
        }
      } else {
        const float4* d4 = reinterpret_cast<const float4*>(row + 2 * dimp + r * LS_PITCH);
        float dv[LS_SLICE], b0 = 0.f, b1 = 0.f;
#pragma unroll
        for (int i = 0; i < LS_SLICE; i += 4) {
          const float4 a = d4[i >> 2];
          dv[i] = a.x; dv[i + 1] = a.y; dv[i + 2] = a.z; dv[i + 3] = a.w;
        }
#pragma unroll
        for (int i = 0; i < LS_SLICE; i += 2) {
          o0 = fmaf(S[i], qv[i], o0);
          o1 = fmaf(S[i + 1], qv[i + 1], o1);
          b0 = fmaf(uu[i] * kv[i], qv[i], b0);
          b1 = fmaf(uu[i + 1] * kv[i + 1], qv[i + 1], b1);
          S[i] = fmaf(dv[i], S[i], kv[i] * v);
          S[i + 1] = fmaf(dv[i + 1], S[i + 1], kv[i + 1] * v);
        }
        o0 = fmaf(b0 + b1, v, o0);
      }
      const float oq = ls_group_sum(o0 + o1, R);
      if (live && r == 0) p.o[(((size_t)b * p.S + s0 + tt) * p.H + h) * ncols + j] = oq;
    }
    __syncthreads();  // every thread is done reading the chunk
#pragma unroll
    for (int u = 0; u < LS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < nn) stage[i] = pf[u];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < LS_SLICE; ++i)
    if (live && i0 + i < p.dim) sp[(size_t)(i0 + i) * ncols] = S[i];
}

int hy_lin_scan(const LinScan& p, hipStream_t s) {
  if (p.mode != 0 && p.mode != 1) return -1;
  if (p.B < 0 || p.S < 1 || p.H < 1 || p.dim < 1 || p.vdim < 1) return -1;
  if (p.dim > 64 * LS_SLICE) return -2;
  if (p.ldq < p.H * p.dim || p.ldk < p.H * p.dim || p.ldv < p.H * p.vdim) return -5;
  if (p.mode == 1 && (p.ldd < p.H * p.dim || !p.w0 || !p.u)) return -6;
  if (p.mode == 0 && !p.write) return -6;
  if (p.B == 0) return 0;
  if (p.H > 65535 || p.B > 65535) return -3;
  int R = 1;
  while (R * LS_SLICE < p.dim) R <<= 1;
  const int nv = p.mode == 1 ? 3 : 2;
  const int per = (nv * R * LS_PITCH + 256 / R + 2 + 3) / 4 * 4;
  if (per > LS_STAGE) return -4;
  const int ct = LS_STAGE / per < 32 ? LS_STAGE / per : 32;
  const long long threads = (long long)(p.mode == 0 ? p.vdim + 1 : p.vdim) * R;
  const unsigned per_magic = (unsigned)((0x100000000ull + per - 1) / per);  // ceil(2^32 / per)
  const dim3 grid((unsigned)((threads + 255) / 256), p.H, p.B);
  if (p.mode == 0) lin_scan_kernel<0><<<grid, 256, 0, s>>>(p, R, ct, per, per_magic);
  else lin_scan_kernel<1><<<grid, 256, 0, s>>>(p, R, ct, per, per_magic);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
