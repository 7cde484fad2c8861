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
//                    with the next chunk's loads in flight. A long sequence is cut into segments that run side by side
//                    (both recurrences are linear in the state): segment states and decay products, one combining
//                    walk, then the scan proper from every segment's incoming state.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

// grid (M, ceil(D / 256)), one thread per (token, column): a one-token step is one round trip, not D / 256 of them
__global__ void __launch_bounds__(256) token_shift_kernel(const float* __restrict__ h, float* prev,
                                                          const float* __restrict__ mu, int n, float* __restrict__ out,
                                                          int S, int D, size_t MD) {
  const int m = blockIdx.x, d = blockIdx.y * 256 + threadIdx.x;
  if (d >= D) return;
  const int b = m / S, s = m - b * S;
  const float* cur = h + (size_t)m * D;
  const float* before = s == 0 ? prev + (size_t)b * D : cur - D;
  const float c = cur[d], diff = before[d] - c;
  const float last = h[((size_t)b * S + S - 1) * D + d];
  for (int i = 0; i < n; ++i) out[(size_t)i * MD + (size_t)m * D + d] = fmaf(diff, mu[(size_t)i * D + d], c);
  if (s == 0) prev[(size_t)b * D + d] = last;  // (this thread was the only reader of prev[b, d])
}

int hy_token_shift(const float* h, float* prev, const float* mu, int n, float* out, int B, int S, int D, hipStream_t s) {
  if (B < 0 || S < 1 || D < 1 || n < 1) return -1;
  if (B == 0) return 0;
  const long long M = (long long)B * S;
  if (M > 0x7fffffffLL || (D + 255) / 256 > 65535) return -2;
  token_shift_kernel<<<dim3((unsigned)M, (D + 255) / 256), 256, 0, s>>>(h, prev, mu, n, out, S, D, (size_t)M * D);
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
  // this lane's gate pre-activations of the chunk at t0 (a lane past the end re-reads the last token)
  auto gates = [&](int t0, float& xi, float& xf) {
    const size_t row = (size_t)b * p.S + min(t0 + lane, p.S - 1);
    xi = p.proj[row * p.ld + p.col_i + h];
    xf = p.proj[row * p.ld + p.col_f + h];
  };
  float xi_next, xf_next;
  gates(0, xi_next, xf_next);
  for (int t0 = 0; t0 < p.S; t0 += 64) {
    const int t = t0 + lane;
    const bool on = t < p.S;
    const size_t row = (size_t)b * p.S + (on ? t : p.S - 1);
    const float xi = xi_next, xf = xf_next;
    if (t0 + 64 < p.S) gates(t0 + 64, xi_next, xf_next);  // (in flight behind this chunk's chain)
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
// Staging is split in three so that a thread's 16 loads of a chunk are all in flight together and cost a few
// instructions each: ls_plan decodes, once per kernel, what the thread's u-th staged element is (its source tensor, its
// offset inside a token's row, the token within the chunk, what becomes of the loaded number: none of that depends on
// the chunk); per chunk an address is then one multiply-add on a base chosen by selects (always a readable address, no
// branch); ls_val turns the loaded number into the staged one when the chunk is written to LDS, a chunk of token
// steps later.
enum { LS_ZERO = 0, LS_PLAIN = 1, LS_ONE = 2, LS_DECAY = 3, LS_QUERY = 4 };
enum { LS_SRC_K = 0, LS_SRC_Q = 1, LS_SRC_D = 2, LS_SRC_V = 3, LS_SRC_KEEP = 4, LS_SRC_WRITE = 5 };
struct LsPlan {
  int meta;  // code | source << 3 | token within the chunk << 6
  int off;   // offset inside the token's row of the source
};

template <int MODE>
JLA_DEV LsPlan ls_plan(const LinScan& p, int h, int j0, int cols, int dimp, int per, unsigned per_magic, int i) {
  constexpr int NV = MODE == 1 ? 3 : 2;  // staged vectors over the key rows
  const int t = (int)__umulhi((unsigned)i, per_magic), e = i - t * per;  // i / per (exact for i < 2^16)
  const bool vec = e < NV * dimp;
  const int which = vec ? e / dimp : 0, ee = vec ? e - which * dimp : 0;
  const int sl = ee / LS_PITCH, w = ee - sl * LS_PITCH, d = sl * LS_SLICE + w;
  const bool pad = w >= LS_SLICE || d >= p.dim;
  const int hd = h * p.dim + (pad ? 0 : d);
  const int c = e - NV * dimp, j = j0 + c;
  const bool is_v = !vec && c < cols, is_g = MODE == 0 && !vec && (c == cols || c == cols + 1);
  const int src = vec ? which : is_v ? LS_SRC_V : is_g ? (c == cols ? LS_SRC_KEEP : LS_SRC_WRITE) : LS_SRC_K;
  const int code = vec ? (pad ? LS_ZERO : which == 1 ? LS_QUERY : which == 2 ? LS_DECAY : LS_PLAIN)
                       : is_v ? ((MODE == 0 && j >= p.vdim) ? LS_ONE : LS_PLAIN)  // (the normaliser's column: value 1)
                              : is_g ? LS_PLAIN : LS_ZERO;
  LsPlan r;
  r.meta = code | src << 3 | t << 6;
  r.off = vec ? hd : is_v ? h * p.vdim + min(max(j, 0), p.vdim - 1) : is_g ? h : h * p.dim;
  return r;
}

template <int MODE>
JLA_DEV float ls_val(int code, float raw, float w0v, float q_scale) {
  if (MODE == 1 && code == LS_DECAY) return expf(-expf(raw + w0v));
  return code == LS_ZERO ? 0.f : code == LS_ONE ? 1.f : code == LS_QUERY ? raw * q_scale : raw;
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

// floats of one staged token, tokens per staged chunk
constexpr int ls_per(int mode, int R) { return ((mode == 1 ? 3 : 2) * R * LS_PITCH + 256 / R + 2 + 3) / 4 * 4; }
constexpr int ls_ct(int mode, int R) { return LS_STAGE / ls_per(mode, R) < 32 ? LS_STAGE / ls_per(mode, R) : 32; }

// grid (ceil(ncols * R / 256), H, B); thread -> (column j = t / R, slice r = t % R), R = lanes per column (a power of
// two, a template parameter: the staged layout, the chunk length and the lane exchange are then compile-time, which took
// a token step from about 200 instructions to what the state update and the read-out need)
//
// A long sequence is cut into nseg segments that run side by side (grid.z = B * nseg), in three launches: (1) STATE_ONLY:
// every segment from a zero state, no read-out, leaving its final state T and the product D of its decays; (2)
// lin_combine_kernel walks the segments once, S_in(p + 1) = D_p S_in(p) + T_p from the carried state, and stores the
// sequence's final state; (3) the full scan of every segment from its S_in. A token's arithmetic inside a segment is that
// of the one-launch form; the incoming state is a two-term sum instead of a running one.
template <int MODE, int R, int STATE_ONLY>
__global__ void __launch_bounds__(256) lin_scan_kernel(LinScan p, const float* s_init, float* s_final, float* seg_decay) {
  constexpr int per = ls_per(MODE, R), ct = ls_ct(MODE, R);
  constexpr unsigned per_magic = (unsigned)((0x100000000ull + per - 1) / per);  // ceil(2^32 / per)
  __shared__ __attribute__((aligned(16))) float stage[LS_STAGE];
  const int ncols = MODE == 0 ? p.vdim + 1 : p.vdim;
  const int tid = threadIdx.x;
  const int t = blockIdx.x * 256 + tid;
  const int h = blockIdx.y, b = blockIdx.z / p.nseg, seg = blockIdx.z - b * p.nseg;
  const int t_lo = seg * p.seg_len, t_hi = min(p.S, t_lo + p.seg_len);  // this block's tokens
  const int j = t / R, r = t - j * R;
  const bool live = j < ncols;  // (dead threads still join the lane exchanges)
  const int jc = live ? j : 0;
  const int i0 = r * LS_SLICE;
  constexpr int cols = 256 / R, dimp = R * LS_PITCH;
  const int j0 = blockIdx.x * cols, jl = j - j0;
  constexpr int NV = MODE == 1 ? 3 : 2;
  float S[LS_SLICE], uu[LS_SLICE], dprod[MODE == 1 ? LS_SLICE : 1];
  const size_t sidx = ((((size_t)b * p.nseg + seg) * p.H + h) * p.dim) * ncols + jc;  // (b, segment, head) of a state array
#pragma unroll
  for (int i = 0; i < LS_SLICE; ++i) {
    const bool in = i0 + i < p.dim;
    S[i] = (s_init && live && in) ? s_init[sidx + (size_t)(i0 + i) * ncols] : 0.f;
    uu[i] = (MODE == 1 && in) ? p.u[(size_t)h * p.dim + i0 + i] : 0.f;
    if (MODE == 1) dprod[i] = 1.f;
  }
  if (MODE == 0) dprod[0] = 1.f;
  float pf[LS_PF], pw[LS_PF];
  LsPlan plan[LS_PF];
#pragma unroll
  for (int u = 0; u < LS_PF; ++u) {
    plan[u] = ls_plan<MODE>(p, h, j0, cols, dimp, per, per_magic, tid + 256 * u);
    // (the decay's offset does not depend on the token: loaded once)
    pw[u] = (MODE == 1 && (plan[u].meta & 7) == LS_DECAY) ? p.w0[plan[u].off] : 0.f;
  }
  const size_t row0 = (size_t)b * p.S;
  // loads of the chunk at token sn (n floats of it): every thread issues all of its loads before any is used
  auto fetch = [&](int sn, int n) {
#pragma unroll
    for (int u = 0; u < LS_PF; ++u) {
      const int i = tid + 256 * u;
      const int src = (plan[u].meta >> 3) & 7;
      const size_t m = row0 + sn + (i < n ? plan[u].meta >> 6 : 0);  // (past the chunk: a row of it, never staged)
      const float* base = src == LS_SRC_K ? p.k : src == LS_SRC_Q ? p.q : src == LS_SRC_V ? p.v
                          : MODE == 1 ? p.decay : src == LS_SRC_KEEP ? p.decay : p.write;
      const int ld = src == LS_SRC_K ? p.ldk : src == LS_SRC_Q ? p.ldq : src == LS_SRC_V ? p.ldv : MODE == 1 ? p.ldd : p.H;
      pf[u] = base[m * ld + plan[u].off];
    }
  };
  auto put = [&](int n) {
#pragma unroll
    for (int u = 0; u < LS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < n) stage[i] = ls_val<MODE>(plan[u].meta & 7, pf[u], pw[u], p.q_scale);
    }
  };
  fetch(t_lo, min(ct, t_hi - t_lo) * per);
  put(min(ct, t_hi - t_lo) * per);
  __syncthreads();
  float* orow = p.o + (((size_t)b * p.S + t_lo) * p.H + h) * ncols + jc;  // this column's read-out of the next token
  const size_t ostride = (size_t)p.H * ncols;
  for (int s0 = t_lo; s0 < t_hi; s0 += ct) {
    const int nt = min(ct, t_hi - s0);
    const int nn = min(ct, max(t_hi - s0 - ct, 0)) * per;  // next chunk's floats
    if (nn > 0) fetch(s0 + ct, nn);
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
        if (STATE_ONLY) dprod[0] *= keep;
#pragma unroll
        for (int i = 0; i < LS_SLICE; i += 2) {
          S[i] = fmaf(keep, S[i], kv[i] * wv);
          S[i + 1] = fmaf(keep, S[i + 1], kv[i + 1] * wv);
          if (!STATE_ONLY) {
            o0 = fmaf(S[i], qv[i], o0);
            o1 = fmaf(S[i + 1], qv[i + 1], o1);
          }
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
          if (!STATE_ONLY) {
            o0 = fmaf(S[i], qv[i], o0);
            o1 = fmaf(S[i + 1], qv[i + 1], o1);
            b0 = fmaf(uu[i] * kv[i], qv[i], b0);
            b1 = fmaf(uu[i + 1] * kv[i + 1], qv[i + 1], b1);
          } else {
            dprod[i] *= dv[i];
            dprod[i + 1] *= dv[i + 1];
          }
          S[i] = fmaf(dv[i], S[i], kv[i] * v);
          S[i + 1] = fmaf(dv[i + 1], S[i + 1], kv[i + 1] * v);
        }
        o0 = fmaf(b0 + b1, v, o0);
      }
      if (!STATE_ONLY) {
        const float oq = ls_group_sum(o0 + o1, R);
        if (live && r == 0) *orow = oq;
        orow += ostride;
      }
    }
    __syncthreads();  // every thread is done reading the chunk
    put(nn);
    __syncthreads();
  }
  if (s_final) {
#pragma unroll
    for (int i = 0; i < LS_SLICE; ++i)
      if (live && i0 + i < p.dim) s_final[sidx + (size_t)(i0 + i) * ncols] = S[i];
  }
  if (STATE_ONLY && seg_decay && j == 0) {  // the segment's decay: one number per head, or one per key row
    const size_t d0 = ((size_t)b * p.nseg + seg) * p.H + h;
    if (MODE == 0) {
      if (r == 0) seg_decay[d0] = dprod[0];
    } else {
#pragma unroll
      for (int i = 0; i < LS_SLICE; ++i)
        if (i0 + i < p.dim) seg_decay[d0 * p.dim + i0 + i] = dprod[MODE == 1 ? i : 0];
    }
  }
}

// one thread per state element of a (row, head): on entry seg[b][s] holds segment s's own final state, on exit the
// state segment s starts from; state (the carried one) is advanced past the whole sequence
__global__ void __launch_bounds__(256) lin_combine_kernel(float* state, float* seg, const float* seg_decay, int nseg,
                                                          int H, int dim, int ncols, int per_row_decay, long long n) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;  // element of [B, H, dim, ncols]
  if (e >= n) return;
  const long long hsz = (long long)dim * ncols, bh = e / hsz, in = e - bh * hsz;
  const long long b = bh / H, h = bh - b * H;
  const int row = (int)(in / ncols);
  float S = state[e];
  for (int s = 0; s < nseg; ++s) {
    const long long at = ((b * nseg + s) * H + h) * hsz + in;
    const long long dh = (b * nseg + s) * H + h;
    const float d = seg_decay[per_row_decay ? dh * dim + row : dh], own = seg[at];
    seg[at] = S;
    S = fmaf(d, S, own);
  }
  state[e] = S;
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
  const long long threads = (long long)(p.mode == 0 ? p.vdim + 1 : p.vdim) * R;
  const int ncols = p.mode == 0 ? p.vdim + 1 : p.vdim;
  const bool cut = p.nseg > 1;
  if (cut && (!p.seg_state || !p.seg_decay || p.seg_len < 1 || (long long)p.nseg * p.seg_len < p.S ||
              (long long)(p.nseg - 1) * p.seg_len >= p.S))
    return -7;
  if (!cut && (p.nseg != 1 || p.seg_len < p.S)) return -7;
  if ((long long)p.B * p.nseg > 65535) return -3;
  const dim3 grid((unsigned)((threads + 255) / 256), p.H, p.B * p.nseg);
#define LS_LAUNCH(RR)                                                                                            \
  case RR:                                                                                                       \
    static_assert(ls_per(1, RR) <= LS_STAGE, "a staged token fits");                                             \
    if (!cut) {                                                                                                  \
      if (p.mode == 0) lin_scan_kernel<0, RR, 0><<<grid, 256, 0, s>>>(p, p.state, p.state, nullptr);             \
      else lin_scan_kernel<1, RR, 0><<<grid, 256, 0, s>>>(p, p.state, p.state, nullptr);                         \
    } else if (pass == 0) {                                                                                      \
      if (p.mode == 0) lin_scan_kernel<0, RR, 1><<<grid, 256, 0, s>>>(p, nullptr, p.seg_state, p.seg_decay);     \
      else lin_scan_kernel<1, RR, 1><<<grid, 256, 0, s>>>(p, nullptr, p.seg_state, p.seg_decay);                 \
    } else {                                                                                                     \
      if (p.mode == 0) lin_scan_kernel<0, RR, 0><<<grid, 256, 0, s>>>(p, p.seg_state, nullptr, nullptr);         \
      else lin_scan_kernel<1, RR, 0><<<grid, 256, 0, s>>>(p, p.seg_state, nullptr, nullptr);                     \
    }                                                                                                            \
    break
  for (int pass = 0; pass < (cut ? 2 : 1); ++pass) {
    switch (R) {
      LS_LAUNCH(1);
      LS_LAUNCH(2);
      LS_LAUNCH(4);
      LS_LAUNCH(8);
      LS_LAUNCH(16);
      LS_LAUNCH(32);
      LS_LAUNCH(64);
      default:
        return -4;
    }
    JLA_CHECK_LAUNCH();
    if (cut && pass == 0) {
      const long long n = (long long)p.B * p.H * p.dim * ncols;
      lin_combine_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p.state, p.seg_state, p.seg_decay, p.nseg, p.H, p.dim,
                                                                    ncols, p.mode == 1, n);
      JLA_CHECK_LAUNCH();
    }
  }
#undef LS_LAUNCH
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
