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
//   hy_conv_state_update : the carried tail <- the last taps - 1 inputs of every channel (after hy_delta_prep; a
//                          one-token step does it inside hy_delta_prep and launches nothing here).
//   hy_delta_scan        : the recurrence, token by token. A thread owns 16 key rows of one value column in registers;
//                          the lanes sharing a column (dim / 16 of them, adjacent) combine their partial S^T k and
//                          S^T q by lane exchange. k, q, v, g, beta of the next tokens are staged through LDS.
//   hy_gated_rmsnorm     : o / rms(o) * w * act(gate) per head (silu or sigmoid; the gain per column or per head and
//                          column; optionally o first divided by its own normaliser column).
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
    if (p.S == 1 && p.taps > 1) {  // one token: this lane is the channel's only reader, so it advances the tail itself
      const int C = 2 * p.G * p.dim + p.H * p.vdim, n = p.taps - 1;
      float* st = p.conv_state + ((size_t)b * C + c) * n;
      for (int i = 0; i + 1 < n; ++i) st[i] = st[i + 1];
      st[n - 1] = p.proj[(size_t)m * p.ld + c];
    }
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
  if (p.B == 0 || p.taps == 1 || p.S == 1) return 0;  // (S = 1: hy_delta_prep advanced the tail itself)
  const long long n = (long long)p.B * (2 * p.G * p.dim + p.H * p.vdim);
  conv_state_update_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

constexpr int DS_SLICE = 16;    // key rows per thread
constexpr int DS_PITCH = 20;    // floats between the staged slices of k / q: the lanes' 16-byte reads fall on distinct banks
constexpr int DS_STAGE = 4096;  // floats of one staged chunk of tokens (k, q, v, decay, beta) in LDS
constexpr int DS_PF = DS_STAGE / 256;

// Staged element i of the chunk starting at token s0: per token [k (dimp) | q (dimp) | v (cols) | decay | beta | pad],
// dimp = R slices of DS_PITCH floats (16 values + 4 pad; zeros past dim), cols = the block's value columns
// [j0, j0 + cols).
JLA_DEV float ds_src(const DeltaScan& p, int b, int h, int kh, int s0, int j0, int cols, int dimp, int per,
                     unsigned per_magic, int i) {
  const int t = (int)__umulhi((unsigned)i, per_magic), e = i - t * per;  // i / per (exact for i < 2^16)
  const size_t m = (size_t)b * p.S + s0 + t;
  if (e < 2 * dimp) {
    const int ee = e < dimp ? e : e - dimp;
    const int sl = ee / DS_PITCH, w = ee - sl * DS_PITCH, d = sl * DS_SLICE + w;
    if (w >= DS_SLICE || d >= p.dim) return 0.f;
    return (e < dimp ? p.kn : p.qn)[(m * p.G + kh) * p.dim + d];
  }
  if (e < 2 * dimp + cols) return p.v[(m * p.H + h) * p.vdim + min(j0 + e - 2 * dimp, p.vdim - 1)];
  if (e == 2 * dimp + cols) return p.decay[m * p.H + h];
  if (e == 2 * dimp + cols + 1) return p.beta[m * p.H + h];
  return 0.f;
}

// Sum over the R adjacent lanes that share a column (R a power of two); DPP moves up to 16 lanes.
JLA_DEV float ds_group_sum(float v, int R) {
  if (R >= 2) v += dppf<0xB1>(v);
  if (R >= 4) v += dppf<0x4E>(v);
  if (R >= 8) v += dppf<0x141>(v);
  if (R >= 16) v += dppf<0x140>(v);
  if (R >= 32) v += __shfl_xor(v, 16, 64);
  if (R >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// grid (ceil(vdim * R / 256), H, B); thread -> (column j = t / R, slice r = t % R), R = lanes per column (power of 2).
// The tokens' k, q, v, decay and beta are staged ct tokens at a time through LDS (the next chunk's global loads are in
// flight while the current chunk's steps run), so a step's operands cost LDS latency, not a trip to memory.
__global__ void __launch_bounds__(256) delta_scan_kernel(DeltaScan p, int R, int ct, int per, unsigned per_magic) {
  __shared__ __attribute__((aligned(16))) float stage[DS_STAGE];
  const int tid = threadIdx.x;
  const int t = blockIdx.x * 256 + tid;
  const int h = blockIdx.y, b = blockIdx.z;
  const int j = t / R, r = t - j * R;
  const bool live = j < p.vdim;  // (dead threads still join the lane exchanges)
  const int jc = live ? j : 0;
  const int kh = h / (p.H / p.G);
  const int i0 = r * DS_SLICE;
  const int j0 = blockIdx.x * (256 / R), cols = 256 / R, jl = j - j0;
  const int dimp = R * DS_PITCH;
  float S[DS_SLICE];
  float* sp = p.state + (((size_t)b * p.H + h) * p.dim) * p.vdim + jc;
#pragma unroll
  for (int i = 0; i < DS_SLICE; ++i) S[i] = (live && i0 + i < p.dim) ? sp[(size_t)(i0 + i) * p.vdim] : 0.f;
  float pf[DS_PF];
  {
    const int n = min(ct, p.S) * per;  // first chunk
#pragma unroll
    for (int u = 0; u < DS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < n) stage[i] = ds_src(p, b, h, kh, 0, j0, cols, dimp, per, per_magic, i);
    }
  }
  __syncthreads();
  for (int s0 = 0; s0 < p.S; s0 += ct) {
    const int nt = min(ct, p.S - s0);
    const int nn = min(ct, max(p.S - s0 - ct, 0)) * per;  // next chunk's floats
#pragma unroll
    for (int u = 0; u < DS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < nn) pf[u] = ds_src(p, b, h, kh, s0 + ct, j0, cols, dimp, per, per_magic, i);
    }
    for (int tt = 0; tt < nt; ++tt) {
      const float* row = stage + tt * per;
      const float4* k4 = reinterpret_cast<const float4*>(row + r * DS_PITCH);
      const float4* q4 = reinterpret_cast<const float4*>(row + dimp + r * DS_PITCH);
      const float v = row[2 * dimp + jl], g = row[2 * dimp + cols], beta = row[2 * dimp + cols + 1];
      float kv[DS_SLICE], qv[DS_SLICE], sk0 = 0.f, sk1 = 0.f;
#pragma unroll
      for (int i = 0; i < DS_SLICE; i += 4) {
        const float4 a = k4[i >> 2], c = q4[i >> 2];
        kv[i] = a.x; kv[i + 1] = a.y; kv[i + 2] = a.z; kv[i + 3] = a.w;
        qv[i] = c.x; qv[i + 1] = c.y; qv[i + 2] = c.z; qv[i + 3] = c.w;
      }
#pragma unroll
      for (int i = 0; i < DS_SLICE; i += 2) {
        S[i] *= g;
        S[i + 1] *= g;
        sk0 = fmaf(S[i], kv[i], sk0);
        sk1 = fmaf(S[i + 1], kv[i + 1], sk1);
      }
      const float sk = ds_group_sum(sk0 + sk1, R);
      const float u = beta * (v - sk);
      float oq0 = 0.f, oq1 = 0.f;
#pragma unroll
      for (int i = 0; i < DS_SLICE; i += 2) {
        S[i] = fmaf(kv[i], u, S[i]);
        S[i + 1] = fmaf(kv[i + 1], u, S[i + 1]);
        oq0 = fmaf(S[i], qv[i], oq0);
        oq1 = fmaf(S[i + 1], qv[i + 1], oq1);
      }
      const float oq = ds_group_sum(oq0 + oq1, R);
      if (live && r == 0) p.o[(((size_t)b * p.S + s0 + tt) * p.H + h) * p.vdim + j] = oq;
    }
    __syncthreads();  // every thread is done reading the chunk
#pragma unroll
    for (int u = 0; u < DS_PF; ++u) {
      const int i = tid + 256 * u;
      if (i < nn) stage[i] = pf[u];
    }
    __syncthreads();
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
  const int per = (2 * R * DS_PITCH + 256 / R + 2 + 3) / 4 * 4;
  if (per > DS_STAGE) return -4;
  const int ct = DS_STAGE / per < 32 ? DS_STAGE / per : 32;
  const long long threads = (long long)p.vdim * R;
  const unsigned per_magic = (unsigned)((0x100000000ull + per - 1) / per);  // ceil(2^32 / per)
  delta_scan_kernel<<<dim3((unsigned)((threads + 255) / 256), p.H, p.B), 256, 0, s>>>(p, R, ct, per, per_magic);
  JLA_CHECK_LAUNCH();
  return 0;
}

// grid (M, ceil(H / 4)), one wave per (token, head)
__global__ void __launch_bounds__(256) gated_rmsnorm_kernel(GatedNorm p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.x, h = blockIdx.y * 4 + wave;
  if (h >= p.H) return;
  const int vdim = p.vdim, ov = p.denom_floor ? vdim + 1 : vdim;
  const float* x = p.o + ((size_t)m * p.H + h) * ov;
  float pre = 1.f;  // the read-out's own normaliser, applied before the statistic
  if (p.denom_floor) pre = 1.f / (fmaxf(fabsf(x[vdim]), p.denom_floor[(size_t)m * p.H + h]) + 1e-6f);
  float ss = 0.f;
  for (int d = lane; d < vdim; d += 64) {
    const float v = x[d] * pre;
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float sc = 1.f / sqrtf(ss / (float)vdim + p.eps);
  const float* gr = p.gate + (size_t)m * p.ldg + (size_t)h * vdim;
  const float* w = p.w + (p.w_heads ? (size_t)h * vdim : 0);
  float* dst = p.out + (size_t)m * p.ldo + (size_t)h * vdim;
  for (int d = lane; d < vdim; d += 64) {
    const float g = p.gate_act == 1 ? hy_sigmoid(gr[d]) : hy_silu(gr[d]);
    dst[d] = (x[d] * pre) * sc * w[d] * g * p.gain;
  }
}

int hy_gated_rmsnorm(const GatedNorm& p, hipStream_t s) {
  if (p.M < 0 || p.H < 1 || p.vdim < 1 || p.ldg < p.H * p.vdim || p.ldo < p.H * p.vdim) return -1;
  if (p.gate_act != 0 && p.gate_act != 1) return -3;
  if (p.M == 0) return 0;
  if ((p.H + 3) / 4 > 65535) return -2;
  gated_rmsnorm_kernel<<<dim3(p.M, (p.H + 3) / 4), 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
