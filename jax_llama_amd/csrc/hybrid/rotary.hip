// Rotary positions in the "halves" layout: within a head, number i pairs with number i + half, and the pair (u, v) at
// position p becomes (u cos a - v sin a, v cos a + u sin a), a = p * freq[i]. The angle is formed and reduced to
// [-pi, pi] in 64-bit (a position in the thousands times a frequency near 1 would lose the low bits of a 32-bit angle),
// sine and cosine of the reduced angle are 32-bit.
//
//   hy_rope_prep    : the step after a fused q | k | v projection: bias per column, q and k heads rotated on their first
//                     2 qk_half numbers, optionally v heads rotated over 2 v_half numbers, q to a dense buffer, k / v into
//                     the caches at slot + s.
//   hy_rotate_heads : every head of a [M, H * n] activation rotated by sign * position and scaled (the inverse turn of
//                     an attention output whose values were cached rotated), written to a column slice. The rotated
//                     numbers may start at an offset within the head and may pair up as (2i, 2i + 1) instead (the
//                     interleaved layout: the rotated tail of a latent attention's queries, in place).
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

JLA_DEV void ro_sincos(int pos, double freq, float sign, float* s, float* c) {
  const double a = (double)pos * freq;
  const double r = a - 6.283185307179586476925 * rint(a * 0.159154943091895335769);
  sincosf((float)r, s, c);
  *s *= sign;
}

JLA_DEV void ro_st(float* p, float v) { *p = v; }
JLA_DEV void ro_st(bf16_t* p, float v) { *p = f2bf(v); }

// grid (M, ceil((H + 2G) / 4)), 4 waves: wave -> item: [0, H) q heads, [H, H + G) k heads, [H + G, H + 2G) v heads
template <typename CT>
__global__ void __launch_bounds__(256) rope_prep_kernel(RopePrep p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.x, item = blockIdx.y * 4 + wave;
  if (item >= p.H + 2 * p.G) return;
  const int b = m / p.S, sidx = m - b * p.S;
  int kind, head, len, col, half;
  const double* freq;
  if (item < p.H) { kind = 0; head = item; len = p.dim; col = head * p.dim; half = p.qk_half; freq = p.qk_freq; }
  else if (item < p.H + p.G) {
    kind = 1; head = item - p.H; len = p.dim; col = (p.H + head) * p.dim; half = p.qk_half; freq = p.qk_freq;
  } else {
    kind = 2; head = item - p.H - p.G; len = p.vdim; col = (p.H + p.G) * p.dim + head * p.vdim;
    half = p.v_freq ? p.v_half : 0; freq = p.v_freq;
  }
  const float* row = p.proj + (size_t)m * p.ld + col;
  const float* bias = p.bias ? p.bias + col : nullptr;
  const int pos = p.positions[m];
  const int t = *p.slot + sidx;
  if (kind != 0 && (t < 0 || t >= p.T)) return;  // cache full: the write is dropped
  float* qd = p.q + ((size_t)m * p.H + head) * p.dim;
  CT* cd = kind == 0 ? nullptr
                     : (kind == 1 ? reinterpret_cast<CT*>(p.kc) : reinterpret_cast<CT*>(p.vc)) +
                           (((size_t)b * p.G + head) * p.T + t) * len;
  for (int i = lane; i < half; i += 64) {
    float sn, cs;
    ro_sincos(pos, freq[i], 1.f, &sn, &cs);
    const float u = row[i] + (bias ? bias[i] : 0.f), v = row[i + half] + (bias ? bias[i + half] : 0.f);
    const float a = u * cs - v * sn, c = v * cs + u * sn;
    if (kind == 0) { qd[i] = a; qd[i + half] = c; }
    else { ro_st(cd + i, a); ro_st(cd + i + half, c); }
  }
  for (int d = 2 * half + lane; d < len; d += 64) {
    const float v = row[d] + (bias ? bias[d] : 0.f);
    if (kind == 0) qd[d] = v;
    else ro_st(cd + d, v);
  }
}

int hy_rope_prep(const RopePrep& p, hipStream_t s) {
  if (p.B < 0 || p.S < 1 || p.H < 1 || p.G < 1 || p.H % p.G || p.dim < 1 || p.vdim < 1 || p.T < 1) return -1;
  if (p.qk_half < 0 || 2 * p.qk_half > p.dim || (p.qk_half > 0 && !p.qk_freq)) return -2;
  if (p.v_freq && (p.v_half < 0 || 2 * p.v_half > p.vdim)) return -2;
  if (p.ld < (p.H + p.G) * p.dim + p.G * p.vdim) return -3;
  const int M = p.B * p.S;
  if (M == 0) return 0;
  const int items = p.H + 2 * p.G;
  if ((items + 3) / 4 > 65535) return -4;
  dim3 grid(M, (items + 3) / 4);
  if (p.cbf16) rope_prep_kernel<bf16_t><<<grid, 256, 0, s>>>(p);
  else rope_prep_kernel<float><<<grid, 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

// grid (M, ceil(H / 4)), one wave per (token, head)
__global__ void __launch_bounds__(256) rotate_heads_kernel(const float* a, int lda,
                                                           const int32_t* __restrict__ positions,
                                                           const double* __restrict__ freq, int half, int H, int n,
                                                           float sign, float gain, float* out, int ldo,
                                                           int offset, int interleaved) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.x, h = blockIdx.y * 4 + wave;
  if (h >= H) return;
  // (out may be a: a thread reads both numbers of its pair before it writes them, and no two threads share a number)
  const float* src = a + (size_t)m * lda + (size_t)h * n;
  float* dst = out + (size_t)m * ldo + (size_t)h * n;
  const int pos = half > 0 ? positions[m] : 0;
  for (int i = lane; i < half; i += 64) {
    float sn, cs;
    ro_sincos(pos, freq[i], sign, &sn, &cs);
    const int iu = offset + (interleaved ? 2 * i : i), iv = offset + (interleaved ? 2 * i + 1 : i + half);
    const float u = src[iu], v = src[iv];
    dst[iu] = (u * cs - v * sn) * gain;
    dst[iv] = (v * cs + u * sn) * gain;
  }
  if (src != dst || gain != 1.f) {
    for (int d = lane; d < offset; d += 64) dst[d] = src[d] * gain;
    for (int d = offset + 2 * half + lane; d < n; d += 64) dst[d] = src[d] * gain;
  }
}

int hy_rotate_heads(const float* a, int lda, const int32_t* positions, const double* freq, int half, int M, int H, int n,
                    float sign, float gain, float* out, int ldo, int offset, int interleaved, hipStream_t s) {
  if (M < 0 || H < 1 || n < 1 || lda < H * n || ldo < H * n) return -1;
  if (half < 0 || offset < 0 || offset + 2 * half > n || (half > 0 && !freq)) return -2;
  if (M == 0) return 0;
  if ((H + 3) / 4 > 65535) return -4;
  rotate_heads_kernel<<<dim3(M, (H + 3) / 4), 256, 0, s>>>(a, lda, positions, freq, half, H, n, sign, gain, out, ldo,
                                                             offset, interleaved);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
