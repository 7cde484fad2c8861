// Attention with per-head RMS-normalised q / k / v, a position-dependent query temperature, a soft cap on the scores
// and a learned bias per key distance, over a per-layer cache of any head size (several layers may read one cache).
//
//   hy_attn_prep : from the fused projection output, per (token, head): divide q and k by their RMS over dim and v by
//                  its RMS over vdim, scale q by 1 + coef * ln(floor((p + 1) / every) + 1), write k / v into the
//                  cache at slot + s (bf16 or fp32), q to a dense fp32 buffer.
//   hy_attn_bias : scores, soft cap, distance bias, causal softmax and PV in fp32. One wave per query (prefill) walks
//                  its keys 64 at a time: a lane scores one key (q broadcast from LDS), the running maximum / sum are
//                  wave reductions, and the lanes then split the value columns. Decode (S = 1) splits the keys of a
//                  (row, head) over several waves whose partials a second kernel merges in split order.
// The bias table is indexed by distance (rows past the last repeat it), so any bucketing is a host-side table fill.
// An optional per-head sink adds exp(sink[h]) to the softmax denominator: the running maximum starts at the sink and
// the running sum at 1 (in decode, for the first key split only), so no kernel needs a branch per key for it.
// Block-local masks (chunk > 0): a query at slot i sees the keys of [floor(i / chunk) * chunk, i]; every kernel starts
// its key walk at that block's first slot, so the keys before it are never read. A per-head factor (head_scale) joins
// the score scale.
// Sliding windows (window > 0): a query at slot i sees the keys of [max(0, i - window + 1), i] and, with keep_first, the
// row's first keep_first slots. Every kernel numbers a query's visible keys 0 .. n - 1 (the kept first ones, then the
// window) and walks that numbering, so hidden keys are never read and the decode splits deal only visible keys; the MFMA
// kernel walks the kept tiles and then the window's tiles. A gate per (token, head) (sigmoid of a projection column)
// multiplies the normalised output in the kernels that write it. Values may be the leading columns of wider rows (ldv):
// a latent cache whose rows carry a rotated key part behind the latent serves as keys (whole row) and values (latent).
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

JLA_DEV float ab_ld(const float* p) { return *p; }
JLA_DEV float ab_ld(const bf16_t* p) { return bf2f(*p); }
JLA_DEV void ab_ld8(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
JLA_DEV void ab_ld8(const bf16_t* p, float* f) { unpack8(*reinterpret_cast<const u32x4*>(p), f); }
JLA_DEV void ab_st(float* p, float v) { *p = v; }
JLA_DEV void ab_st(bf16_t* p, float v) { *p = f2bf(v); }

// grid (M, ceil(items / 4)), 4 waves: wave -> item: [0, H) q heads, [H, H + G) k heads, [H + G, H + 2G) v heads
template <typename CT>
__global__ void __launch_bounds__(256) attn_prep_kernel(AttnPrep p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = blockIdx.x, item = blockIdx.y * 4 + wave;
  const int items = p.H + (p.has_kv ? 2 * p.G : 0);
  if (item >= items) return;
  const float* row = p.proj + (size_t)m * p.ld;
  const int b = m / p.S, sidx = m - b * p.S;
  int kind, head, len, col;
  if (item < p.H) { kind = 0; head = item; len = p.dim; col = head * p.dim; }
  else if (item < p.H + p.G) { kind = 1; head = item - p.H; len = p.dim; col = p.H * p.dim + head * p.dim; }
  else { kind = 2; head = item - p.H - p.G; len = p.vdim; col = (p.H + p.G) * p.dim + head * p.vdim; }
  float sc = 1.f;
  if (kind != 2 || p.norm_v) {
    float ss = 0.f;
    for (int d = lane; d < len; d += 64) {
      const float v = row[col + d];
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    sc = 1.f / sqrtf(ss / (float)len + p.eps);
  }
  const float* gw = kind == 0 ? p.q_w : (kind == 1 ? p.k_w : nullptr);  // gain of the norm, shared by the heads
  if (kind == 0) {
    if (p.temp_coef != 0.f) {
      const int pos = p.positions[m];
      sc *= 1.f + p.temp_coef * logf((float)((pos + 1) / p.temp_every) + 1.f);
    }
    float* q = p.q + ((size_t)m * p.H + head) * p.dim;
    for (int d = lane; d < len; d += 64) q[d] = row[col + d] * sc * (gw ? gw[d] : 1.f);
    return;
  }
  const int t = *p.slot + sidx;
  if (t < 0 || t >= p.T) return;  // cache full: the write is dropped
  CT* dst = (kind == 1 ? reinterpret_cast<CT*>(p.kc) : reinterpret_cast<CT*>(p.vc)) +
            (((size_t)b * p.G + head) * p.T + t) * len;
  for (int d = lane; d < len; d += 64) ab_st(dst + d, row[col + d] * sc * (gw ? gw[d] : 1.f));
}

int hy_attn_prep(const AttnPrep& p, hipStream_t s) {
  if (p.B < 0 || p.S < 1 || p.H < 1 || p.G < 1 || p.H % p.G || p.dim < 1 || p.vdim < 1 || p.T < 1) return -1;
  if (p.temp_coef != 0.f && p.temp_every < 1) return -2;
  const int M = p.B * p.S;
  if (M == 0) return 0;
  const int items = p.H + (p.has_kv ? 2 * p.G : 0);
  if ((items + 3) / 4 > 65535) return -3;
  dim3 grid(M, (items + 3) / 4);
  if (p.cbf16) attn_prep_kernel<bf16_t><<<grid, 256, 0, s>>>(p);
  else attn_prep_kernel<float><<<grid, 256, 0, s>>>(p);
  JLA_CHECK_LAUNCH();
  return 0;
}

constexpr int AB_MAX_DIM = 1024;  // q head held in LDS per wave (keys may be wider than values: a latent cache row
                                  // with a rotated part behind the latent)
constexpr int AB_MAX_VREG = 8;    // value columns per lane: vdim <= 512

// The keys a query at slot qi sees: slots [0, kf) (kept first keys, only beside a window) and [lo, qi], numbered
// 0 .. n - 1 in that order.
struct AbSpan {
  int kf, lo, n;
};
JLA_DEV AbSpan ab_span(const AttnBias& p, int qi) {
  AbSpan sp;
  sp.lo = p.chunk > 0 ? qi / p.chunk * p.chunk : (p.window > 0 ? max(0, qi - p.window + 1) : 0);
  sp.kf = p.window > 0 ? min(p.keep_first, sp.lo) : 0;
  sp.n = sp.kf + qi + 1 - sp.lo;
  return sp;
}
JLA_DEV int ab_key(const AbSpan& sp, int v) { return v < sp.kf ? v : sp.lo + (v - sp.kf); }
JLA_DEV float ab_gate(const AttnBias& p, size_t m, int h) { return p.gate ? hy_sigmoid(p.gate[m * p.ldg + h]) : 1.f; }

// One wave: visible keys number [j_lo, j_hi) of query (b, h) at slot qi (span); returns the running max m, sum l and
// unnormalised acc. with_sink: the wave whose keys start the row also counts the head's sink.
template <typename CT, int VREG>  // VREG: value columns per lane (vdim <= 64 VREG)
JLA_DEV void ab_wave(const AttnBias& p, const float* qs, int b, int h, int qi, const AbSpan& span, int j_lo, int j_hi,
                     bool with_sink, float& m_run, float& l_run, float* acc) {
  constexpr int KB = VREG <= 2 ? 16 : 8;  // keys whose value rows are in flight at a time
  const int lane = threadIdx.x & 63;
  const int g = h / (p.H / p.G);
  const CT* kbase = reinterpret_cast<const CT*>(p.kc) + ((size_t)b * p.G + g) * p.T * p.dim;
  const CT* vbase = reinterpret_cast<const CT*>(p.vc) + ((size_t)b * p.G + g) * p.T * p.ldv;
  const bool fastk = (p.dim & 7) == 0 && ((uintptr_t)kbase & 15) == 0;
  const bool sunk = with_sink && p.sink;
  const float hs = p.head_scale ? p.head_scale[h] : 1.f;
  m_run = sunk ? p.sink[h] : -INFINITY;
  l_run = sunk ? 1.f : 0.f;
#pragma unroll
  for (int i = 0; i < VREG; ++i) acc[i] = 0.f;
  for (int j0 = j_lo; j0 < j_hi; j0 += 64) {
    const int j = j0 + lane;
    const int kj = ab_key(span, min(j, j_hi - 1));  // cache slot of this lane's key
    float sc = -INFINITY;
    if (j < j_hi) {
      const CT* kr = kbase + (size_t)kj * p.dim;
      float d0 = 0.f, d1 = 0.f;
      if (fastk) {  // whole 16-byte groups: branch-free loads the scheduler can batch
#pragma unroll 4
        for (int d = 0; d < p.dim; d += 8) {
          float kf[8];
          ab_ld8(kr + d, kf);
#pragma unroll
          for (int i = 0; i < 8; i += 2) {
            d0 = fmaf(qs[d + i], kf[i], d0);
            d1 = fmaf(qs[d + i + 1], kf[i + 1], d1);
          }
        }
      } else {
        for (int d = 0; d < p.dim; ++d) d0 = fmaf(qs[d], ab_ld(kr + d), d0);
      }
      sc = (d0 + d1) * p.scale * hs;
      if (p.softcap > 0.f) sc = p.softcap * tanhf(sc / p.softcap);
      if (p.bias) sc += p.bias[(size_t)min(qi - kj, p.nbias - 1) * p.H + h];
    }
    const float m_new = fmaxf(m_run, wave_max(sc));
    const float corr = expf(m_run - m_new);  // first chunk: exp(-inf) = 0
    const float pr = j < j_hi ? expf(sc - m_new) : 0.f;
    l_run = l_run * corr + wave_sum(pr);
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < VREG; ++i) acc[i] *= corr;
    const int nk = min(64, j_hi - j0);
    for (int jj = 0; jj < nk; jj += KB) {
      float vv[KB][VREG];
#pragma unroll
      for (int u = 0; u < KB; ++u) {
        const CT* vr = vbase + (size_t)ab_key(span, min(j0 + jj + u, j_hi - 1)) * p.ldv;
#pragma unroll
        for (int i = 0; i < VREG; ++i) {
          vv[u][i] = ab_ld(vr + min(lane + 64 * i, p.vdim - 1));  // (columns past vdim: never stored)
        }
      }
#pragma unroll
      for (int u = 0; u < KB; ++u) {
        const float pj = __shfl(pr, min(jj + u, 63), 64);  // (keys past nk have pr = 0 or repeat a row times 0)
        const float pw = jj + u < nk ? pj : 0.f;
#pragma unroll
        for (int i = 0; i < VREG; ++i) acc[i] = fmaf(pw, vv[u][i], acc[i]);
      }
    }
  }
}

// visible keys number [j_lo, j_hi) of decode split sp: the query's n visible keys dealt to the splits in runs of 64
JLA_DEV void ab_split_range(const AttnBias& p, const AbSpan& span, int sp, int& j_lo, int& j_hi) {
  const int n = span.n;
  const int per = ((n + p.splits - 1) / p.splits + 63) / 64 * 64;
  j_lo = min(n, sp * per);
  j_hi = min(n, j_lo + per);
}

// prefill: grid (ceil(S / 4), H, B), one wave per query
template <typename CT, int VREG>
__global__ void __launch_bounds__(256) attn_bias_prefill_kernel(AttnBias p) {
  __shared__ float qs_all[4][AB_MAX_DIM];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int s = blockIdx.x * 4 + wave, h = blockIdx.y, b = blockIdx.z;
  if (s >= p.S) return;
  float* qs = qs_all[wave];
  const float* q = p.q + (((size_t)b * p.S + s) * p.H + h) * p.dim;
  for (int d = lane; d < p.dim; d += 64) qs[d] = q[d];
  __builtin_amdgcn_wave_barrier();
  const int qi = min(*p.slot + s, p.T - 1);
  float m_run, l_run, acc[VREG];
  const AbSpan span = ab_span(p, qi);
  ab_wave<CT, VREG>(p, qs, b, h, qi, span, 0, span.n, true, m_run, l_run, acc);
  float* o = p.out + ((size_t)b * p.S + s) * (p.H * p.vdim) + (size_t)h * p.vdim;
  const float inv = ab_gate(p, (size_t)b * p.S + s, h) / l_run;
#pragma unroll
  for (int i = 0; i < VREG; ++i) {
    const int c = lane + 64 * i;
    if (c < p.vdim) o[c] = acc[i] * inv;
  }
}

// decode: grid (splits, H, B), one wave per (row, head, split); partial = [m, l, acc[vdim]]
template <typename CT, int VREG>
__global__ void __launch_bounds__(64) attn_bias_decode_kernel(AttnBias p) {
  __shared__ float qs[AB_MAX_DIM];
  const int lane = threadIdx.x;
  const int sp = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const float* q = p.q + ((size_t)b * p.H + h) * p.dim;
  for (int d = lane; d < p.dim; d += 64) qs[d] = q[d];
  __syncthreads();
  const int qi = min(*p.slot, p.T - 1);
  int j_lo, j_hi;
  const AbSpan span = ab_span(p, qi);
  ab_split_range(p, span, sp, j_lo, j_hi);
  float m_run, l_run, acc[VREG];
  ab_wave<CT, VREG>(p, qs, b, h, qi, span, j_lo, j_hi, sp == 0, m_run, l_run, acc);
  float* w = p.ws + (((size_t)b * p.H + h) * p.splits + sp) * (p.vdim + 2);
  if (lane == 0) {
    w[0] = m_run;
    w[1] = l_run;
  }
#pragma unroll
  for (int i = 0; i < VREG; ++i) {
    const int c = lane + 64 * i;
    if (c < p.vdim) w[2 + c] = acc[i];
  }
}

// decode, bf16 caches, dim = 8 DK8 in {64, 128}, vdim = 64 VREG in {64, 128}: the same split as above with every load of
// a 64-key chunk (the lane's key row, its bias, all 64 value rows) issued before the first use, and q staged into LDS
// behind them: a decode step is a chain of memory round trips, and this form has two.
template <int DK8, int VREG>
__global__ void __launch_bounds__(64) attn_bias_decode_fast_kernel(AttnBias p) {
  constexpr int dim = 8 * DK8, vdim = 64 * VREG;
  __shared__ float qs[dim];
  const int lane = threadIdx.x;
  const int sp = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int g = h / (p.H / p.G);
  const float* q = p.q + ((size_t)b * p.H + h) * dim;
  float qv[dim / 64];
#pragma unroll
  for (int i = 0; i < dim / 64; ++i) qv[i] = q[lane + 64 * i];
  const int qi = min(*p.slot, p.T - 1);
  int j_lo, j_hi;
  const AbSpan span = ab_span(p, qi);
  ab_split_range(p, span, sp, j_lo, j_hi);
  const bf16_t* kbase = reinterpret_cast<const bf16_t*>(p.kc) + ((size_t)b * p.G + g) * p.T * dim;
  const bf16_t* vbase = reinterpret_cast<const bf16_t*>(p.vc) + ((size_t)b * p.G + g) * p.T * p.ldv;
  const bool sunk = p.sink && sp == 0;
  const float hs = p.head_scale ? p.head_scale[h] : 1.f;
  float m_run = sunk ? p.sink[h] : -INFINITY, l_run = sunk ? 1.f : 0.f, acc[VREG];
#pragma unroll
  for (int i = 0; i < VREG; ++i) acc[i] = 0.f;
  bool staged = false;
  for (int j0 = j_lo; j0 < j_hi; j0 += 64) {
    const int j = j0 + lane, jc = ab_key(span, min(j, j_hi - 1));  // (jc: the cache slot)
    u32x4 kf[DK8];
#pragma unroll
    for (int u = 0; u < DK8; ++u) kf[u] = *reinterpret_cast<const u32x4*>(kbase + (size_t)jc * dim + 8 * u);
    const float bl = p.bias ? p.bias[(size_t)min(qi - jc, p.nbias - 1) * p.H + h] : 0.f;
    bf16_t vv[64][VREG];
#pragma unroll
    for (int jj = 0; jj < 64; ++jj) {
      const bf16_t* vr = vbase + (size_t)ab_key(span, min(j0 + jj, j_hi - 1)) * p.ldv + lane;
#pragma unroll
      for (int i = 0; i < VREG; ++i) vv[jj][i] = vr[64 * i];
    }
    if (!staged) {
#pragma unroll
      for (int i = 0; i < dim / 64; ++i) qs[lane + 64 * i] = qv[i];
      __syncthreads();
      staged = true;
    }
    float d0 = 0.f, d1 = 0.f;
#pragma unroll
    for (int u = 0; u < DK8; ++u) {
      float f[8];
      unpack8(kf[u], f);
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        d0 = fmaf(qs[8 * u + i], f[i], d0);
        d1 = fmaf(qs[8 * u + i + 1], f[i + 1], d1);
      }
    }
    float sc = (d0 + d1) * p.scale * hs;
    if (p.softcap > 0.f) sc = p.softcap * tanhf(sc / p.softcap);
    sc += bl;
    if (j >= j_hi) sc = -INFINITY;
    const float m_new = fmaxf(m_run, wave_max(sc));
    const float corr = expf(m_run - m_new);
    const float pr = j < j_hi ? expf(sc - m_new) : 0.f;
    l_run = l_run * corr + wave_sum(pr);
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < VREG; ++i) acc[i] *= corr;
#pragma unroll
    for (int jj = 0; jj < 64; ++jj) {
      const float pj = __shfl(pr, jj, 64);  // (0 for keys past the split)
#pragma unroll
      for (int i = 0; i < VREG; ++i) acc[i] = fmaf(pj, bf2f(vv[jj][i]), acc[i]);
    }
  }
  float* w = p.ws + (((size_t)b * p.H + h) * p.splits + sp) * (vdim + 2);
  if (lane == 0) {
    w[0] = m_run;
    w[1] = l_run;
  }
#pragma unroll
  for (int i = 0; i < VREG; ++i) w[2 + lane + 64 * i] = acc[i];
}

// decode over a shared latent: keys = values = ONE bf16 cache head (kc == vc, G == 1), rows of 136 to 512 numbers of
// which the first vdim are the values (all of them, or a latent in front of a rotated key part), no bias / soft cap. The lanes split a row's numbers, 16 bytes each, so one coalesced load per key serves both the score
// (row totals by DPP, the four rows through scalar registers: no LDS round trips) and the value sum; all loads of a
// chunk of keys are issued before the first use. A wave serves HQ heads of one row (HQ = 4 measured slower than 1 at 8
// rows x 16 heads, 94 against 58 us: four times the scalar-register traffic per key on a quarter of the waves; dealing
// the batch rows to XCDs by workgroup id, so that each L2 holds one row's latent, changed nothing: the kernel is bound
// by its own instruction stream, about 50 per key, not by what it reads).
// Grid (splits, H / HQ, B); partial layout as the kernels above.
constexpr int AL_KC = 16;
JLA_DEV float al_lane(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

template <int HQ, int KC>  // heads per wave, keys per chunk
__global__ void __launch_bounds__(64) attn_latent_decode_kernel(AttnBias p) {
  const int lane = threadIdx.x;
  const int sp = blockIdx.x, h0 = blockIdx.y * HQ, b = blockIdx.z;
  const int rank = p.dim;
  const bool on = 8 * lane < rank;
  const int c0 = on ? 8 * lane : 0;  // (surplus lanes re-read the row's start against a zero query)
  float qv[HQ][8];
#pragma unroll
  for (int q = 0; q < HQ; ++q) {
    hy_load8(p.q + ((size_t)b * p.H + h0 + q) * rank + c0, 8, qv[q]);
#pragma unroll
    for (int i = 0; i < 8; ++i) qv[q][i] = on ? qv[q][i] : 0.f;
  }
  const int qi = min(*p.slot, p.T - 1);
  int j_lo, j_hi;
  const AbSpan span = ab_span(p, qi);
  ab_split_range(p, span, sp, j_lo, j_hi);
  const bf16_t* base = reinterpret_cast<const bf16_t*>(p.kc) + (size_t)b * p.T * rank + c0;
  const bool sunk = p.sink && sp == 0;
  float m_run[HQ], l_run[HQ], acc[HQ][8], hs[HQ];
#pragma unroll
  for (int q = 0; q < HQ; ++q) {
    hs[q] = p.head_scale ? p.head_scale[h0 + q] : 1.f;
    m_run[q] = sunk ? p.sink[h0 + q] : -INFINITY;
    l_run[q] = sunk ? 1.f : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[q][i] = 0.f;
  }
  for (int j0 = j_lo; j0 < j_hi; j0 += KC) {
    u32x4 rows[KC];
#pragma unroll
    for (int u = 0; u < KC; ++u)
      rows[u] = *reinterpret_cast<const u32x4*>(base + (size_t)ab_key(span, min(j0 + u, j_hi - 1)) * rank);
    float sc[HQ][KC], cmax[HQ];
#pragma unroll
    for (int q = 0; q < HQ; ++q) cmax[q] = -INFINITY;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      float f[8];
      unpack8(rows[u], f);
#pragma unroll
      for (int q = 0; q < HQ; ++q) {
        float d0 = 0.f, d1 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
          d0 = fmaf(qv[q][i], f[i], d0);
          d1 = fmaf(qv[q][i + 1], f[i + 1], d1);
        }
        const float rt = row16_sum(d0 + d1);
        const float dot = (al_lane(rt, 0) + al_lane(rt, 16) + al_lane(rt, 32) + al_lane(rt, 48)) * p.scale * hs[q];
        sc[q][u] = j0 + u < j_hi ? dot : -INFINITY;
        cmax[q] = fmaxf(cmax[q], sc[q][u]);
      }
    }
    float m_new[HQ];
#pragma unroll
    for (int q = 0; q < HQ; ++q) {
      m_new[q] = fmaxf(m_run[q], cmax[q]);  // (a chunk holds at least one key, so m_new is finite)
      const float corr = expf(m_run[q] - m_new[q]);
      l_run[q] *= corr;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[q][i] *= corr;
      m_run[q] = m_new[q];
    }
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      float f[8];
      unpack8(rows[u], f);
#pragma unroll
      for (int q = 0; q < HQ; ++q) {
        const float pr = expf(sc[q][u] - m_new[q]);  // (0 past the split's end)
        l_run[q] += pr;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[q][i] = fmaf(pr, f[i], acc[q][i]);
      }
    }
  }
#pragma unroll
  for (int q = 0; q < HQ; ++q) {
    float* w = p.ws + (((size_t)b * p.H + h0 + q) * p.splits + sp) * (p.vdim + 2);
    if (lane == 0) {
      w[0] = m_run[q];
      w[1] = l_run[q];
    }
    if (on && c0 < p.vdim) {  // (the values are the row's first vdim numbers)
#pragma unroll
      for (int i = 0; i < 8; ++i) w[2 + c0 + i] = acc[q][i];
    }
  }
}

// grid (H, B, ceil(vdim / 64)), 64 threads: merge the splits (at most 64: lane sp holds split sp's maximum and sum) for
// one 64-column slice of the head's output
__global__ void __launch_bounds__(64) attn_bias_merge_kernel(AttnBias p) {
  const int lane = threadIdx.x, h = blockIdx.x, b = blockIdx.y, c0 = blockIdx.z * 64;
  const float* w = p.ws + ((size_t)b * p.H + h) * p.splits * (p.vdim + 2);
  float ms = -INFINITY, ls = 0.f;
  if (lane < p.splits) {
    ms = w[(size_t)lane * (p.vdim + 2)];
    ls = w[(size_t)lane * (p.vdim + 2) + 1];
  }
  const int c = min(c0 + lane, p.vdim - 1);
  float part[64];
#pragma unroll
  for (int sp = 0; sp < 64; ++sp) part[sp] = w[(size_t)min(sp, p.splits - 1) * (p.vdim + 2) + 2 + c];  // one round trip
  const float m = wave_max(ls > 0.f ? ms : -INFINITY);
  const float wt = ls > 0.f ? expf(ms - m) : 0.f;  // weight of this lane's split
  const float l = wave_sum(ls * wt);
  float* o = p.out + (size_t)b * (p.H * p.vdim) + (size_t)h * p.vdim;
  float a = 0.f;
#pragma unroll
  for (int sp = 0; sp < 64; ++sp) {  // (a split without keys holds zeros and has weight 0)
    const float ws = __shfl(wt, sp, 64);
    a = fmaf(part[sp], sp < p.splits ? ws : 0.f, a);
  }
  if (c0 + lane < p.vdim) o[c] = a / l * ab_gate(p, b, h);
}

// ---- MFMA flash prefill (bf16 caches) ----------------------------------------------------------------------------------
// One wave = 32 queries of one head, no LDS and no barriers. Keys go by in tiles of 32:
//   S^T = K Q^T on v_mfma_f32_32x32x16_bf16 with the QUERY on the lane (lane l: query l & 31; its 16 accumulators are 16
//   of the tile's keys, the other half-wave holds the other 16), so scale, soft cap, bias, mask and the online softmax
//   are lane-local plus one exchange with lane ^ 32. The key rows are fed in an order (bits 2 and 3 of the row index
//   swapped) that leaves a lane's accumulators 8c .. 8c + 7 holding keys 16c + 8 (l >> 5) + 0..7: exactly the k-slots
//   of the B operand of O^T += V^T P^T, so P is used in place. V^T comes from a transposed bf16 copy of the values
//   (attn_vt_kernel, zero past the last key), 16-byte loads along the keys.
//   The softmax weights stay 32-bit: P is split into a bf16 high part and a bf16 remainder, two MFMAs per value tile.
//   Scores of the fast path use exp-based tanh and v_exp_f32; the fp32 format keeps the exact kernel above.
constexpr int AM_Q = 32, AM_K = 32;
using f32x16 = __attribute__((ext_vector_type(16))) float;

// Vt[b][g][c][j] = V[b][g][j][c] for j < n = *slot + S (0 for n <= j < round_up(n, 32)); grid (Tp / 32, vdim / 32, B * G)
__global__ void __launch_bounds__(256) attn_vt_kernel(const bf16_t* __restrict__ vc, bf16_t* __restrict__ vt,
                                                      const int32_t* slot, int S, int T, int Tp, int vdim) {
  __shared__ bf16_t tile[32][34];
  const int n = min(*slot + S, T);
  const int j0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
  if (j0 >= n) return;
  const size_t bg = blockIdx.z;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  for (int r = ty; r < 32; r += 8) {
    const int j = j0 + r;
    tile[r][tx] = j < n ? vc[(bg * T + j) * vdim + c0 + tx] : (bf16_t)0;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) vt[(bg * vdim + c0 + r) * Tp + j0 + tx] = tile[tx][r];
}

JLA_DEV float am_tanh(float x) {  // 1 - 2 / (e^(2x) + 1), saturating cleanly for large |x|
  const float e = __expf(2.f * x);
  return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}

template <int DK, int VT>  // dim = 16 DK, vdim = 32 VT
__global__ void __launch_bounds__(256) attn_bias_mma_kernel(AttnBias p, const bf16_t* __restrict__ vt, int Tp) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ql = lane & 31, hi = lane >> 5;
  const int qblk = (gridDim.x - 1 - blockIdx.x) * 4 + wave;  // long rows first
  const int s0 = qblk * AM_Q;
  if (s0 >= p.S) return;
  const int h = blockIdx.y, b = blockIdx.z;
  const int g = h / (p.H / p.G);
  const int slot = *p.slot;
  const int q0 = slot + s0;                 // cache slot of this wave's first query
  const int sq = min(s0 + ql, p.S - 1);     // (surplus lanes repeat the last query; never stored)
  const int qi = slot + sq;
  constexpr int dim = 16 * DK, vdim = 32 * VT;
  // Q as the B operand: query ql, k-slots 16 kk + 8 hi + e
  bf16x8_t qf[DK];
  {
    const float* q = p.q + (((size_t)b * p.S + sq) * p.H + h) * dim + 8 * hi;
#pragma unroll
    for (int kk = 0; kk < DK; ++kk) {
      float f[8];
      hy_load8(q + 16 * kk, 8, f);
      qf[kk] = __builtin_bit_cast(bf16x8_t, pack8(f));
    }
  }
  const bf16_t* kbase = reinterpret_cast<const bf16_t*>(p.kc) + ((size_t)b * p.G + g) * p.T * dim;
  const bf16_t* vbase = vt + ((size_t)b * p.G + g) * vdim * Tp;
  const int krow = (ql & 0x13) | ((ql & 4) << 1) | ((ql & 8) >> 1);  // bits 2 and 3 swapped
  f32x16 o[VT];
#pragma unroll
  for (int v = 0; v < VT; ++v)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[v][r] = 0.f;
  // (l_run holds this half-wave's part of the sum: the sink counts once, in the lower half)
  float m_run = p.sink ? p.sink[h] : -INFINITY, l_run = p.sink && hi == 0 ? 1.f : 0.f;
  const int q_last = min(q0 + AM_Q - 1, slot + p.S - 1);
  const float inv_cap = p.softcap > 0.f ? 1.f / p.softcap : 0.f;
  const float hs = p.head_scale ? p.head_scale[h] : 1.f;
  // block-local mask: this query's first key, the last query's (the largest of the wave), and the tile the walk starts at
  const int lo_q = ab_span(p, qi).lo, lo_last = ab_span(p, q_last).lo;
  const int j_begin = ab_span(p, q0).lo / AM_K * AM_K;
  // kept first keys (beside a window): their tiles [0, kf_end) come first, then the walk jumps to the window's tiles
  const int kfirst = p.window > 0 ? p.keep_first : 0;
  const int kf_end = min((kfirst + AM_K - 1) / AM_K * AM_K, j_begin);
  auto next_tile = [&](int j0) { return j0 + AM_K == kf_end ? j_begin : j0 + AM_K; };
  // the next tile's key and value fragments are loaded while the current tile is computed (one wave per SIMD at small
  // batch: nothing else hides the loads)
  u32x4 kn[DK], vn[2][VT];
  auto fetch = [&](int j0) {
    const bf16_t* kr = kbase + (size_t)min(j0 + krow, p.T - 1) * dim + 8 * hi;
#pragma unroll
    for (int kk = 0; kk < DK; ++kk) kn[kk] = *reinterpret_cast<const u32x4*>(kr + 16 * kk);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int v = 0; v < VT; ++v)
        vn[c][v] = *reinterpret_cast<const u32x4*>(vbase + (size_t)(32 * v + ql) * Tp + min(j0, Tp - AM_K) + 16 * c + 8 * hi);
  };
  const int j_first = kf_end > 0 ? 0 : j_begin;
  fetch(j_first);
  for (int j0 = j_first; j0 <= q_last; j0 = next_tile(j0)) {
    u32x4 kc_[DK], vc_[2][VT];
#pragma unroll
    for (int kk = 0; kk < DK; ++kk) kc_[kk] = kn[kk];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int v = 0; v < VT; ++v) vc_[c][v] = vn[c][v];
    fetch(next_tile(j0));  // (past the last tile: clamped addresses, never used)
    // scores: rows = keys (fed permuted), columns = queries
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < DK; ++kk)
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kc_[kk]), qf[kk], sacc, 0, 0, 0);
    // bias of this tile's 63 distances, one per lane: lane t holds distance q0 - j0 - 31 + t
    float bl = 0.f;
    const int dbase = q0 - j0 - (AM_K - 1);
    const bool far = p.bias && dbase >= p.nbias - 1;
    if (p.bias) bl = p.bias[(size_t)min(max(dbase + lane, 0), p.nbias - 1) * p.H + h];
    // some (query, key) of the tile is masked
    const bool diag = j0 + AM_K - 1 > q0 || (j0 < lo_last && j0 + AM_K - 1 >= kfirst);
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kl = 16 * (r >> 3) + 8 * hi + (r & 7);  // key of accumulator r within the tile
      float sc = sacc[r] * p.scale * hs;
      if (p.softcap > 0.f) sc = p.softcap * am_tanh(sc * inv_cap);
      if (p.bias) sc += far ? bl : __shfl(bl, ql - kl + (AM_K - 1), 64);
      if (diag && (j0 + kl > qi || (j0 + kl < lo_q && j0 + kl >= kfirst))) sc = -INFINITY;
      sacc[r] = sc;
      tmax = fmaxf(tmax, sc);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    // (a query without a sink may have no visible key in a tile it shares with its neighbours' earlier blocks)
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __expf(m_run - m_use);
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sacc[r] = __expf(sacc[r] - m_use);
      psum += sacc[r];
    }
    l_run = l_run * corr + psum;  // (this half-wave's keys; the halves are added at the end)
#pragma unroll
    for (int v = 0; v < VT; ++v)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[v][r] *= corr;
    // O^T += V^T P^T, P = high bf16 part + bf16 remainder
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      float ph[8], pl[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ph[e] = bf2f(f2bf(sacc[8 * c + e]));
        pl[e] = sacc[8 * c + e] - ph[e];
      }
      const bf16x8_t bh = __builtin_bit_cast(bf16x8_t, pack8(ph)), bo = __builtin_bit_cast(bf16x8_t, pack8(pl));
#pragma unroll
      for (int v = 0; v < VT; ++v) {
        const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, vc_[c][v]);
        o[v] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, bh, o[v], 0, 0, 0);
        o[v] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, bo, o[v], 0, 0, 0);
      }
    }
  }
  l_run += __shfl_xor(l_run, 32, 64);
  if (s0 + ql >= p.S) return;
  const float inv = ab_gate(p, (size_t)b * p.S + s0 + ql, h) / l_run;
  float* out = p.out + ((size_t)b * p.S + s0 + ql) * (p.H * vdim) + (size_t)h * vdim;
#pragma unroll
  for (int v = 0; v < VT; ++v)
#pragma unroll
    for (int r = 0; r < 16; r += 4) {  // rows (value columns) (r & 3) + 8 (r >> 2) + 4 hi: runs of four
      const float4 w = {o[v][r] * inv, o[v][r + 1] * inv, o[v][r + 2] * inv, o[v][r + 3] * inv};
      *reinterpret_cast<float4*>(out + 32 * v + 8 * (r >> 2) + 4 * hi) = w;
    }
}

template <int DK, int VT>
static int am_launch(const AttnBias& p, bf16_t* vt, int Tp, hipStream_t s) {
  attn_vt_kernel<<<dim3(Tp / 32, p.vdim / 32, p.B * p.G), 256, 0, s>>>(reinterpret_cast<const bf16_t*>(p.vc), vt, p.slot,
                                                                     p.S, p.T, Tp, p.vdim);
  JLA_CHECK_LAUNCH();
  attn_bias_mma_kernel<DK, VT><<<dim3((p.S + 127) / 128, p.H, p.B), 256, 0, s>>>(p, vt, Tp);
  JLA_CHECK_LAUNCH();
  return 0;
}

// bytes of the transposed-value workspace the MFMA prefill needs, 0 when the shape goes to the plain kernel
long long hy_attn_prefill_ws_bytes(int B, int S, int G, int dim, int vdim, int T, int cbf16) {
  if (!cbf16 || S < 2) return 0;
  if (!((dim == 64 || dim == 128) && (vdim == 64 || vdim == 128))) return 0;
  if ((long long)B * G > 65535) return 0;
  return (long long)B * G * vdim * ((T + 31) / 32 * 32) * 2;
}

int hy_attn_decode_splits(int B, int H, int t_cap) {
  // enough waves for the chip (256 CUs x 4 SIMDs x 2), at least one 64-key step per split
  const long long pairs = (long long)B * H;
  long long want = (2048 + pairs - 1) / (pairs > 0 ? pairs : 1);
  const long long by_len = (t_cap + 63) / 64;
  if (want > by_len) want = by_len;
  if (want < 1) want = 1;
  if (want > 64) want = 64;
  return (int)want;
}

// launch KERNEL<cache type, value registers per lane> for p.vdim
#define AB_BY_VREG(KERNEL, GRID, THREADS)                                              \
  do {                                                                                 \
    const int vr = (p.vdim + 63) / 64;                                                 \
    if (p.cbf16) {                                                                     \
      if (vr <= 1) KERNEL<bf16_t, 1><<<GRID, THREADS, 0, s>>>(p);                      \
      else if (vr <= 2) KERNEL<bf16_t, 2><<<GRID, THREADS, 0, s>>>(p);                 \
      else if (vr <= 4) KERNEL<bf16_t, 4><<<GRID, THREADS, 0, s>>>(p);                 \
      else KERNEL<bf16_t, 8><<<GRID, THREADS, 0, s>>>(p);                              \
    } else {                                                                           \
      if (vr <= 1) KERNEL<float, 1><<<GRID, THREADS, 0, s>>>(p);                       \
      else if (vr <= 2) KERNEL<float, 2><<<GRID, THREADS, 0, s>>>(p);                  \
      else if (vr <= 4) KERNEL<float, 4><<<GRID, THREADS, 0, s>>>(p);                  \
      else KERNEL<float, 8><<<GRID, THREADS, 0, s>>>(p);                               \
    }                                                                                  \
  } while (0)

int hy_attn_bias(const AttnBias& p, hipStream_t s) {
  if (p.B < 0 || p.S < 1 || p.H < 1 || p.G < 1 || p.H % p.G || p.T < 1) return -1;
  if (p.dim < 1 || p.dim > AB_MAX_DIM || p.vdim < 1 || p.vdim > 64 * AB_MAX_VREG) return -2;
  if (p.bias && p.nbias < 1) return -3;
  if (p.chunk < 0 || p.window < 0 || p.keep_first < 0 || (p.chunk > 0 && p.window > 0)) return -7;
  if (p.ldv < p.vdim || (p.gate && p.ldg < p.H)) return -8;
  if (p.B == 0) return 0;
  if (p.H > 65535 || p.B > 65535) return -4;
  if (p.S == 1) {
    if (p.splits < 1 || !p.ws) return -5;
    if (p.splits > 64) return -6;  // (the merge holds one split per lane)
    dim3 grid(p.splits, p.H, p.B);
    if (p.cbf16 && (p.dim == 64 || p.dim == 128) && (p.vdim == 64 || p.vdim == 128) && p.ldv == p.vdim) {
      if (p.dim == 64 && p.vdim == 64) attn_bias_decode_fast_kernel<8, 1><<<grid, 64, 0, s>>>(p);
      else if (p.dim == 64) attn_bias_decode_fast_kernel<8, 2><<<grid, 64, 0, s>>>(p);
      else if (p.vdim == 64) attn_bias_decode_fast_kernel<16, 1><<<grid, 64, 0, s>>>(p);
      else attn_bias_decode_fast_kernel<16, 2><<<grid, 64, 0, s>>>(p);
    } else if (p.cbf16 && p.kc == p.vc && p.G == 1 && p.ldv == p.dim && p.vdim <= p.dim && p.vdim % 8 == 0 &&
               p.dim % 8 == 0 && p.dim > 128 && p.dim <= 512 && !p.bias && p.softcap <= 0.f &&
               ((uintptr_t)p.kc & 15) == 0) {
      attn_latent_decode_kernel<1, AL_KC><<<grid, 64, 0, s>>>(p);
    } else {
      AB_BY_VREG(attn_bias_decode_kernel, grid, 64);
    }
    JLA_CHECK_LAUNCH();
    attn_bias_merge_kernel<<<dim3(p.H, p.B, (p.vdim + 63) / 64), 64, 0, s>>>(p);
    JLA_CHECK_LAUNCH();
    return 0;
  }
  if (p.vt_ws && p.ldv == p.vdim && hy_attn_prefill_ws_bytes(p.B, p.S, p.G, p.dim, p.vdim, p.T, p.cbf16) > 0) {
    const int Tp = (p.T + 31) / 32 * 32;
    bf16_t* vt = reinterpret_cast<bf16_t*>(p.vt_ws);
    if (p.dim == 64 && p.vdim == 64) return am_launch<4, 2>(p, vt, Tp, s);
    if (p.dim == 64 && p.vdim == 128) return am_launch<4, 4>(p, vt, Tp, s);
    if (p.dim == 128 && p.vdim == 64) return am_launch<8, 2>(p, vt, Tp, s);
    return am_launch<8, 4>(p, vt, Tp, s);
  }
  dim3 grid((p.S + 3) / 4, p.H, p.B);
  AB_BY_VREG(attn_bias_prefill_kernel, grid, 256);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
