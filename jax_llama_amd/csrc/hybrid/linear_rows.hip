// Row-gathered, expert-grouped linear on row-major weights of any shape (no N % 16 / K % 32 packing constraint):
//   out[dst(r), :] = act(A[src(r), :] @ W[expert(r)]^T)
// A is fp32 in memory. With bf16 weights the A tile is rounded to bf16 while it is staged (v_mfma_f32_32x32x16_bf16,
// fp32 accumulation); with fp32 weights everything stays fp32 on the exact-f32 MFMA (v_mfma_f32_32x32x2_f32).
//
//  * tiles: 64 x 64 or (with rows to fill them) 128 x 64 outputs per 256-thread workgroup, four waves of 32 x 32 /
//    64 x 32, K staged 32 deep through LDS (several workgroups per CU hide each other's staging; a 128 x 128 tile with
//    register prefetch and a 64-deep K stage measured slower). The activations may be a bf16 copy and the output bf16
//    (the expert pair of a prompt: x -> bf16 once, hidden kept bf16), which halves the activation traffic. With an
//    expert offset table the m-tiles of the launch are dealt to the experts in order (a workgroup finds its expert by
//    walking the table; surplus workgroups exit), so one launch covers every expert of a token-sorted batch.
//  * few rows (decode): a wave streams one or four weight rows once and dots them with up to 8 activation rows.
//  * epilogues (RowAct): squared ReLU on one accumulator; gated forms accumulate the gate and the up rows of a column
//    side by side: silu(g) * u, or the clamped form g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = clamp(u).
//  * an optional per-row scale multiplies the activation row while it is staged (before the operand is rounded): the
//    input-weighted experts of a score-routed mixture.
// The table router's counting sort is here too.
#include "hy_util.h"
#include "hybrid.h"

namespace jla {

using f32x16 = __attribute__((ext_vector_type(16))) float;

constexpr int LR_BM = 64, LR_BN = 64, LR_BK = 32, LR_THREADS = 256;

template <typename WT>
struct LrTile;
template <>
struct LrTile<bf16_t> {
  static constexpr int LD = LR_BK + 8;  // 80-byte rows: 16-byte aligned fragment reads, rows spread over the banks
};
template <>
struct LrTile<float> {
  static constexpr int LD = LR_BK + 1;
};

JLA_DEV void lr_store8(bf16_t* dst, const float* f) { *reinterpret_cast<u32x4*>(dst) = pack8(f); }
JLA_DEV void lr_store8(float* dst, const float* f) {
#pragma unroll
  for (int i = 0; i < 8; ++i) dst[i] = f[i];
}

JLA_DEV void lr_mma(const bf16_t* a_row, const bf16_t* b_row, int hi, f32x16& acc) {
#pragma unroll
  for (int kk = 0; kk < LR_BK / 16; ++kk) {
    const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(a_row + 16 * kk + 8 * hi);
    const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(b_row + 16 * kk + 8 * hi);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
  }
}
JLA_DEV void lr_mma(const float* a_row, const float* b_row, int hi, f32x16& acc) {
#pragma unroll
  for (int kk = 0; kk < LR_BK / 2; ++kk)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_row[2 * kk + hi], b_row[2 * kk + hi], acc, 0, 0, 0);
}

// 8 consecutive k of a row into the LDS tile (zeros past `left`); a bf16 source going to a bf16 tile is copied as is
JLA_DEV void lr_stage8(const float* src, int left, bf16_t* dst, float sc = 1.f) {
  float f[8];
  hy_load8(src, left, f);
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] *= sc;
  lr_store8(dst, f);
}
JLA_DEV void lr_stage8(const float* src, int left, float* dst, float sc = 1.f) {
  float f[8];
  hy_load8(src, left, f);
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] *= sc;
  lr_store8(dst, f);
}
JLA_DEV void lr_stage8(const bf16_t* src, int left, bf16_t* dst, float = 1.f) {
  if (left >= 8 && ((uintptr_t)src & 15) == 0) {
    *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
  } else {
    float f[8];
    hy_load8(src, left, f);
    lr_store8(dst, f);
  }
}
JLA_DEV void lr_stage8(const bf16_t* src, int left, float* dst, float = 1.f) {
  float f[8];
  hy_load8(src, left, f);
  lr_store8(dst, f);
}
template <typename T>
JLA_DEV void lr_zero8(T* dst) {
  const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  lr_store8(dst, z);
}
JLA_DEV void lr_out(float* p, float v) { *p = v; }
JLA_DEV void lr_out(bf16_t* p, float v) { *p = f2bf(v); }

// the epilogue of one output element: g the (gate) accumulator, u the up accumulator of the gated forms
JLA_DEV float lr_act(const RowLinear& p, float g, float u) {
  switch (p.act) {
    case HY_ACT_RELU2: {
      const float r = fmaxf(g, 0.f);
      return r * r;
    }
    case HY_ACT_SWIGLU:
      return hy_silu(g) * u;
    case HY_ACT_CLAMP_GLU: {
      const float gc = fminf(g, p.act_limit), uc = fminf(fmaxf(u, -p.act_limit), p.act_limit);
      return gc * hy_sigmoid(p.act_alpha * gc) * (uc + 1.f);
    }
    case HY_ACT_SOFTCAP:
      return p.act_limit * tanhf(g / p.act_limit);
    default:
      return g;
  }
}
JLA_DEV float lr_in(const float* p) { return *p; }
JLA_DEV float lr_in(const bf16_t* p) { return bf2f(*p); }

// WT: weight / tile type; AT: activation type in memory (fp32, or a bf16 copy); OT: output type; TMM: 32-row tiles per
// wave along M (workgroup tile 64 TMM x 64: the 128-row form halves the weight traffic per output row).
template <typename WT, int SWIGLU, typename AT, typename OT, int TMM>
__global__ void __launch_bounds__(LR_THREADS) lr_gemm_kernel(RowLinear p) {
  constexpr int LD = LrTile<WT>::LD;
  constexpr int BM = LR_BM * TMM;
  __shared__ __attribute__((aligned(16))) WT As[BM * LD];
  __shared__ __attribute__((aligned(16))) WT Bs[(SWIGLU ? 2 : 1) * LR_BN * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, hi = lane >> 5;
  // which expert and which rows
  int e = 0, r0 = blockIdx.y * BM, rend = p.R;
  if (p.offs) {
    int tile = blockIdx.y;
    bool found = false;
    for (e = 0; e < p.E; ++e) {
      const int b = p.offs[e], cnt = p.offs[e + 1] - b, nt = (cnt + BM - 1) / BM;
      if (tile < nt) {
        r0 = b + tile * BM;
        rend = b + cnt;
        found = true;
        break;
      }
      tile -= nt;
    }
    if (!found) return;
  } else if (r0 >= rend) {
    return;
  }
  const int n0 = blockIdx.x * LR_BN;
  const WT* W = reinterpret_cast<const WT*>(p.w) + (size_t)e * p.w_stride;
  const int K = p.K, N = p.N;

  // staging role: 8 consecutive k of row (tid >> 2) (+ 64 for the second half of a 128-row tile)
  const int srow = tid >> 2, skq = (tid & 3) * 8;
  const AT* a_ptr[TMM];
  float a_sc[TMM];
#pragma unroll
  for (int t = 0; t < TMM; ++t) {
    const int ar = r0 + srow + 64 * t;
    a_ptr[t] = ar < rend ? reinterpret_cast<const AT*>(p.a) + (size_t)(p.a_idx ? p.a_idx[ar] : ar) * p.lda : nullptr;
    a_sc[t] = (p.a_scale && ar < rend) ? p.a_scale[ar] : 1.f;
  }
  const int wr = n0 + srow;
  const WT* w_ptr = wr < N ? W + (size_t)wr * K : nullptr;
  const WT* w2_ptr = (SWIGLU && wr < N) ? W + (size_t)(N + wr) * K : nullptr;

  f32x16 acc[TMM], acc2[TMM];
#pragma unroll
  for (int t = 0; t < TMM; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = acc2[t][r] = 0.f;

  for (int k0 = 0; k0 < K; k0 += LR_BK) {
    const int gk = k0 + skq, left = K - gk;
#pragma unroll
    for (int t = 0; t < TMM; ++t) {
      if (a_ptr[t] && left > 0) lr_stage8(a_ptr[t] + gk, left, &As[(srow + 64 * t) * LD + skq], a_sc[t]);
      else lr_zero8(&As[(srow + 64 * t) * LD + skq]);
    }
    if (w_ptr && left > 0) lr_stage8(w_ptr + gk, left, &Bs[srow * LD + skq]);
    else lr_zero8(&Bs[srow * LD + skq]);
    if (SWIGLU) {
      if (w2_ptr && left > 0) lr_stage8(w2_ptr + gk, left, &Bs[(LR_BN + srow) * LD + skq]);
      else lr_zero8(&Bs[(LR_BN + srow) * LD + skq]);
    }
    __syncthreads();
    const WT* b_row = &Bs[(wn * 32 + (lane & 31)) * LD];
#pragma unroll
    for (int t = 0; t < TMM; ++t) {
      const WT* a_row = &As[(wm * 32 * TMM + 32 * t + (lane & 31)) * LD];
      lr_mma(a_row, b_row, hi, acc[t]);
      if (SWIGLU) lr_mma(a_row, b_row + LR_BN * LD, hi, acc2[t]);
    }
    __syncthreads();
  }
  // C/D map of the 32 x 32 shapes: col = lane & 31, row = (r & 3) + 8 (r >> 2) + 4 (lane >> 5)
  const int col = n0 + wn * 32 + (lane & 31);
  if (col >= N) return;
  OT* out = reinterpret_cast<OT*>(p.out);
#pragma unroll
  for (int t = 0; t < TMM; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = r0 + wm * 32 * TMM + 32 * t + (r & 3) + 8 * (r >> 2) + 4 * hi;
      if (row < rend) {
        const int drow = p.dst_idx ? p.dst_idx[row] : row;
        OT* dst = out + (size_t)drow * p.ldo + col;
        const float val = lr_act(p, acc[t][r], SWIGLU ? acc2[t][r] : 0.f);
        lr_out(dst, p.add_out ? lr_in(dst) + val : val);
      }
    }
}

JLA_DEV float lr_round(float v, const bf16_t*) { return bf2f(f2bf(v)); }
JLA_DEV float lr_round(float v, const float*) { return v; }

// A wave owns LR_CPW consecutive output columns (4 for wide outputs such as a vocabulary head, 1 where that would
// leave too few workgroups): their weight rows are streamed once (16-byte loads, LR_CPW rows in flight per lane) and
// dotted with the rows of group blockIdx.y: a fixed count of rows, one row with its own expert (row_expert), or every
// row of one expert of an expert-sorted batch (offs).
// NORM: each activation row is RMS-normed with a gain first (one more pass over the row, which is a few KB in L2): the
// input norm of a sublayer computed by the linear that reads it, in the order (a * scale) * gain of the norm kernel.
// NRT: activation rows dotted per pass (1, 2, 4 or 8). Up to 4 the row loops are branch-free (a pass with fewer rows
// repeats its last row and stores nothing for the repeats), so the loads of several 512-column steps are in flight
// together; inside `if (row < rows)` branches each step waits for its own loads. The 8-row form keeps the branches:
// without them it holds too many registers to keep the chip occupied (measured slower, 1.0 -> 1.36 ms on an 8-row step).
template <typename WT, int SWIGLU, int LR_CPW, int NORM, int NRT>
__global__ void __launch_bounds__(LR_THREADS) lr_gemv_kernel(RowLinear p, int rows_per_group) {
  constexpr int MAXR = NRT;
  // 512-column steps whose loads go out together: fewer where a step already holds many rows x columns in registers
  constexpr bool GUARD = NRT == 8;
  constexpr int LR_WORK = NRT * LR_CPW * (SWIGLU ? 2 : 1);
  constexpr int LR_UNR = GUARD ? 4 : (LR_WORK >= 16 ? 1 : (LR_WORK >= 8 ? 2 : 4));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * (LR_THREADS / 64) + wave) * LR_CPW;
  if (n0 >= p.N) return;
  // rows of this group: a fixed count, one row with its own expert, or (offs) every row of expert blockIdx.y
  int g0 = blockIdx.y * rows_per_group, g1 = min(g0 + rows_per_group, p.R), e = 0;
  if (p.offs) {
    e = blockIdx.y;
    g0 = p.offs[e];
    g1 = p.offs[e + 1];
  } else if (p.row_expert) {
    e = p.row_expert[g0];
    if (e < 0 || e >= p.E) return;  // (a row of an expert without weights, an identity expert: nothing to compute)
  }
  const int K = p.K;
  for (int r0 = g0; r0 < g1; r0 += MAXR) {  // (more than MAXR rows: the weights are streamed again per 8 rows)
  const int nr = min(MAXR, g1 - r0);
  const WT* wbase = reinterpret_cast<const WT*>(p.w) + (size_t)e * p.w_stride;
  const WT* w[LR_CPW];
#pragma unroll
  for (int c = 0; c < LR_CPW; ++c) w[c] = wbase + (size_t)min(n0 + c, p.N - 1) * K;  // (surplus columns re-read the last)
  const size_t up = (size_t)p.N * K;
  const float* a[MAXR];
  float asc[MAXR];
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    const int rr = r0 + min(r, nr - 1);
    a[r] = reinterpret_cast<const float*>(p.a) + (size_t)(p.a_idx ? p.a_idx[rr] : rr) * p.lda;
    asc[r] = p.a_scale ? p.a_scale[rr] : 1.f;
  }
  float nsc[MAXR];
#pragma unroll
  for (int r = 0; r < MAXR; ++r) nsc[r] = 1.f;
  if (NORM) {
    float ss[MAXR];
#pragma unroll
    for (int r = 0; r < MAXR; ++r) ss[r] = 0.f;
#pragma unroll 4
    for (int k = lane * 8; k < K; k += 64 * 8) {
#pragma unroll
      for (int r = 0; r < MAXR; ++r) {
        if (!GUARD || r < nr) {
          float xf[8];
          hy_load8(a[r] + k, K - k, xf);
#pragma unroll
          for (int i = 0; i < 8; ++i) ss[r] = fmaf(xf[i], xf[i], ss[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < MAXR; ++r) nsc[r] = 1.f / sqrtf(wave_sum(ss[r]) / (float)K + p.a_norm_eps);
  }
  float acc[MAXR][LR_CPW], acc2[MAXR][LR_CPW];
#pragma unroll
  for (int r = 0; r < MAXR; ++r)
#pragma unroll
    for (int c = 0; c < LR_CPW; ++c) acc[r][c] = acc2[r][c] = 0.f;
#pragma unroll LR_UNR
  for (int k = lane * 8; k < K; k += 64 * 8) {
    const int left = K - k;
    float wf[LR_CPW][8], uf[LR_CPW][8], gf[8];
#pragma unroll
    for (int c = 0; c < LR_CPW; ++c) {
      hy_load8(w[c] + k, left, wf[c]);
      if (SWIGLU) hy_load8(w[c] + up + k, left, uf[c]);
    }
    if (NORM) hy_load8(p.a_norm_w + k, left, gf);
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      if (!GUARD || r < nr) {
        float xf[8];
        hy_load8(a[r] + k, left, xf);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float xn = NORM ? (xf[i] * nsc[r]) * gf[i] : xf[i];
          const float xv = lr_round(xn * asc[r], wbase);
#pragma unroll
          for (int c = 0; c < LR_CPW; ++c) {
            acc[r][c] = fmaf(xv, wf[c][i], acc[r][c]);
            if (SWIGLU) acc2[r][c] = fmaf(xv, uf[c][i], acc2[r][c]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    if (r < nr) {  // (wave-uniform)
      const int row = r0 + r, drow = p.dst_idx ? p.dst_idx[row] : row;
#pragma unroll
      for (int c = 0; c < LR_CPW; ++c) {
        const float g = wave_sum(acc[r][c]);
        const float u = SWIGLU ? wave_sum(acc2[r][c]) : 0.f;
        if (lane == 0 && n0 + c < p.N) {
          float* dst = reinterpret_cast<float*>(p.out) + (size_t)drow * p.ldo + n0 + c;
          const float val = lr_act(p, g, u);
          *dst = p.add_out ? *dst + val : val;
        }
      }
    }
  }
  }
}

// rows at or below which an expert-sorted batch runs the expert-grouped GEMV (each expert's weights streamed once)
constexpr int HY_GROUPED_GEMV_MAX_R = 64;
// output columns at or below which a dense linear of any row count runs the GEMV
constexpr int HY_SKINNY_MAX_N = 16;

// (the GEMV forms read and write fp32: a bf16 activation copy or a bf16 output always takes the tiles)
static bool lr_fp32_io(const RowLinear& p) { return !p.a_bf16 && !p.out_bf16; }
static bool lr_grouped(const RowLinear& p) { return p.offs && p.R <= HY_GROUPED_GEMV_MAX_R && lr_fp32_io(p); }
static bool lr_skinny(const RowLinear& p) {
  // a handful of output columns (a router): tiles would leave the chip empty, so any number of rows runs the GEMV, each
  // group of 8 rows streaming the few weight rows again
  return !p.offs && !p.row_expert && p.E == 1 && p.N <= HY_SKINNY_MAX_N && !p.a_bf16 && !p.out_bf16 &&
         (p.R + HY_GEMV_MAX_R - 1) / HY_GEMV_MAX_R <= 65535;
}
bool hy_linear_rows_is_gemv(const RowLinear& p) {
  return lr_grouped(p) || lr_skinny(p) || (p.R <= HY_GEMV_MAX_R && (!p.offs || p.row_expert) && lr_fp32_io(p));
}

int hy_linear_rows(const RowLinear& p, hipStream_t s) {
  if (p.R < 0 || p.N <= 0 || p.K <= 0 || p.lda < p.K || p.ldo < p.N || p.E < 1) return -1;
  if (p.act < HY_ACT_NONE || p.act > HY_ACT_SOFTCAP) return -8;
  if (p.act == HY_ACT_SOFTCAP && !(p.act_limit > 0.f)) return -8;
  if (p.add_out && p.out_bf16) return -11;
  if (p.a_scale && p.a_bf16) return -9;  // (a bf16 copy cannot be scaled before its rounding)
  const int gated = hy_act_gated(p.act);
  if (p.R == 0) return 0;
  if (p.offs && p.E > 65535) return -2;
  const bool grouped = lr_grouped(p);
  const bool small = hy_linear_rows_is_gemv(p);
  if (p.a_norm_w && (!small || p.a_bf16)) return -10;  // (the tiles take a normed activation, they do not norm it)
  if (small) {
    if (p.a_bf16 || p.out_bf16) return -7;  // (the GEMV reads and writes fp32)
    // rows per pass: one for per-row experts, the row count rounded up to 2 / 4 / 8 for a dense batch
    // (expert-grouped: 8 per pass over an expert's rows, whose count only the device knows, unless the caller says that
    // every expert has the same few)
    const int want = p.row_expert && !grouped ? 1 : (grouped ? (p.even_rows > 0 ? p.even_rows : HY_GEMV_MAX_R) : p.R);
    const int nrt = want > 4 ? HY_GEMV_MAX_R : (want > 2 ? 4 : (want > 1 ? 2 : 1));
    const int rpg = nrt;
    if (p.a_norm_w && nrt > 2) return -11;  // (the norm-fusing instances exist for one and two rows)
    const int cpw = p.N >= 8192 ? 4 : 1;
    dim3 grid((p.N + 4 * cpw - 1) / (4 * cpw), grouped ? p.E : (p.R + rpg - 1) / rpg);
    RowLinear q = p;
    if (!grouped) q.offs = nullptr;
#define LR_GEMV_N(WT, SW, NORM, NRT)                                                         \
  do {                                                                                       \
    if (cpw == 4) lr_gemv_kernel<WT, SW, 4, NORM, NRT><<<grid, LR_THREADS, 0, s>>>(q, rpg);  \
    else lr_gemv_kernel<WT, SW, 1, NORM, NRT><<<grid, LR_THREADS, 0, s>>>(q, rpg);           \
  } while (0)
#define LR_GEMV(WT, SW)                                  \
  do {                                                   \
    if (p.a_norm_w) {                                    \
      if (nrt == 1) LR_GEMV_N(WT, SW, 1, 1);             \
      else LR_GEMV_N(WT, SW, 1, 2);                      \
    } else if (nrt == 1) LR_GEMV_N(WT, SW, 0, 1);        \
    else if (nrt == 2) LR_GEMV_N(WT, SW, 0, 2);          \
    else if (nrt == 4) LR_GEMV_N(WT, SW, 0, 4);          \
    else LR_GEMV_N(WT, SW, 0, 8);                        \
  } while (0)
    if (p.wbf16) {
      if (gated) LR_GEMV(bf16_t, 1);
      else LR_GEMV(bf16_t, 0);
    } else {
      if (gated) LR_GEMV(float, 1);
      else LR_GEMV(float, 0);
    }
#undef LR_GEMV
#undef LR_GEMV_N
    JLA_CHECK_LAUNCH();
    return 0;
  }
  if (!p.offs && p.E != 1) return -3;
  if ((p.a_bf16 || p.out_bf16) && !p.wbf16) return -5;
  // 128-row tiles once every expert (or the whole batch) has rows to fill them; the SwiGLU form (two accumulator sets)
  // only with many such tiles per expert (measured: 512 rows per expert run faster on 64-row tiles, 4096 on 128-row)
  const long long per_e = p.R / (p.offs ? p.E : 1);
  const int tmm = per_e >= (gated ? 1024 : (p.offs ? 128 : 256)) ? 2 : 1;
  const int bm = LR_BM * tmm;
  const long long mt = (p.R + bm - 1) / bm + (p.offs ? p.E : 0);
  if (mt > 65535) return -4;
  dim3 grid((p.N + LR_BN - 1) / LR_BN, (unsigned)mt);
  RowLinear q = p;
  q.row_expert = nullptr;
#define LR_GEMM(WT, SW, AT, OT)                                                           \
  do {                                                                                    \
    if (tmm == 2) lr_gemm_kernel<WT, SW, AT, OT, 2><<<grid, LR_THREADS, 0, s>>>(q);       \
    else lr_gemm_kernel<WT, SW, AT, OT, 1><<<grid, LR_THREADS, 0, s>>>(q);                \
  } while (0)
  if (p.wbf16) {
    if (p.a_bf16 && p.out_bf16 && gated) LR_GEMM(bf16_t, 1, bf16_t, bf16_t);
    else if (p.a_bf16 && !p.out_bf16 && !gated) LR_GEMM(bf16_t, 0, bf16_t, float);
    else if (p.a_bf16 && p.out_bf16 && !gated) LR_GEMM(bf16_t, 0, bf16_t, bf16_t);
    else if (!p.a_bf16 && p.out_bf16 && gated) LR_GEMM(bf16_t, 1, float, bf16_t);
    else if (!p.a_bf16 && p.out_bf16) LR_GEMM(bf16_t, 0, float, bf16_t);
    else if (p.a_bf16 || p.out_bf16) return -6;  // (combinations nothing uses)
    else if (gated) LR_GEMM(bf16_t, 1, float, float);
    else LR_GEMM(bf16_t, 0, float, float);
  } else {
    if (gated) LR_GEMM(float, 1, float, float);
    else LR_GEMM(float, 0, float, float);
  }
#undef LR_GEMM
  JLA_CHECK_LAUNCH();
  return 0;
}

// ---- routers: (token, choice) rows -> experts, and the counting sort of the rows by expert (one workgroup) -----------
constexpr int RT_MAX_E = 1024;

// Sorts rows [0, R) by row_expert (written before the call by this workgroup; `cnt` holds the per-expert counts):
// offs[E + 1], sort_tok[p] = token of sorted row p, sort_dst[p] = its (token, choice) row, sort_w[p] = its weight.
JLA_DEV void rt_sort(int* cnt, int* cur, int R, int top, int E, const int32_t* row_expert, const float* row_w,
                     int32_t* sort_tok, int32_t* sort_dst, float* sort_w, int32_t* offs) {
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cnt[e];
      cur[e] = run;
      offs[e] = run;
      run += c;
    }
    offs[E] = run;
  }
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += blockDim.x) {
    const int e = row_expert[r];
    const int pos = atomicAdd(&cur[e], 1);
    sort_tok[pos] = r / top;
    sort_dst[pos] = r;
    if (sort_w) sort_w[pos] = row_w[r];
  }
}

__global__ void __launch_bounds__(256) route_table_kernel(const int32_t* ids, const int32_t* table, int V, int M, int top,
                                                          int E, int32_t* row_expert, int32_t* row_tok,
                                                          int32_t* sort_tok, int32_t* sort_dst, int32_t* offs) {
  __shared__ int cnt[RT_MAX_E + 1];
  __shared__ int cur[RT_MAX_E];
  const int R = M * top;
  for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += blockDim.x) {
    const int m = r / top, c = r - m * top;
    int id = ids[m];
    id = id < 0 || id >= V ? 0 : id;
    int e = table[(size_t)id * top + c];
    e = e < 0 || e >= E ? 0 : e;
    row_expert[r] = e;
    row_tok[r] = m;
    atomicAdd(&cnt[e], 1);
  }
  rt_sort(cnt, cur, R, top, E, row_expert, nullptr, sort_tok, sort_dst, nullptr, offs);
}

int hy_route_table(const int32_t* ids, const int32_t* table, int V, int M, int top, int E, int32_t* row_expert,
                   int32_t* row_tok, int32_t* sort_tok, int32_t* sort_dst, int32_t* offs, hipStream_t s) {
  if (M < 0 || top < 1 || E < 1 || E > RT_MAX_E || V < 1) return -1;
  if (M == 0) return 0;
  route_table_kernel<<<1, 256, 0, s>>>(ids, table, V, M, top, E, row_expert, row_tok, sort_tok, sort_dst, offs);
  JLA_CHECK_LAUNCH();
  return 0;
}

// Score router, selection: one wave per token. A lane holds the logits e = lane, lane + 64, ... in registers; each of
// the `top` rounds takes the wave's largest remaining (value, then lower index) and retires it.
constexpr int RK_PER_LANE = RT_MAX_E / 64;

__global__ void __launch_bounds__(256) route_topk_select_kernel(const float* z, int ldz, int M, int top, int E,
                                                                int32_t* row_expert, int32_t* row_tok, float* row_w) {
  const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;
  const float* zr = z + (size_t)m * ldz;
  float v[RK_PER_LANE];
#pragma unroll
  for (int u = 0; u < RK_PER_LANE; ++u) {
    const int e = lane + 64 * u;
    float f = e < E ? zr[e] : -INFINITY;
    v[u] = f == f ? f : -INFINITY;  // (a NaN logit is never chosen ahead of a number)
  }
  for (int c = 0; c < top; ++c) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < RK_PER_LANE; ++u) {
      const int e = lane + 64 * u;
      if (e < E && (v[u] > best || (v[u] == best && e < bi)) && v[u] != -INFINITY) {
        best = v[u];
        bi = e;
      }
    }
#pragma unroll
    for (int off = 32; off; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (bi == 0x7fffffff) {  // fewer than `top` usable logits: the lowest expert not yet taken is not tracked; take 0
      bi = 0;
      best = -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < RK_PER_LANE; ++u)
      if (lane + 64 * u == bi) v[u] = -INFINITY;
    if (lane == 0) {
      const int r = m * top + c;
      row_expert[r] = bi;
      row_tok[r] = m;
      row_w[r] = hy_sigmoid(best);
    }
  }
}

__global__ void route_sort_kernel(int R, int top, int E, const int32_t* row_expert, const float* row_w, int32_t* sort_tok,
                                  int32_t* sort_dst, float* sort_w, int32_t* offs);

// Grouped softmax router, selection: one wave per token, logits in registers as above. Scores = softmax over all E
// logits; choice = score + correction; a group's score is its largest choice; experts outside the `keep` best groups
// are retired before the `top` rounds. The weight of a chosen expert is its score (without the correction).
JLA_DEV void rk_argmax(float& best, int& bi) {  // wave-wide (value, then lower index)
#pragma unroll
  for (int off = 32; off; off >>= 1) {
    const float ob = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    if (ob > best || (ob == best && oi < bi)) {
      best = ob;
      bi = oi;
    }
  }
}

__global__ void __launch_bounds__(256) route_grouped_select_kernel(const float* z, int ldz, const float* correction, int M,
                                                                   int top, int E, int groups, int keep,
                                                                   int32_t* row_expert, int32_t* row_tok, float* row_w) {
  const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;
  const float* zr = z + (size_t)m * ldz;
  float sc[RK_PER_LANE], ch[RK_PER_LANE];
  float zmax = -INFINITY;
#pragma unroll
  for (int u = 0; u < RK_PER_LANE; ++u) {
    const int e = lane + 64 * u;
    const float f = e < E ? zr[e] : -INFINITY;
    sc[u] = f == f ? f : -INFINITY;  // (a NaN logit counts as minus infinity)
    zmax = fmaxf(zmax, sc[u]);
  }
  zmax = wave_max(zmax);
  float den = 0.f;
#pragma unroll
  for (int u = 0; u < RK_PER_LANE; ++u) {
    sc[u] = lane + 64 * u < E ? expf(sc[u] - zmax) : 0.f;
    den += sc[u];
  }
  den = wave_sum(den);
#pragma unroll
  for (int u = 0; u < RK_PER_LANE; ++u) {
    const int e = lane + 64 * u;
    sc[u] = sc[u] / den;
    ch[u] = e < E ? sc[u] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  if (groups > 1) {
    // lane g < groups holds group g's score; `keep` rounds mark the best groups
    const int per = E / groups;
    float gs = -INFINITY;
    for (int g = 0; g < groups; ++g) {
      float mx = -INFINITY;
#pragma unroll
      for (int u = 0; u < RK_PER_LANE; ++u) {
        const int e = lane + 64 * u;
        if (e < E && e / per == g) mx = fmaxf(mx, ch[u]);
      }
      mx = wave_max(mx);
      if (lane == g) gs = mx;
    }
    unsigned long long kept = 0ull;
    for (int c = 0; c < keep; ++c) {
      float best = lane < groups && !((kept >> lane) & 1ull) ? gs : -INFINITY;
      int bi = lane < groups && !((kept >> lane) & 1ull) ? lane : 0x7fffffff;
      rk_argmax(best, bi);
      if (bi != 0x7fffffff) kept |= 1ull << bi;
    }
#pragma unroll
    for (int u = 0; u < RK_PER_LANE; ++u) {
      const int e = lane + 64 * u;
      if (e < E && !((kept >> (e / per)) & 1ull)) ch[u] = -INFINITY;
    }
  }
  unsigned taken[RK_PER_LANE / 32 + 1] = {0};
  for (int c = 0; c < top; ++c) {
    float best = -INFINITY, bw = 0.f;
    int bi = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < RK_PER_LANE; ++u) {
      const int e = lane + 64 * u;
      const bool free_ = !((taken[u >> 5] >> (u & 31)) & 1u);
      if (e < E && free_ && ch[u] != -INFINITY && (ch[u] > best || (ch[u] == best && e < bi))) {
        best = ch[u];
        bi = e;
      }
    }
    rk_argmax(best, bi);
    if (bi == 0x7fffffff) bi = 0;  // fewer than `top` eligible experts (the host checks the sizes): expert 0, weight 0
#pragma unroll
    for (int u = 0; u < RK_PER_LANE; ++u)
      if (lane + 64 * u == bi) {
        taken[u >> 5] |= 1u << (u & 31);
        bw = best == -INFINITY ? 0.f : sc[u];
      }
    bw = wave_sum(bw);  // (one lane holds the chosen expert's score)
    if (lane == 0) {
      const int r = m * top + c;
      row_expert[r] = bi;
      row_tok[r] = m;
      row_w[r] = bw;
    }
  }
}

// The same selection for at most 64 experts, one per lane, without serial rounds: a group's score by per-lane reads of
// its members, then ranks (how many groups / experts come before this one, ties to the lower index) from reads of every
// other lane, all independent of each other. A decode step's router is one token: its latency is what shows.
__global__ void __launch_bounds__(256) route_grouped_select64_kernel(const float* z, int ldz, const float* correction,
                                                                     int M, int top, int E, int groups, int keep,
                                                                     int32_t* row_expert, int32_t* row_tok, float* row_w) {
  const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;
  const bool valid = lane < E;
  float zv = valid ? z[(size_t)m * ldz + lane] : -INFINITY;
  const float cr = valid && correction ? correction[lane] : 0.f;
  zv = zv == zv ? zv : -INFINITY;
  const float zmax = wave_max(zv);
  const float ex = valid ? expf(zv - zmax) : 0.f;
  const float sc = ex / wave_sum(ex);
  float ch = valid ? sc + cr : -INFINITY;
  if (groups > 1) {
    const int per = E / groups, g = min(lane / per, groups - 1);
    float gmax = -INFINITY;
    for (int i = 0; i < per; ++i) gmax = fmaxf(gmax, __shfl(ch, g * per + i, 64));
    int before = 0;  // groups ahead of this lane's
    for (int g2 = 0; g2 < groups; ++g2) {
      const float o = __shfl(gmax, g2 * per, 64);
      before += (o > gmax || (o == gmax && g2 < g)) ? 1 : 0;
    }
    if (before >= keep) ch = -INFINITY;
  }
  int rank = 0;  // experts ahead of this lane's
  for (int e2 = 0; e2 < E; ++e2) {
    const float o = __shfl(ch, e2, 64);
    rank += (o > ch || (o == ch && e2 < lane)) ? 1 : 0;
  }
  if (valid && rank < top) {
    const int r = m * top + rank;
    row_expert[r] = lane;
    row_tok[r] = m;
    row_w[r] = ch == -INFINITY ? 0.f : sc;
  }
}

int hy_route_grouped(const float* z, int ldz, const float* correction, int M, int top, int E, int groups, int keep,
                     int32_t* row_expert, int32_t* row_tok, float* row_w, int32_t* sort_tok, int32_t* sort_dst,
                     float* sort_w, int32_t* offs, hipStream_t s) {
  if (M < 0 || top < 1 || E < 1 || E > RT_MAX_E || ldz < E) return -1;
  if (groups < 1 || groups > 64 || E % groups || keep < 1 || keep > groups || top > keep * (E / groups)) return -3;
  if (M == 0) return 0;
  if (E <= 64)
    route_grouped_select64_kernel<<<(M + 3) / 4, 256, 0, s>>>(z, ldz, correction, M, top, E, groups, keep, row_expert,
                                                              row_tok, row_w);
  else
    route_grouped_select_kernel<<<(M + 3) / 4, 256, 0, s>>>(z, ldz, correction, M, top, E, groups, keep, row_expert,
                                                            row_tok, row_w);
  JLA_CHECK_LAUNCH();
  if (!sort_tok) return 0;
  if (!sort_dst || !sort_w || !offs) return -2;
  route_sort_kernel<<<1, 256, 0, s>>>(M * top, top, E, row_expert, row_w, sort_tok, sort_dst, sort_w, offs);
  JLA_CHECK_LAUNCH();
  return 0;
}

__global__ void __launch_bounds__(256) route_sort_kernel(int R, int top, int E, const int32_t* row_expert,
                                                         const float* row_w, int32_t* sort_tok, int32_t* sort_dst,
                                                         float* sort_w, int32_t* offs) {
  __shared__ int cnt[RT_MAX_E + 1];
  __shared__ int cur[RT_MAX_E];
  for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < R; r += blockDim.x) atomicAdd(&cnt[row_expert[r]], 1);
  rt_sort(cnt, cur, R, top, E, row_expert, row_w, sort_tok, sort_dst, sort_w, offs);
}

int hy_route_topk(const float* z, int ldz, int M, int top, int E, int32_t* row_expert, int32_t* row_tok, float* row_w,
                  int32_t* sort_tok, int32_t* sort_dst, float* sort_w, int32_t* offs, hipStream_t s) {
  if (M < 0 || top < 1 || E < 1 || E > RT_MAX_E || top > E || ldz < E) return -1;
  if (M == 0) return 0;
  route_topk_select_kernel<<<(M + 3) / 4, 256, 0, s>>>(z, ldz, M, top, E, row_expert, row_tok, row_w);
  JLA_CHECK_LAUNCH();
  if (!sort_tok) return 0;
  if (!sort_dst || !sort_w || !offs) return -2;
  route_sort_kernel<<<1, 256, 0, s>>>(M * top, top, E, row_expert, row_w, sort_tok, sort_dst, sort_w, offs);
  JLA_CHECK_LAUNCH();
  return 0;
}

}  // namespace jla
