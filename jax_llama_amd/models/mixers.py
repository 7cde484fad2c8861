"""Building blocks of layer-list decoders (``models/zavevik.py``): each block is a thin view over one layer's weights
that issues the ``ops.hybrid`` kernels, like ``models/modules.py`` does for LLaMA. Every constant is a constructor
argument (taken from the layer's ``MixerSpec`` / ``MoESpec``), so another architecture of the registry can assemble
the same mechanisms with other values.

  BiasedAttention : fused q|k|v projection, per-head RMS-normed q / k / v, query temperature, cache write; soft-capped
                    scores + learned distance bias + causal softmax; o projection. May read another layer's keys and
                    values (``kv_from``) -- then it projects queries only.
  GatedDeltaMixer : fused q|k|v|gate|b|a projection, short causal convolutions + SiLU, unit-length q / k, the gated
                    delta-rule recurrence over a carried fp32 state, gated RMS norm, o projection.
  TableMoE        : mixture of SwiGLU experts chosen by a token-id table (no router), averaged.
  TokenSide       : per-layer token-side input: gelu_tanh(gate x) * (slice of a second embedding), projected back,
                    RMS-normed with a vector gain, added to the residual.
  LatentAttention : attention over one cached low-rank vector per token, per-head key / value maps applied around the
                    attention, a learned sink in the softmax, no positions.
  DenseFF         : dense feed-forward with a one-accumulator activation (squared ReLU).
  RoutedMoE       : sigmoid-score top-k router, input-weighted clamped-gate experts, gated shared expert.
  SandwichNormBlock : RMS norms on both sides of each sublayer, per-channel output gains.
  RotaryChunkAttention : projection biases, rotary positions on part of each q / k head, values cached rotated by their
                    position with the sum turned back, block-local causal mask, per-head temperature and sink.
  MatrixLSTM      : matrix memory with capped exponential gates, a running maximum and a normaliser.
  TimeMix         : token-shifted projections, per-channel decay from a low-rank map, bonus for the current token.
  SideBySide      : several mixers on one input, their features concatenated in front of one output matrix.
  GatedDenseFF    : dense feed-forward with a two-accumulator (gated) activation.
  PreNormBlock    : ``x += sublayer(rms_norm(x))`` with the residual add in the output projection's epilogue.

  RotaryLatentAttention : latent attention whose queries go through a normed latent too, with one rotated key part per
                    token shared by all heads, a sliding window and a sigmoid gate per head on the output.
  NormedGatedAttention : attention without positions: weighted per-head RMS norm of q and k, a sliding window that may
                    keep the sequence's first keys, a sigmoid gate per head on the output.
  GroupedMoE      : softmax-score router with a selection bias, expert groups and identity experts; squared-ReLU experts
                    weighted on their output; a shared expert.
  HyperBlock      : pre-norm sublayers over several residual streams (hyper-connections): a sublayer reads a weighted
                    sum of the streams, and its result is added to a mixed copy of them.

The blocks of the group before the last split a sublayer into ``features(h, ctx, out=None, gain=1.0)`` (everything up to the output
projection; ``out`` a column slice to write into, ``gain`` a scalar folded into the last elementwise step) and the
matrix ``w_o``, so a block can fuse the projection with the residual add and ``SideBySide`` can run one projection for
all of its members.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import hybrid as hy


@dataclass
class StepContext:
    """What one forward step hands to every block: the tokens, where they sit, and the cache."""

    ids: torch.Tensor        # int32 [B * S]
    positions: torch.Tensor  # int32 [B * S]
    b: int
    s: int
    cache: object            # HybridCache (or a row view)
    slot0: object            # int, or device int32[1] (graph-capturable)
    u: Optional[torch.Tensor] = None  # hyper-connected stacks: the next sublayer's input sum, left by the last write


class BiasedAttention:
    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, w_o: torch.Tensor,
                 bias_by_distance: Optional[torch.Tensor]):
        self.i = layer_idx
        self.spec = spec
        self.eps = eps
        self.w_in = w_in            # [H dim (+ G dim + G vdim), D]
        self.w_o = w_o              # [D, H vdim]
        self.bias = bias_by_distance  # fp32 [bias_max + 1, H] or None

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        proj = hy.linear(x, self.w_in)
        kc, vc = ctx.cache.layer(self.i)
        own = sp.kv_from is None
        q = hy.attn_prep(proj, ctx.positions, ctx.slot0, ctx.b, ctx.s, sp.heads, sp.kv_heads, sp.dim, sp.vdim,
                         kc if own else None, vc if own else None, self.eps, sp.q_temp_coef, sp.q_temp_every)
        a = hy.attn_bias(q, kc, vc, ctx.slot0, sp.scale, sp.softcap, self.bias)
        return hy.linear(a, self.w_o)


class GatedDeltaMixer:
    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, conv_w: torch.Tensor,
                 a_log: torch.Tensor, dt_bias: torch.Tensor, norm_w: torch.Tensor, w_o: torch.Tensor):
        self.i = layer_idx
        self.spec = spec
        self.eps = eps
        self.w_in = w_in      # [2 G dim + 2 H vdim + 2 H, D]: q | k | v | gate | b | a
        self.conv_w = conv_w  # fp32 [2 G dim + H vdim, taps]
        self.a_log, self.dt_bias, self.norm_w = a_log, dt_bias, norm_w
        self.w_o = w_o

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        proj = hy.linear(x, self.w_in)
        state, tail = ctx.cache.recurrent(self.i)
        q, k, v, beta, decay = hy.delta_prep(proj, ctx.b, ctx.s, sp.heads, sp.kv_heads, sp.dim, sp.vdim, self.conv_w,
                                             tail, self.a_log, self.dt_bias)
        o = hy.delta_scan(q, k, v, beta, decay, state, ctx.b, ctx.s)
        c = 2 * sp.kv_heads * sp.dim + sp.heads * sp.vdim
        gate = proj[:, c:c + sp.heads * sp.vdim]
        return hy.linear(hy.gated_rmsnorm(o, gate, self.norm_w, self.eps), self.w_o)


class TableMoE:
    def __init__(self, spec, table: torch.Tensor, w_gu: torch.Tensor, w_down: torch.Tensor):
        self.spec = spec
        self.table = table    # int32 [vocab, top]
        self.w_gu = w_gu      # [E, 2 ff, D] gate rows then up rows
        self.w_down = w_down  # [E, D, ff]

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        """The chosen experts' outputs ``[M * top, D]``; the caller's output norm averages them."""
        return hy.moe_table(x, ctx.ids, self.table, self.w_gu, self.w_down)


class TokenSide:
    def __init__(self, table: torch.Tensor, col0: int, w_gate: torch.Tensor, w_proj: torch.Tensor, norm_w: torch.Tensor,
                 eps: float):
        self.table, self.col0 = table, col0
        self.w_gate, self.w_proj, self.norm_w, self.eps = w_gate, w_proj, norm_w, eps

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> None:
        g = hy.gelu_gate_rows(hy.linear(x, self.w_gate), ctx.ids, self.table, self.col0)
        hy.norm_residual_(x, hy.linear(g, self.w_proj), self.norm_w, self.eps)


class OutputNormBlock:
    """``x += norm1(mixer(x)); x += norm2(ff(x)); x += side(x)``: the norm sits on each sublayer's OUTPUT (a scalar
    gain), the sublayers read the residual itself."""

    def __init__(self, mixer, norm1: torch.Tensor, mlp: Optional[TableMoE], norm2: Optional[torch.Tensor],
                 side: Optional[TokenSide], eps: float):
        self.mixer, self.norm1, self.mlp, self.norm2, self.side, self.eps = mixer, norm1, mlp, norm2, side, eps

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> None:
        hy.norm_residual_(x, self.mixer(x, ctx), self.norm1, self.eps)
        if self.mlp is not None:
            top = self.mlp.spec.top
            hy.norm_residual_(x, self.mlp(x, ctx), self.norm2, self.eps, nsum=top, ysc=1.0 / top)
        if self.side is not None:
            self.side(x, ctx)


class LatentAttention:
    """Attention over one cached vector per token (``kv_rank`` numbers, RMS-normed with a plain gain) from which every
    head's keys and values are linear maps. No positions; a learned per-head sink joins the softmax denominator. Two
    forms of the same sums, chosen per step by their cost:

    * in the latent space (decode, short portions): a head's query is mapped through its key map first
      (``q' = W_uk[h]^T q``), all heads attend over the shared latent (keys = values = the cache, one cache head), and
      the head's value map is applied to the attended latent. Nothing per cached token is computed.
    * expanded (long portions): keys and values of every head are computed from the cached latents of the whole prefix
      into scratch tensors, and the heads attend over those at their own (smaller) sizes."""

    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, dkv_norm: torch.Tensor,
                 w_uk: torch.Tensor, w_uv: torch.Tensor, sink: Optional[torch.Tensor], w_o: torch.Tensor):
        self.i = layer_idx
        self.spec = spec
        self.eps = eps
        self.w_in = w_in          # [H dim + rank, D]: queries, then the down projection
        self.dkv_norm = dkv_norm  # fp32 [rank]
        self.w_uk = w_uk          # [H, dim, rank]
        self.w_qk = w_uk.transpose(1, 2).contiguous()  # [H, rank, dim]: queries into the latent space
        self.w_uv = w_uv          # [H, vdim, rank]
        self.sink = sink          # fp32 [H] or None
        self.w_o = w_o            # [D, H vdim]

    # head sizes the MFMA attention kernels take (others run the plain kernels, several times slower per product)
    MMA_SIZES = (64, 128)
    PLAIN_KERNEL_COST = 8.0
    EXPAND_MIN_TOKENS = 16

    def expands(self, s: int, n: int, bf16: bool) -> bool:
        """Whether a step of ``s`` tokens ending at ``n`` cached tokens runs the expanded form: multiply-adds of both
        forms, attention products on the plain kernels weighted by ``PLAIN_KERNEL_COST``."""
        sp = self.spec
        if s < self.EXPAND_MIN_TOKENS:
            return False
        pairs = s * (n - s) + s * (s + 1) / 2.0
        plain = lambda *sizes: 1.0 if bf16 and all(x in self.MMA_SIZES for x in sizes) else self.PLAIN_KERNEL_COST  # noqa: E731
        latent = s * sp.kv_rank * (sp.dim + sp.vdim) + pairs * 2.0 * sp.kv_rank * plain(sp.kv_rank)
        expanded = n * sp.kv_rank * (sp.dim + sp.vdim) + pairs * (sp.dim + sp.vdim) * plain(sp.dim, sp.vdim)
        return expanded < latent

    def __call__(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        m, nh, rank = ctx.b * ctx.s, sp.heads, sp.kv_rank
        proj = hy.linear(h, self.w_in)
        c, _ = ctx.cache.layer(self.i)
        q = hy.latent_prep(proj, nh * sp.dim, self.dkv_norm, ctx.slot0, ctx.b, ctx.s, c, self.eps, q_cols=nh * sp.dim)
        n = (ctx.cache.index if torch.is_tensor(ctx.slot0) else int(ctx.slot0)) + ctx.s  # (host mirror of the slot)
        # (a latent wider than the attention kernels' head limit can only be attended in the expanded form, whose key
        # count is a host number: such a layer cannot be part of a captured decode step)
        wide = rank > hy.ATTN_MAX_HEAD
        if wide and c.is_cuda and torch.cuda.is_current_stream_capturing():
            raise NotImplementedError(f"latent attention: kv_rank {rank} > {hy.ATTN_MAX_HEAD} in a captured step")
        if wide or (ctx.s > 1 and self.expands(ctx.s, n, c.dtype == torch.bfloat16)):
            k, v = hy.latent_expand(c, n, self.w_uk), hy.latent_expand(c, n, self.w_uv)
            o = hy.attn_bias(q.reshape(ctx.b, ctx.s, nh, sp.dim), k, v, ctx.slot0, sp.scale, sink=self.sink)
            return hy.linear(o, self.w_o)
        ql = hy.heads_linear(q.reshape(m, nh, sp.dim), self.w_qk)
        a = hy.attn_bias(ql.reshape(ctx.b, ctx.s, nh, rank), c, c, ctx.slot0, sp.scale, sink=self.sink)
        o = hy.heads_linear(a.reshape(m, nh, rank), self.w_uv)
        return hy.linear(o.reshape(m, nh * sp.vdim), self.w_o)


@dataclass
class FFOut:
    """A feed-forward's result before the block's output norm: ``y [M * nsum, D]`` (a token's ``nsum`` rows are summed)
    plus an optional per-token summand ``extra [M, D]`` weighted by ``sigmoid(extra_gate [M, 1])``."""

    y: torch.Tensor
    nsum: int = 1
    extra: Optional[torch.Tensor] = None
    extra_gate: Optional[torch.Tensor] = None


class DenseFF:
    """``W_down act(W_up h)`` with a one-accumulator activation (squared ReLU by default)."""

    def __init__(self, w_up: torch.Tensor, w_down: torch.Tensor, act: int = hy.ACT_RELU2):
        self.w_up, self.w_down, self.act = w_up, w_down, act

    def __call__(self, h: torch.Tensor, ctx: StepContext) -> FFOut:
        return FFOut(hy.ff_dense(h, self.w_up, self.w_down, self.act))


class RoutedMoE:
    """Mixture of clamped-gate experts chosen by a sigmoid-score router: the ``top`` largest scores per token, the
    scores themselves as weights (not renormalised), each weight applied to its expert's INPUT. An optional shared
    expert runs for every token, weighted on its output by the sigmoid of one more router row. The router (and the
    shared gate) is an fp32 matrix in both number formats."""

    def __init__(self, experts: int, top: int, limit: float, alpha: float, w_router: torch.Tensor, w_gu: torch.Tensor,
                 w_down: torch.Tensor, shared_gu: Optional[torch.Tensor] = None,
                 shared_down: Optional[torch.Tensor] = None, shared_limit: float = 0.0):
        self.experts, self.top, self.limit, self.alpha = experts, top, limit, alpha
        self.w_router = w_router  # fp32 [E (+ 1), D]: expert rows, then the shared expert's gate row
        self.w_gu = w_gu          # [E, 2 ff, D]
        self.w_down = w_down      # [E, D, ff]
        self.shared_gu, self.shared_down, self.shared_limit = shared_gu, shared_down, shared_limit

    def __call__(self, h: torch.Tensor, ctx: StepContext) -> FFOut:
        z = hy.linear(h, self.w_router)
        y = hy.moe_routed(h, z, self.top, self.w_gu, self.w_down, hy.ACT_CLAMP_GLU, self.limit, self.alpha)
        if self.shared_gu is None:
            return FFOut(y, self.top)
        hs = hy.linear(h, self.shared_gu, act=hy.ACT_CLAMP_GLU, limit=self.shared_limit, alpha=self.alpha)
        return FFOut(y, self.top, hy.linear(hs, self.shared_down), z[:, self.experts:self.experts + 1])


class SandwichNormBlock:
    """``x += post1 * rms(mixer(pre1 * rms(x)))``, ``x += post2 * rms(ff(pre2 * rms(x)))``: an RMS norm on each
    sublayer's input and another on its output. The gains are fp32 vectors prepared by the loader (a norm stored
    around zero arrives as ``1 + w``; a per-channel layer scale is folded into the output gain)."""

    def __init__(self, mixer, pre1: torch.Tensor, post1: torch.Tensor, mlp, pre2: Optional[torch.Tensor],
                 post2: Optional[torch.Tensor], eps: float):
        self.mixer, self.pre1, self.post1 = mixer, pre1, post1
        self.mlp, self.pre2, self.post2, self.eps = mlp, pre2, post2, eps

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> None:
        # (the sublayers read their input through hy.linear / hy.moe_routed, whose GEMVs apply the input norm themselves)
        hy.norm_residual_(x, self.mixer(hy.RmsInput(x, self.pre1, self.eps), ctx), self.post1, self.eps)
        if self.mlp is not None:
            f = self.mlp(hy.RmsInput(x, self.pre2, self.eps), ctx)
            hy.norm_residual_(x, f.y, self.post2, self.eps, nsum=f.nsum, extra=f.extra, extra_gate=f.extra_gate)


def _value(h):
    return h.value() if isinstance(h, hy.RmsInput) else h


class RotaryChunkAttention:
    """Softmax attention over this layer's own keys and values with: one bias per projection column; rotary positions
    on the first ``rot_dims`` numbers of every q / k head (number ``i`` paired with ``i + rot_dims / 2``); optionally
    (``v_freq``) values rotated by their own position over the whole head before they are cached, and each head's summed
    values turned back by the query's position; score ``q . k * scale * temp[h]``; optionally (``chunk``) a query sees
    only the keys of its own block of ``chunk`` positions; optionally a learned sink per head in the denominator."""

    def __init__(self, layer_idx: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, w_in: torch.Tensor,
                 bias: Optional[torch.Tensor], qk_freq: torch.Tensor, v_freq: Optional[torch.Tensor],
                 temp: Optional[torch.Tensor], sink: Optional[torch.Tensor], chunk: int, w_o: torch.Tensor):
        self.i = layer_idx
        self.heads, self.kv_heads, self.dim, self.vdim, self.scale = heads, kv_heads, dim, vdim, scale
        self.w_in = w_in        # [H dim + G dim + G vdim, D]
        self.bias = bias        # fp32 [H dim + G dim + G vdim] or None
        self.qk_freq = qk_freq  # float64 [rot_dims / 2]
        self.v_freq = v_freq    # float64 [vdim / 2] or None
        self.temp, self.sink, self.chunk = temp, sink, chunk  # fp32 [H], fp32 [H], block length (0: causal only)
        self.w_o = w_o          # [D, H vdim]
        self.width = heads * vdim

    def features(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None, gain: float = 1.0) -> torch.Tensor:
        proj = hy.linear(h, self.w_in)
        kc, vc = ctx.cache.layer(self.i)
        q = hy.rope_prep(proj, self.bias, ctx.positions, ctx.slot0, ctx.b, ctx.s, self.heads, self.kv_heads, self.dim,
                         self.vdim, kc, vc, self.qk_freq, self.v_freq)
        a = hy.attn_bias(q, kc, vc, ctx.slot0, self.scale, sink=self.sink, chunk=self.chunk, head_scale=self.temp)
        if self.v_freq is None and out is None and gain == 1.0:
            return a
        return hy.rotate_heads(a, ctx.positions, self.v_freq, self.heads, sign=-1.0, gain=gain, out=out)

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        return hy.linear(self.features(h, ctx), self.w_o)


class MatrixLSTM:
    """Matrix memory with exponential gates. Per head, with the capped gate pre-activations ``a`` (input) and ``f``
    (log forget) and the running maximum ``m``: ``S <- e^(f + m' - m) S + e^(a - m) k v^T``, the normaliser ``z``
    likewise with ``k`` alone, ``o = S^T q / (max(|z . q|, e^-m) + 1e-6)`` with ``q`` scaled by ``dim^-1/2``; then each
    head's ``o`` over its root mean square, times a gain per column, times ``sigmoid(gate)``."""

    def __init__(self, layer_idx: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, w_in: torch.Tensor,
                 gate_bias: torch.Tensor, norm_w: torch.Tensor, w_o: torch.Tensor):
        self.i = layer_idx
        self.heads, self.dim, self.vdim, self.cap, self.eps = heads, dim, vdim, gate_cap, eps
        self.w_in = w_in            # [2 H dim + 2 H vdim + 2 H, D]: q | k | v | gate | input gate | forget gate
        self.gate_bias = gate_bias  # fp32 [2 H]: input-gate biases, then forget-gate biases
        self.norm_w = norm_w        # fp32 [H vdim]
        self.w_o = w_o              # [D, H vdim]
        self.width = heads * vdim

    def features(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None, gain: float = 1.0) -> torch.Tensor:
        nh, dim, vdim, m = self.heads, self.dim, self.vdim, ctx.b * ctx.s
        proj = hy.linear(h, self.w_in)
        state, mrun = ctx.cache.recurrent(self.i)
        qk, vv = nh * dim, nh * vdim
        keep, write, floor = hy.mlstm_prep(proj, 2 * qk + 2 * vv, 2 * qk + 2 * vv + nh, self.gate_bias, self.cap, mrun,
                                           ctx.b, ctx.s, nh)
        o = hy.mlstm_scan(proj[:, :qk].unflatten(1, (nh, dim)), proj[:, qk:2 * qk].unflatten(1, (nh, dim)),
                          proj[:, 2 * qk:2 * qk + vv].unflatten(1, (nh, vdim)), keep, write, state, ctx.b, ctx.s,
                          q_scale=dim ** -0.5)
        return hy.gated_rmsnorm(o, proj[:, 2 * qk + vv:2 * qk + 2 * vv], self.norm_w, self.eps, hy.GATE_SIGMOID,
                                denom_floor=floor, gain=gain, out=out)

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        return hy.linear(self.features(h, ctx), self.w_o)


class TimeMix:
    """Token-shifted linear recurrence. Each of the five projections reads its own blend of the current and the
    previous token's input (``h + (h' - h) mu``); receptance, key, value per head; gate ``silu(.)``; a decay per key
    channel ``exp(-exp(W_2 tanh(W_1 .) + w0))``; per head ``o = (S + diag(u) k v^T)^T r``, ``S <- diag(d) S + k v^T``;
    then each head's ``o`` over its root mean square, times a gain per column, times the gate."""

    def __init__(self, layer_idx: int, heads: int, dim: int, eps: float, mu: torch.Tensor, w_rkvg: torch.Tensor,
                 w_d1: torch.Tensor, w_d2: torch.Tensor, w0: torch.Tensor, u: torch.Tensor, norm_w: torch.Tensor,
                 w_o: torch.Tensor):
        self.i = layer_idx
        self.heads, self.dim, self.eps = heads, dim, eps
        self.mu = mu          # fp32 [5, D]: blends of r, k, v, gate, decay
        self.w_rkvg = w_rkvg  # [4, H dim, D]
        self.w_each = list(w_rkvg.unbind(0))  # (the same four view objects at every call: weight-keyed caches hit)
        self.w_d1, self.w_d2 = w_d1, w_d2  # [rank, D], [H dim, rank]
        self.w0, self.u = w0, u            # fp32 [H, dim]
        self.norm_w = norm_w  # fp32 [H dim]
        self.w_o = w_o        # [D, H dim]
        self.width = heads * dim

    def features(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None, gain: float = 1.0) -> torch.Tensor:
        nh, dim, m = self.heads, self.dim, ctx.b * ctx.s
        state, prev = ctx.cache.recurrent(self.i)
        mixes = hy.token_shift(_value(h), prev, self.mu, ctx.b, ctx.s)
        if 4 * m <= hy.STACKED_MAX_ROWS:  # a few tokens: the four same-shaped projections as one grouped launch
            r, k, v, g = hy.stacked_linear(mixes[:4], self.w_rkvg).unbind(0)
        else:
            r, k, v, g = (hy.linear(mixes[j], self.w_each[j]) for j in range(4))
        wpre = hy.linear(hy.linear_softcap(mixes[4], self.w_d1, 1.0), self.w_d2)
        hd = (nh, dim)
        o = hy.timemix_scan(r.unflatten(1, hd), k.unflatten(1, hd), v.unflatten(1, hd), wpre.unflatten(1, hd), self.w0,
                            self.u, state, ctx.b, ctx.s)
        return hy.gated_rmsnorm(o, g, self.norm_w, self.eps, hy.GATE_SILU, gain=gain, out=out)

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        return hy.linear(self.features(h, ctx), self.w_o)


class SideBySide:
    """Mixers that read the same input; the result is ``sum_k scale_k * mixer_k(h)``. Their features are written side by
    side (each scaled by its weight in its last elementwise step) and multiplied by the members' output matrices laid
    side by side: one projection for all of them."""

    def __init__(self, members, scales):
        self.members, self.scales = list(members), [float(x) for x in scales]
        self.w_o = torch.cat([mm.w_o for mm in self.members], 1).contiguous()
        self.width = sum(mm.width for mm in self.members)

    def features(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None, gain: float = 1.0) -> torch.Tensor:
        hv = _value(h)
        if out is None:
            out = torch.empty(ctx.b * ctx.s, self.width, dtype=torch.float32, device=hv.device)
        c = 0
        for mm, sc in zip(self.members, self.scales):
            mm.features(hv, ctx, out=out[:, c:c + mm.width], gain=gain * sc)
            c += mm.width
        return out

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        return hy.linear(self.features(h, ctx), self.w_o)


class GatedDenseFF:
    """``W_down act(W_gate h, W_up h)`` with a two-accumulator activation (the clamped gate by default:
    ``g' sigmoid(alpha g') (u' + 1)``, ``g' = min(g, limit)``, ``u' = clamp(u, -limit, limit)``)."""

    def __init__(self, w_gu: torch.Tensor, w_down: torch.Tensor, limit: float, alpha: float, act: int = hy.ACT_CLAMP_GLU):
        self.w_gu, self.w_o, self.limit, self.alpha, self.act = w_gu, w_down, limit, alpha, act

    def features(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None, gain: float = 1.0) -> torch.Tensor:
        return hy.linear(h, self.w_gu, act=self.act, limit=self.limit, alpha=self.alpha)

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        return hy.linear(self.features(h, ctx), self.w_o)


class PreNormBlock:
    """``x += mixer(norm1 * rms(x))``, ``x += ff(norm2 * rms(x))``: vector gains on the sublayers' inputs, the residual
    add in the epilogue of each sublayer's output projection."""

    def __init__(self, mixer, norm1: torch.Tensor, mlp, norm2: Optional[torch.Tensor], eps: float):
        self.mixer, self.norm1, self.mlp, self.norm2, self.eps = mixer, norm1, mlp, norm2, eps

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> None:
        hy.linear_add_(x, self.mixer.features(hy.RmsInput(x, self.norm1, self.eps), ctx), self.mixer.w_o)
        if self.mlp is not None:
            hy.linear_add_(x, self.mlp.features(hy.RmsInput(x, self.norm2, self.eps), ctx), self.mlp.w_o)


class RotaryLatentAttention(LatentAttention):
    """Latent attention with positions. Per token the cache holds ``kv_rank`` RMS-normed numbers (from which every head's
    plain keys and its values are linear maps) followed by ``rot_dim`` numbers rotated by the token's position: one
    rotated key part shared by all heads. Queries come from a latent of their own (down projection, RMS norm with a plain
    gain, up projection) and are laid out per head as ``dim`` plain numbers, then ``rot_dim`` rotated ones; the score is
    ``(q_plain . k_plain + q_rot . k_rot) * scale``. Rotation pairs number ``2i`` with ``2i + 1``. ``window > 0``: a
    query sees the last ``window`` positions (and the first ``keep_first`` of the sequence). Each head's output is
    multiplied by the sigmoid of one more projection of the mixer's input.

    Both forms of ``LatentAttention`` carry over with the rotated part as ``rot_dim`` more key numbers: in the latent
    space a head's query becomes ``[W_uk[h]^T q_plain | q_rot]`` against the cache row itself (the values are the row's
    first ``kv_rank`` numbers); expanded, a head's key is ``[W_uk[h] c | k_rot]``. The maps are stored with an identity
    block for the rotated part, so both run as the same per-head linears."""

    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, dq_norm: torch.Tensor, w_uq: torch.Tensor,
                 dkv_norm: torch.Tensor, w_uk: torch.Tensor, w_uv: torch.Tensor, freq: Optional[torch.Tensor],
                 w_o: torch.Tensor, gated: bool = True):
        self.i = layer_idx
        self.gated = gated        # whether w_in ends with one gate row per head
        self.spec = spec
        self.eps = eps
        self.w_in = w_in          # [q_rank + kv_rank + rot_dim (+ H), D]: query latent, key / value latent, rotated key, gates
        self.dq_norm, self.dkv_norm = dq_norm, dkv_norm  # fp32 [q_rank], [kv_rank]
        self.w_uq = w_uq          # [H (dim + rot_dim), q_rank]
        self.freq = freq          # float64 [rot_dims / 2] or None
        self.w_o = w_o            # [D, H vdim]
        nh, dim, rot, rank = spec.heads, spec.dim, spec.rot_dim, spec.kv_rank
        eye = torch.eye(rot, dtype=w_uk.dtype, device=w_uk.device)
        wk = torch.zeros(nh, dim + rot, rank + rot, dtype=w_uk.dtype, device=w_uk.device)
        wk[:, :dim, :rank] = w_uk
        wk[:, dim:, rank:] = eye
        self.w_uk = wk                                   # [H, dim + rot, rank + rot]: a head's keys from a cache row
        self.w_qk = wk.transpose(1, 2).contiguous()      # [H, rank + rot, dim + rot]: queries into the cache row's space
        wv = torch.zeros(nh, spec.vdim, rank + rot, dtype=w_uv.dtype, device=w_uv.device)
        wv[:, :, :rank] = w_uv
        self.w_uv_row = wv        # [H, vdim, rank + rot]: a head's values from a cache row
        self.w_uv = w_uv          # [H, vdim, rank]: ... from the attended latent

    def expands(self, s: int, n: int, bf16: bool) -> bool:
        sp = self.spec
        if s < self.EXPAND_MIN_TOKENS:
            return False
        seen = min(n, sp.window + sp.keep_first) if sp.window else n
        pairs = s * min(seen, (n - s) + (s + 1) / 2.0)
        row, kd = sp.kv_rank + sp.rot_dim, sp.dim + sp.rot_dim
        mma = bf16 and kd in self.MMA_SIZES and sp.vdim in self.MMA_SIZES
        # (in the latent space keys and values differ in width: always the plain kernels)
        latent = s * row * (kd + sp.vdim) + pairs * (row + sp.kv_rank) * self.PLAIN_KERNEL_COST
        expanded = min(n, s + seen) * row * (kd + sp.vdim) + pairs * (kd + sp.vdim) * (1.0 if mma else self.PLAIN_KERNEL_COST)
        return expanded < latent

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        m, nh, rank, rot = ctx.b * ctx.s, sp.heads, sp.kv_rank, sp.rot_dim
        kd, row = sp.dim + rot, rank + rot
        proj = hy.linear(h, self.w_in)
        c, _ = ctx.cache.layer(self.i)
        cq = hy.latent_rope_prep(proj, 0, self.dq_norm, sp.q_rank, self.dkv_norm, self.freq, ctx.positions, ctx.slot0,
                                 ctx.b, ctx.s, c, self.eps)
        q = hy.linear(cq, self.w_uq)
        if self.freq is not None:
            hy.rotate_heads(q, ctx.positions, self.freq, nh, out=q, offset=sp.dim, interleaved=True)
        gate = proj[:, sp.q_rank + row:sp.q_rank + row + nh] if self.gated else None
        s0 = ctx.cache.index if torch.is_tensor(ctx.slot0) else int(ctx.slot0)  # (host mirror of the slot)
        n = s0 + ctx.s
        wide = row > hy.ATTN_MAX_KEY or rank > hy.ATTN_MAX_HEAD
        if wide and c.is_cuda and torch.cuda.is_current_stream_capturing():
            raise NotImplementedError(f"latent attention: a cache row of {rank} + {rot} in a captured step")
        if wide or (ctx.s > 1 and self.expands(ctx.s, n, c.dtype == torch.bfloat16)):
            # only the keys some query of the step can see are expanded: with a window and no kept first keys, the
            # scratch keys start at `first` and the step's slot is counted from there
            first = max(0, s0 - sp.window + 1) // 64 * 64 if sp.window and not sp.keep_first else 0
            k = hy.latent_expand(c, n, self.w_uk, first)
            v = hy.latent_expand(c, n, self.w_uv_row, first)
            o = hy.attn_bias(q.reshape(ctx.b, ctx.s, nh, kd), k, v, ctx.slot0 if first == 0 else s0 - first, sp.scale,
                             window=sp.window, keep_first=sp.keep_first, gate=gate)
            return hy.linear(o, self.w_o)
        ql = hy.heads_linear(q.reshape(m, nh, kd), self.w_qk)
        a = hy.attn_bias(ql.reshape(ctx.b, ctx.s, nh, row), c, c, ctx.slot0, sp.scale, window=sp.window,
                         keep_first=sp.keep_first, gate=gate, vdim=rank)
        o = hy.heads_linear(a.reshape(m, nh, rank), self.w_uv)
        return hy.linear(o.reshape(m, nh * sp.vdim), self.w_o)


class NormedGatedAttention:
    """Softmax attention over this layer's own keys and values, without positions: every q / k head is divided by its
    root mean square and multiplied by a gain vector shared by all heads (``q_norm`` / ``k_norm [dim]``), values are
    cached as projected; ``window > 0``: a query sees the last ``window`` positions and the first ``keep_first`` of the
    sequence; each head's output is multiplied by the sigmoid of one more projection of the mixer's input."""

    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, q_norm: Optional[torch.Tensor],
                 k_norm: Optional[torch.Tensor], gated: bool, w_o: torch.Tensor):
        self.i = layer_idx
        self.spec = spec
        self.eps = eps
        self.w_in = w_in  # [H dim + G dim + G vdim (+ H), D]: q | k | v | gates
        self.q_norm, self.k_norm, self.gated = q_norm, k_norm, gated
        self.w_o = w_o    # [D, H vdim]

    def __call__(self, h, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        proj = hy.linear(h, self.w_in)
        cols = (sp.heads + sp.kv_heads) * sp.dim + sp.kv_heads * sp.vdim
        kc, vc = ctx.cache.layer(self.i)
        q = hy.attn_prep(proj[:, :cols], ctx.positions, ctx.slot0, ctx.b, ctx.s, sp.heads, sp.kv_heads, sp.dim, sp.vdim,
                         kc, vc, self.eps, q_w=self.q_norm, k_w=self.k_norm, norm_v=False)
        gate = proj[:, cols:cols + sp.heads] if self.gated else None
        a = hy.attn_bias(q, kc, vc, ctx.slot0, sp.scale, window=sp.window, keep_first=sp.keep_first, gate=gate)
        return hy.linear(a, self.w_o)


@dataclass
class MixtureOut:
    """A mixture's result before it is summed: ``y [M * nsum, D]`` with a weight and an expert per row (rows of experts
    ``>= n_real`` stand for identity experts: the weight times ``ident [M, D]``), plus a per-token summand ``extra``."""

    y: torch.Tensor
    nsum: int
    row_w: torch.Tensor
    row_expert: torch.Tensor
    n_real: int
    ident: torch.Tensor
    extra: Optional[torch.Tensor] = None


class GroupedMoE:
    """Mixture of one-accumulator experts (``W_down relu(W_up h)^2``) chosen by a softmax-score router: logits over the
    real experts and ``identity`` identity experts behind them (an identity expert returns its input), scores = softmax,
    the choice made on score + ``correction`` within the ``keep`` best of ``groups`` equal groups, the ``top`` largest
    chosen, each weighted on its OUTPUT by its score (not renormalised). An optional shared expert of the same form runs
    for every token. The router is an fp32 matrix in both number formats."""

    def __init__(self, experts: int, identity: int, top: int, groups: int, keep: int, w_router: torch.Tensor,
                 correction: Optional[torch.Tensor], w_up: Optional[torch.Tensor], w_down: Optional[torch.Tensor],
                 shared_up: Optional[torch.Tensor] = None, shared_down: Optional[torch.Tensor] = None,
                 act: int = hy.ACT_RELU2):
        self.experts, self.identity, self.top, self.groups, self.keep = experts, identity, top, groups, keep
        self.w_router = w_router      # fp32 [E + I, D]
        self.correction = correction  # fp32 [E + I] or None
        self.w_up, self.w_down = w_up, w_down  # [E, ff, D], [E, D, ff]
        self.shared_up, self.shared_down, self.act = shared_up, shared_down, act

    def __call__(self, h, ctx: StepContext) -> MixtureOut:
        hv = _value(h)  # (three products and the identity experts read the normed input: written out once)
        z = hy.linear(hv, self.w_router)
        y, row_expert, row_w = hy.moe_grouped(hv, z, self.correction, self.top, self.groups, self.keep, self.w_up,
                                              self.w_down, self.act)
        extra = None
        if self.shared_up is not None:
            extra = hy.ff_dense(hv, self.shared_up, self.shared_down, self.act)
        return MixtureOut(y, self.top, row_w, row_expert, self.experts, hv, extra)


class HyperBlock:
    """Pre-norm sublayers over ``S`` residual streams ``xs [S, M, D]`` (hyper-connections). Sublayer ``q`` reads
    ``u = sum_s in_q[s] xs[s]``, computes ``y = sublayer(norm_q * rms(u))``, and replaces all streams at once:
    ``xs[t] <- sum_s mix_q[s, t] xs[s] + out_q[t] * y``. ``S = 1`` with unit weights is the plain pre-norm residual.
    The write of a sublayer also produces the next sublayer's ``u`` (``ctx.u``; the model's last block is given ones as
    its successor's read weights, so it leaves the sum of the streams there)."""

    def __init__(self, mixer, norm1: torch.Tensor, hc1, mlp, norm2: Optional[torch.Tensor], hc2, eps: float):
        self.mixer, self.norm1, self.hc1 = mixer, norm1, hc1  # hc: (in [S], mix [S, S], out [S]) fp32
        self.mlp, self.norm2, self.hc2, self.eps = mlp, norm2, hc2, eps
        self.next_in: Optional[torch.Tensor] = None  # read weights of whatever follows this block

    def __call__(self, xs: torch.Tensor, ctx) -> None:
        u = ctx.u if ctx.u is not None else hy.hc_in(xs, self.hc1[0])
        y = self.mixer(hy.RmsInput(u, self.norm1, self.eps), ctx)
        after = self.hc2[0] if self.mlp is not None else self.next_in
        u = hy.hc_update_(xs, self.hc1[1], self.hc1[2], y, next_in=after)
        if self.mlp is not None:
            f = self.mlp(hy.RmsInput(u, self.norm2, self.eps), ctx)
            u = hy.hc_update_(xs, self.hc2[1], self.hc2[2], f.y, f.nsum, f.row_w, f.row_expert, f.n_real, f.ident, f.extra,
                              next_in=self.next_in)
        ctx.u = u
