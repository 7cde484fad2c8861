"""Besulix: a layer-list decoder that alternates matrix-memory layers with layers whose mixer is a block-local rotary
attention beside a token-shifted linear recurrence.

Per layer (``models/mixers.PreNormBlock``): ``x += mixer(g1 * rms(x))`` and, where the layer has one,
``x += ff(g2 * rms(x))``. Mixers: ``mlstm`` (``MatrixLSTM``) and ``parallel`` (``SideBySide`` of a
``RotaryChunkAttention`` and a ``TimeMix``, summed with the configuration's two weights). Feed-forward: dense with the
clamped gate. The embedding is RMS-normed with a gain on the way in; the logits are soft-capped.

Checkpoint: ``config.json`` + ``model.safetensors`` with tensors ``embed``, ``embed.norm``, ``l<i>.norm1|norm2``,
``l<i>.mix.q|k|v|g|o|norm|i|i.b|f|f.b`` (mlstm), ``l<i>.mix.left.q|q.b|k|k.b|v|v.b|temp|sink|o`` and
``l<i>.mix.right.mu.r|k|v|g|w``, ``l<i>.mix.right.r|k|v|g|w1|w2|w0|u|norm|o`` (parallel), ``l<i>.mlp.gate|up|down``,
``final.norm``, ``head`` (linear weights ``[out, in]``). Loading fuses each mixer's input projections into one matrix
(``q|k|v|g|i|f`` for the matrix memory, ``q|k|v`` with one bias vector for the attention, the four same-shaped time-mix
projections stacked), lays the two output matrices of a parallel layer side by side, and keeps every constant of a
recurrence, the temperatures, sinks and gains in fp32.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config import BesulixConfig
from ..ops import hybrid as hy
from .layer_list import LayerListLM
from .mixers import GatedDenseFF, MatrixLSTM, PreNormBlock, RotaryChunkAttention, SideBySide, TimeMix

BF16 = torch.bfloat16
F32 = torch.float32

# the gate nonlinearity of the feed-forward is g * sigmoid(GATE_ALPHA * g): fixed by the design
GATE_ALPHA = 1.702
MU_NAMES = ("r", "k", "v", "g", "w")


def cache_specs(config: BesulixConfig) -> list:
    out = []
    for ls in config.layers:
        m = ls.mixer
        if m.type == "mlstm":
            out.append(("mlstm", m.heads, m.dim, m.vdim))
        else:
            out.append(("multi", ("kv", m.left.kv_heads, m.left.dim, m.left.vdim),
                        ("timemix", m.right.heads, m.right.dim, m.right.dim, config.hidden_size)))
    return out


def random_state_dict(config: BesulixConfig, seed: int = 0, decay_rank: int = 64) -> Dict[str, torch.Tensor]:
    """A random checkpoint of ``config`` with the checkpoint's tensor names (bf16): synthetic benchmarks and tests.
    Scales keep every sublayer's output O(1), the gates away from saturation and the decays spread over (0, 1)."""
    g = torch.Generator().manual_seed(seed)
    d, v = config.hidden_size, config.vocab_size

    def mat(n, k, std=None):
        return (torch.randn(n, k, generator=g) * (std if std is not None else k ** -0.5)).to(BF16)

    def vec(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).to(BF16)

    sd: Dict[str, torch.Tensor] = {"embed": mat(v, d, 1.0), "embed.norm": vec(d, 0.7, 1.3), "head": mat(v, d),
                                   "final.norm": vec(d, 0.7, 1.3)}
    for i, ls in enumerate(config.layers):
        p, m = f"l{i}.", ls.mixer
        sd[p + "norm1"] = vec(d, 0.7, 1.3)
        if m.type == "mlstm":
            x = p + "mix."
            sd[x + "q"], sd[x + "k"] = mat(m.heads * m.dim, d), mat(m.heads * m.dim, d)
            sd[x + "v"], sd[x + "g"] = mat(m.heads * m.vdim, d), mat(m.heads * m.vdim, d)
            sd[x + "i"], sd[x + "f"] = mat(m.heads, d, 2.0 * d ** -0.5), mat(m.heads, d, 2.0 * d ** -0.5)
            sd[x + "i.b"], sd[x + "f.b"] = vec(m.heads, -1.0, 1.0), vec(m.heads, 1.0, 4.0)
            sd[x + "norm"] = vec(m.heads * m.vdim, 0.7, 1.3)
            sd[x + "o"] = mat(d, m.heads * m.vdim)
        else:
            a, x = m.left, p + "mix.left."
            for n, rows in (("q", a.heads * a.dim), ("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)):
                sd[x + n] = mat(rows, d)
                sd[x + n + ".b"] = vec(rows, -0.3, 0.3)
            sd[x + "temp"] = vec(a.heads, 0.6, 1.6)
            sd[x + "sink"] = torch.randn(a.heads, generator=g).to(BF16)
            sd[x + "o"] = mat(d, a.heads * a.vdim)
            r, x = m.right, p + "mix.right."
            hd = r.heads * r.dim
            for n in MU_NAMES:
                sd[x + "mu." + n] = vec(d, 0.0, 1.0)
            for n in ("r", "k", "v", "g"):
                sd[x + n] = mat(hd, d)
            sd[x + "w1"] = mat(decay_rank, d)
            sd[x + "w2"] = mat(hd, decay_rank, 1.0)
            sd[x + "w0"] = vec(hd, -4.0, 0.5)
            sd[x + "u"] = vec(hd, -0.5, 0.5).reshape(r.heads, r.dim)
            sd[x + "norm"] = vec(hd, 0.7, 1.3)
            sd[x + "o"] = mat(d, hd)
        if ls.mlp is not None:
            sd[p + "norm2"] = vec(d, 0.7, 1.3)
            sd[p + "mlp.gate"], sd[p + "mlp.up"] = mat(ls.mlp.ff, d), mat(ls.mlp.ff, d)
            sd[p + "mlp.down"] = mat(d, ls.mlp.ff)
    return sd


class BesulixForCausalLM(LayerListLM):
    """Besulix on the layer-list step function (``models/layer_list.py``)."""

    config_class = BesulixConfig
    family = "Besulix"
    random_state_dict = staticmethod(random_state_dict)

    def cache_specs(self) -> list:
        return cache_specs(self.config)

    def load_state_dict(self, sd: Dict[str, torch.Tensor]) -> "BesulixForCausalLM":
        c, dev, wdt, eps = self.config, self.device, self.param_dtype, self.eps
        d = c.hidden_size

        def mat(*names):  # one matrix, or several stacked along the rows
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            return t.to(dev, wdt).contiguous()

        def f32(*names):
            return torch.cat([sd[n].reshape(-1) for n in names]).to(dev, F32).contiguous()

        def shaped(name, *shape):
            if tuple(sd[name].shape) != shape:
                raise ValueError(f"{name}: shape {tuple(sd[name].shape)}, expected {shape}")

        self.embed = mat("embed")
        self.embed_norm = f32("embed.norm")
        self.final_norm = f32("final.norm")
        self.head = mat("head")
        self.logit_softcap = c.logit_softcap
        self.blocks = []
        for i, ls in enumerate(c.layers):
            p, m = f"l{i}.", ls.mixer
            if m.type == "mlstm":
                x = p + "mix."
                shaped(x + "q", m.heads * m.dim, d), shaped(x + "v", m.heads * m.vdim, d), shaped(x + "i", m.heads, d)
                mixer = MatrixLSTM(i, m.heads, m.dim, m.vdim, m.gate_cap, eps,
                                   mat(*(x + n for n in ("q", "k", "v", "g", "i", "f"))), f32(x + "i.b", x + "f.b"),
                                   f32(x + "norm"), mat(x + "o"))
            else:
                a, x = m.left, p + "mix.left."
                shaped(x + "q", a.heads * a.dim, d), shaped(x + "k", a.kv_heads * a.dim, d)
                shaped(x + "v", a.kv_heads * a.vdim, d)
                left = RotaryChunkAttention(i, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, mat(x + "q", x + "k", x + "v"),
                                            f32(x + "q.b", x + "k.b", x + "v.b"),
                                            hy.rotary_freqs(a.rot_base, a.rot_dims, dev),
                                            hy.rotary_freqs(a.rot_base, a.vdim, dev), f32(x + "temp"), f32(x + "sink"),
                                            a.chunk, mat(x + "o"))
                r, x = m.right, p + "mix.right."
                hd = r.heads * r.dim
                shaped(x + "r", hd, d), shaped(x + "u", r.heads, r.dim)
                mu = torch.stack([sd[x + "mu." + n].reshape(-1) for n in MU_NAMES]).to(dev, F32).contiguous()
                w_rkvg = torch.stack([sd[x + n] for n in ("r", "k", "v", "g")]).to(dev, wdt).contiguous()
                right = TimeMix(i, r.heads, r.dim, eps, mu, w_rkvg, mat(x + "w1"), mat(x + "w2"),
                                f32(x + "w0").reshape(r.heads, r.dim), f32(x + "u").reshape(r.heads, r.dim),
                                f32(x + "norm"), mat(x + "o"))
                mixer = SideBySide([left, right], [m.left_scale, m.right_scale])
            mlp = norm2 = None
            if ls.mlp is not None:
                mlp = GatedDenseFF(mat(p + "mlp.gate", p + "mlp.up"), mat(p + "mlp.down"), ls.mlp.limit, GATE_ALPHA)
                norm2 = f32(p + "norm2")
            self.blocks.append(PreNormBlock(mixer, f32(p + "norm1"), mlp, norm2, eps))
        return self
