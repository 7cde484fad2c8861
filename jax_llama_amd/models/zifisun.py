"""Zifisun: a layer-list decoder of windowed latent-attention and normed-attention layers over several residual streams.

Per layer (``models/mixers.HyperBlock``): a sublayer reads a weighted sum of the ``streams`` residual streams through an
RMS norm and writes its result into a mixed copy of all of them (hyper-connections; without ``streams`` a plain pre-norm
residual). Mixers: ``latent_attention`` (``RotaryLatentAttention``: keys and values from one cached latent per token plus
one rotated key part shared by the heads, queries through a latent of their own, a sliding window, an output gate per
head) and ``attention`` (``NormedGatedAttention``: grouped-query attention without positions, weighted q / k norms, a
window that keeps the sequence's first keys, an output gate per head). Feed-forward: none, or a mixture chosen by a
softmax-score router with a selection bias, expert groups and identity experts, plus a shared expert
(``GroupedMoE``). ``loop``: a run of layers is repeated with the same weights; every pass has its own cache, so the
model's blocks (and cache layers) are the layer RUNS, and the blocks of one layer share its weight tensors.

Checkpoint: ``config.json`` + ``model.safetensors`` with tensors ``embed``, ``l<i>.norm1|norm2``,
``l<i>.hc1|hc2.in|mix|out``, ``l<i>.mix.dq|dq.norm|uq|dkv|dkv.norm|uk|uv|g|o`` (latent attention) or
``l<i>.mix.q|k|v|q.norm|k.norm|g|o`` (attention), ``l<i>.mlp.router|correction``, ``l<i>.mlp.e<j>.up|down``,
``l<i>.mlp.shared.up|down``, ``final.norm``, ``head`` (linear weights ``[out, in]``). Loading fuses a mixer's input
projections (and its gate rows) into one matrix, stacks the experts, and keeps routers, corrections, norms and the
hyper-connection weights fp32 in both number formats.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..config import NormedAttentionSpec, RotaryLatentSpec, ZifisunConfig
from ..ops import hybrid as hy
from .layer_list import LayerListLM
from .mixers import GroupedMoE, HyperBlock, NormedGatedAttention, RotaryLatentAttention

BF16 = torch.bfloat16
F32 = torch.float32


def cache_specs(config: ZifisunConfig) -> list:
    """One entry per layer run."""
    specs = []
    for i in config.layer_runs():
        m = config.layers[i].mixer
        if isinstance(m, RotaryLatentSpec):
            specs.append(("latent", m.kv_rank + m.rot_dim))
        else:
            specs.append(("kv", m.kv_heads, m.dim, m.vdim))
    return specs


def random_state_dict(config: ZifisunConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """A random checkpoint of ``config`` with the checkpoint's tensor names (bf16): synthetic benchmarks and tests.
    Scales keep every sublayer's output O(1), the streams from growing, and the router's scores apart."""
    g = torch.Generator().manual_seed(seed)
    d, v = config.hidden_size, config.vocab_size
    ns = max(config.streams, 1)

    def mat(n, k, std=None):
        return (torch.randn(n, k, generator=g) * (std if std is not None else k ** -0.5)).to(BF16)

    def vec(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).to(BF16)

    sd: Dict[str, torch.Tensor] = {"embed": mat(v, d, 1.0), "final.norm": vec(d, 0.7, 1.3), "head": mat(v, d)}
    for i, ls in enumerate(config.layers):
        p, m = f"l{i}.", ls.mixer
        sd[p + "norm1"] = vec(d, 0.7, 1.3)
        if isinstance(m, RotaryLatentSpec):
            sd[p + "mix.dq"] = mat(m.q_rank, d)
            sd[p + "mix.dq.norm"] = vec(m.q_rank, 0.7, 1.3)
            sd[p + "mix.uq"] = mat(m.heads * (m.dim + m.rot_dim), m.q_rank)
            sd[p + "mix.dkv"] = mat(m.kv_rank + m.rot_dim, d)
            sd[p + "mix.dkv.norm"] = vec(m.kv_rank, 0.7, 1.3)
            sd[p + "mix.uk"] = mat(m.heads * m.dim, m.kv_rank)
            sd[p + "mix.uv"] = mat(m.heads * m.vdim, m.kv_rank)
        else:
            sd[p + "mix.q"] = mat(m.heads * m.dim, d)
            sd[p + "mix.k"] = mat(m.kv_heads * m.dim, d)
            sd[p + "mix.v"] = mat(m.kv_heads * m.vdim, d)
            sd[p + "mix.q.norm"] = vec(m.dim, 0.7, 1.3)
            sd[p + "mix.k.norm"] = vec(m.dim, 0.7, 1.3)
        sd[p + "mix.g"] = mat(m.heads, d)
        sd[p + "mix.o"] = mat(d, m.heads * m.vdim)
        f = ls.mlp
        if f is not None:
            sd[p + "norm2"] = vec(d, 0.7, 1.3)
            sd[p + "mlp.router"] = mat(f.experts + f.identity, d, 2.0 * d ** -0.5)
            sd[p + "mlp.correction"] = vec(f.experts + f.identity, -0.05, 0.05)
            for e in range(f.experts):
                sd[p + f"mlp.e{e}.up"] = mat(f.ff, d)
                sd[p + f"mlp.e{e}.down"] = mat(d, f.ff)
            if f.shared_ff:
                sd[p + "mlp.shared.up"] = mat(f.shared_ff, d)
                sd[p + "mlp.shared.down"] = mat(d, f.shared_ff)
        if config.streams:
            for q in ("hc1.", "hc2.") if f is not None else ("hc1.",):
                sd[p + q + "in"] = vec(ns, 0.2, 0.6)
                sd[p + q + "out"] = vec(ns, 0.3, 1.0)
                sd[p + q + "mix"] = (0.8 * torch.eye(ns) + 0.2 * torch.rand(ns, ns, generator=g) / ns).to(BF16)
    return sd


class ZifisunForCausalLM(LayerListLM):
    """Zifisun on the layer-list step function (``models/layer_list.py``)."""

    config_class = ZifisunConfig
    family = "Zifisun"
    random_state_dict = staticmethod(random_state_dict)

    def cache_specs(self) -> list:
        return cache_specs(self.config)

    def load_state_dict(self, sd: Dict[str, torch.Tensor]) -> "ZifisunForCausalLM":
        c, dev, wdt, eps = self.config, self.device, self.param_dtype, self.eps
        ns = max(c.streams, 1)

        def mat(*names):  # one matrix, or several stacked along the rows
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            return t.to(dev, wdt).contiguous()

        def f32(name, shape=None):
            t = sd[name].to(dev, F32).contiguous()
            return t.reshape(shape) if shape is not None else t.reshape(-1)

        def want(name, shape):
            if tuple(sd[name].shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(sd[name].shape)}, the configuration says {tuple(shape)}")

        def hyper(pre):  # (read weights, mixing matrix [from, to], write weights); absent: the plain residual
            if pre + "in" in sd:
                want(pre + "mix", (ns, ns))
                return f32(pre + "in"), f32(pre + "mix", (ns, ns)), f32(pre + "out")
            if ns != 1:
                raise ValueError(f"{pre}*: {ns} streams need hyper-connection weights")
            one = torch.ones(1, dtype=F32, device=dev)
            return one, one.reshape(1, 1), one

        self.embed = mat("embed")
        self.head = mat("head")
        self.final_norm = f32("final.norm")
        self.streams = ns
        layers = []
        for i, ls in enumerate(c.layers):
            p, m = f"l{i}.", ls.mixer
            if isinstance(m, RotaryLatentSpec):
                want(p + "mix.dq", (m.q_rank, c.hidden_size))
                want(p + "mix.dkv", (m.kv_rank + m.rot_dim, c.hidden_size))
                want(p + "mix.uq", (m.heads * (m.dim + m.rot_dim), m.q_rank))
                want(p + "mix.uk", (m.heads * m.dim, m.kv_rank))
                want(p + "mix.uv", (m.heads * m.vdim, m.kv_rank))
                w_uk = sd[p + "mix.uk"].reshape(m.heads, m.dim, m.kv_rank).to(dev, wdt)
                w_uv = sd[p + "mix.uv"].reshape(m.heads, m.vdim, m.kv_rank).to(dev, wdt).contiguous()
                freq = hy.rotary_freqs(m.rot_base, m.rot_dims, dev) if m.rot_dims else None
                gated = p + "mix.g" in sd
                names = [p + "mix.dq", p + "mix.dkv"] + ([p + "mix.g"] if gated else [])
                args = (m, eps, mat(*names), f32(p + "mix.dq.norm"), mat(p + "mix.uq"), f32(p + "mix.dkv.norm"), w_uk, w_uv,
                        freq, mat(p + "mix.o"), gated)
                make = RotaryLatentAttention
            elif isinstance(m, NormedAttentionSpec):
                want(p + "mix.q", (m.heads * m.dim, c.hidden_size))
                want(p + "mix.k", (m.kv_heads * m.dim, c.hidden_size))
                want(p + "mix.v", (m.kv_heads * m.vdim, c.hidden_size))
                gated = p + "mix.g" in sd
                names = [p + "mix.q", p + "mix.k", p + "mix.v"] + ([p + "mix.g"] if gated else [])
                args = (m, eps, mat(*names), f32(p + "mix.q.norm") if p + "mix.q.norm" in sd else None,
                        f32(p + "mix.k.norm") if p + "mix.k.norm" in sd else None, gated, mat(p + "mix.o"))
                make = NormedGatedAttention
            else:
                raise ValueError(f"layer {i}: unknown mixer {m!r}")
            f = ls.mlp
            mlp = norm2 = hc2 = None
            if f is not None:
                total = f.experts + f.identity
                want(p + "mlp.router", (total, c.hidden_size))
                w_up = torch.stack([sd[p + f"mlp.e{e}.up"] for e in range(f.experts)]).to(dev, wdt).contiguous()
                w_down = torch.stack([sd[p + f"mlp.e{e}.down"] for e in range(f.experts)]).to(dev, wdt).contiguous()
                shared = p + "mlp.shared.up" in sd
                mlp = GroupedMoE(f.experts, f.identity, f.top, f.groups, f.keep_groups,
                                 sd[p + "mlp.router"].to(dev, F32).contiguous(),
                                 f32(p + "mlp.correction") if p + "mlp.correction" in sd else None, w_up, w_down,
                                 mat(p + "mlp.shared.up") if shared else None,
                                 mat(p + "mlp.shared.down") if shared else None)
                norm2, hc2 = f32(p + "norm2"), hyper(p + "hc2.")
            layers.append((make, args, f32(p + "norm1"), hyper(p + "hc1."), mlp, norm2, hc2))
        # one block per layer run: its own cache layer, the layer's tensors
        self.blocks = []
        for run, i in enumerate(c.layer_runs()):
            make, args, norm1, hc1, mlp, norm2, hc2 = layers[i]
            self.blocks.append(HyperBlock(make(run, *args), norm1, hc1, mlp, norm2, hc2, eps))
        ones = torch.ones(ns, dtype=F32, device=dev)
        for blk, nxt in zip(self.blocks, self.blocks[1:] + [None]):
            blk.next_in = nxt.hc1[0] if nxt is not None else ones
        return self
