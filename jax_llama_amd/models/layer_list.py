"""Layer-list causal LM on the hybrid op layer: what every architecture of the registry that is assembled from
``models/mixers.py`` blocks shares -- the checkpoint directory round trip, the layered cache, and the step function
``forward_tokens`` that the generation engine (``runtime/engine.py``) and the request stepper (``runtime/stepper.py``)
call. A family subclasses it with its configuration class, ``cache_specs`` and ``load_state_dict`` (which fills
``embed``, ``blocks``, ``final_norm``, ``head`` and, if it has them, ``embed_scale``, ``embed_norm``, ``logit_softcap``).

Number formats: ``dtype=bfloat16`` (serving: bf16 matrix operands and caches, fp32 accumulation, and fp32 residual,
norms, scores, recurrent state) or ``dtype=float32`` (everything exact fp32).
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch

from ..ops import hybrid as hy
from ..parallel.comm import NO_COMM
from .kv_cache import HybridCache
from .mixers import StepContext

BF16 = torch.bfloat16
F32 = torch.float32


class LayerListLM:
    """Causal LM over the hybrid op layer (inference)."""

    config_class: type = None
    family = "layer-list"
    supports_padding = False  # (no block takes a key mask; recurrent layers could not)

    def __init__(self, config, device="cpu", dtype=BF16, seed: int = 0, _do_init: bool = True):
        if dtype not in (BF16, F32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype}")
        self.config = config
        self.device = torch.device(device)
        self.param_dtype = dtype  # matrix operand / cache element type
        self.dtype = F32          # logits
        self.comm = NO_COMM
        self.vocab_local = config.vocab_size
        self.eps = config.norm_eps
        self.blocks: List = []
        self.embed: Optional[torch.Tensor] = None
        self.embed_scale = 1.0
        self.embed_norm: Optional[torch.Tensor] = None  # fp32 [D]: gain of an RMS norm on the embedding
        self.logit_softcap = 0.0                        # logits <- cap * tanh(logits / cap) when > 0
        self.streams = 0  # > 0: the blocks work on that many residual streams [S, M, D] (hyper-connections)
        self.final_norm: Optional[torch.Tensor] = None  # fp32 gain of the last norm: one number or [D]
        self.head: Optional[torch.Tensor] = None
        if _do_init:
            self.load_state_dict(self.random_state_dict(config, seed))

    # ------------------------------------------------------------------ family hooks
    @staticmethod
    def random_state_dict(config, seed: int = 0) -> Dict[str, torch.Tensor]:
        raise NotImplementedError

    def load_state_dict(self, sd: Dict[str, torch.Tensor]):
        raise NotImplementedError

    def cache_specs(self) -> list:
        raise NotImplementedError

    def _weight_tensors(self) -> list:
        """Every tensor the model holds (for ``weight_bytes``)."""
        stack = [self.embed, self.head]

        def walk(obj, depth):
            for val in (vars(obj).values() if hasattr(obj, "__dict__") else obj if isinstance(obj, (list, tuple)) else ()):
                if torch.is_tensor(val):
                    stack.append(val)
                elif val is not None and depth < 3 and (hasattr(val, "__dict__") or isinstance(val, (list, tuple))):
                    walk(val, depth + 1)

        for blk in self.blocks:
            walk(blk, 0)
        return stack

    # ------------------------------------------------------------------ checkpoints
    @classmethod
    def from_pretrained(cls, directory: str, device="cpu", dtype=BF16):
        from safetensors import safe_open
        config = cls.config_class.from_pretrained(directory)
        model = cls(config, device=device, dtype=dtype, _do_init=False)
        sd = {}
        with safe_open(os.path.join(directory, "model.safetensors"), framework="pt", device="cpu") as f:
            for k in f.keys():
                sd[k] = f.get_tensor(k)
        return model.load_state_dict(sd)

    def save_pretrained(self, directory: str, state_dict: Dict[str, torch.Tensor]) -> None:
        """Write ``config.json`` + ``model.safetensors`` (checkpoint names) from a checkpoint-named state dict."""
        from safetensors.torch import save_file
        self.config.save_pretrained(directory)
        save_file({k: v.contiguous() for k, v in state_dict.items()}, os.path.join(directory, "model.safetensors"))

    def weight_bytes(self) -> int:
        seen, n = set(), 0
        for t in self._weight_tensors():
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ cache
    def init_cache(self, batch_size: int, max_length: int) -> HybridCache:
        return HybridCache(self.cache_specs(), batch_size, max_length, self.device, self.param_dtype)

    def cache_nbytes(self, batch_size: int, max_length: int) -> int:
        return HybridCache.bytes_per(self.cache_specs(), batch_size, max_length, self.param_dtype)

    # ------------------------------------------------------------------ forward
    def forward_tokens(self, ids: torch.Tensor, positions: torch.Tensor, cache, slot0, kv_start=None, key_mask=None,
                       logits_mode: str = "last", collect_hidden: bool = False, collect_attn: bool = False,
                       logit_rows: Optional[torch.Tensor] = None):
        """Run all layers for ``ids [B, S]`` placed at cache slots ``slot0 .. slot0 + S - 1`` (``slot0``: int or a
        device int32[1]); keys / values and recurrent state of ``cache`` advance. Returns ``(logits, x, hidden, [])``:
        fp32 logits ``[B, V]`` ("last" / "argmax": the sampler reduces them), ``[B*S, V]`` ("all"), the rows
        ``logit_rows`` of the flattened ``[B*S]`` tokens ("rows"), or None ("none"). ``hidden`` (``collect_hidden``):
        the residual stream after every layer. Recurrent layers carry no padding mask: every row's tokens must be
        real (``kv_start`` all zero, no ``key_mask``)."""
        if key_mask is not None or collect_attn:
            raise NotImplementedError(f"{self.family}: key masks / attention maps are not supported")
        b, s = ids.shape
        d = self.config.hidden_size
        idf = ids.reshape(-1).to(self.device, torch.int32).contiguous()
        ctx = StepContext(idf, positions.reshape(-1).to(self.device, torch.int32).contiguous(), b, s, cache, slot0)
        hidden = []
        if self.streams:
            # every stream starts as the embedding; a block leaves the next one's input sum in ctx.u, the last block the
            # sum of the streams: the residual that the final norm reads
            xs = hy.embed_rows(idf, self.embed, scale=self.embed_scale, copies=self.streams).reshape(self.streams, b * s, d)
            ones = self._stream_ones()
            for blk in self.blocks:
                blk(xs, ctx)
                if collect_hidden:
                    hidden.append(hy.hc_in(xs, ones).reshape(b, s, d))
            x = ctx.u if ctx.u is not None else hy.hc_in(xs, ones)
        else:
            x = hy.embed_rows(idf, self.embed, scale=self.embed_scale)
            if self.embed_norm is not None:
                x = hy.rms_rows(x, self.embed_norm, self.eps)
            for blk in self.blocks:
                blk(x, ctx)
                if collect_hidden:
                    hidden.append(x.reshape(b, s, d).clone())
        if logits_mode == "none":
            return None, x, hidden, []
        if logits_mode in ("last", "argmax"):
            xl = x.reshape(b, s, d)[:, -1].contiguous()
        elif logits_mode == "rows":
            xl = x.index_select(0, logit_rows.to(self.device, torch.long))
        elif logits_mode == "all":
            xl = x
        else:
            raise ValueError(f"unknown logits_mode {logits_mode!r}")
        cap = float(self.logit_softcap or 0.0)
        logits = hy.linear(hy.rms_rows(xl, self.final_norm, self.eps), self.head,
                           act=hy.ACT_SOFTCAP if cap > 0 else hy.ACT_NONE, limit=cap)
        return logits, x, hidden, []

    def _stream_ones(self) -> torch.Tensor:
        ones = getattr(self, "_ones", None)
        if ones is None or ones.numel() != self.streams:
            ones = self._ones = torch.ones(self.streams, dtype=F32, device=self.device)
        return ones

    def gather_logits(self, logits_local: torch.Tensor) -> torch.Tensor:
        return logits_local

    def __call__(self, input_ids, position_ids=None, past_key_values: Optional[HybridCache] = None,
                 output_hidden_states: bool = False):
        """Logits for every position ``[B, S, V]`` (fp32); ``past_key_values`` (an ``init_cache`` object) is advanced in
        place when given. Returns ``CausalLMOutput``."""
        from .llama import CausalLMOutput
        ids = torch.as_tensor(input_ids).to(self.device, torch.int32)
        b, s = ids.shape
        cache = past_key_values if past_key_values is not None else self.init_cache(b, s)
        slot0 = cache.index
        if slot0 + s > cache.max_length:
            raise ValueError(f"cache overflow: {slot0}+{s} > {cache.max_length}")
        if position_ids is None:
            position_ids = torch.arange(slot0, slot0 + s, dtype=torch.int32).expand(b, s)
        pos = torch.as_tensor(position_ids).to(self.device, torch.int32).reshape(b, s).contiguous()
        logits, _, hidden, _ = self.forward_tokens(ids, pos, cache, slot0, logits_mode="all",
                                                   collect_hidden=output_hidden_states)
        if past_key_values is not None:
            cache.advance(s)
        return CausalLMOutput(logits=logits.reshape(b, s, -1), past_key_values=past_key_values,
                              hidden_states=tuple(hidden) if output_hidden_states else None)

    def generate(self, input_ids, attention_mask=None, generation_config=None, prng_key=None, **kwargs):
        """Greedy / sampled generation on the framework's decode engine (``runtime/engine.py``)."""
        from ..runtime.engine import generate as _generate
        if attention_mask is not None and not bool(torch.as_tensor(attention_mask).bool().all()):
            raise NotImplementedError(f"{self.family}: padded batches are not supported (no block takes a key mask)")
        return _generate(self, input_ids, None, generation_config, prng_key=prng_key, **kwargs)
