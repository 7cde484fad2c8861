"""Model configuration.

Parity with the reference:
  * ``LLaMAConfig`` mirrors ``jax_llama/config.py:70-116`` (same field names and
    defaults: the 7B shape, ``num_key_value_heads`` defaulting to
    ``num_attention_heads``, dropouts 0, ``rope_theta`` 1e4).
  * ``ModelArgs`` / ``config_from_params`` mirror ``jax_llama/convert_weights.py:13-50``
    (Meta ``params.json`` -> config, including the SwiGLU hidden-size formula).

Unlike the reference we do not subclass ``transformers.PretrainedConfig`` (importing
transformers costs seconds and drags in an unrelated framework); the class offers the
subset of that API the reference relies on (``to_dict``/``from_dict``/
``save_pretrained``/``from_pretrained``, ``return_dict``/``output_*`` flags).
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Optional


class LLaMAConfig:
    """Architecture hyper-parameters of a LLaMA-1/2/3 decoder (reference ``config.py:70``)."""

    model_type = "llama"

    def __init__(
        self,
        vocab_size: int = 32000,
        hidden_size: int = 4096,
        intermediate_size: int = 11008,
        num_hidden_layers: int = 32,
        num_attention_heads: int = 32,
        num_key_value_heads: Optional[int] = None,
        max_sequence_length: int = 2048,
        rms_norm_eps: float = 1e-6,
        initializer_range: float = 0.02,
        use_cache: bool = True,
        pad_token_id: int = -1,
        bos_token_id: int = 1,
        eos_token_id: int = 2,
        resid_pdrop: float = 0.0,
        embd_pdrop: float = 0.0,
        attn_pdrop: float = 0.0,
        tie_word_embeddings: bool = False,
        gradient_checkpointing: bool = False,
        rope_theta: float = 10000.0,
        output_attentions: bool = False,
        output_hidden_states: bool = False,
        return_dict: bool = True,
        **kwargs: Any,
    ):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.initializer_range = initializer_range
        self.intermediate_size = intermediate_size
        self.num_hidden_layers = num_hidden_layers
        self.num_attention_heads = num_attention_heads
        if num_key_value_heads is None:
            num_key_value_heads = num_attention_heads
        self.num_key_value_heads = num_key_value_heads
        self.max_sequence_length = max_sequence_length
        self.rms_norm_eps = rms_norm_eps
        self.use_cache = use_cache
        self.pad_token_id = pad_token_id
        self.bos_token_id = bos_token_id
        self.eos_token_id = eos_token_id
        self.resid_pdrop = resid_pdrop
        self.embd_pdrop = embd_pdrop
        self.attn_pdrop = attn_pdrop
        self.tie_word_embeddings = tie_word_embeddings
        self.gradient_checkpointing = gradient_checkpointing
        self.rope_theta = rope_theta
        self.output_attentions = output_attentions
        self.output_hidden_states = output_hidden_states
        self.return_dict = return_dict
        # Unknown keys are kept (HF PretrainedConfig behaviour) so configs round-trip.
        for k, v in kwargs.items():
            setattr(self, k, v)
        if self.hidden_size % self.num_attention_heads:
            raise ValueError("hidden_size must be divisible by num_attention_heads")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ValueError("num_attention_heads must be divisible by num_key_value_heads")

    # ---- derived -------------------------------------------------------------------
    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def num_key_value_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def num_parameters(self) -> int:
        d, f, v, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_hidden_layers
        kv = self.num_key_value_heads * self.head_dim
        per_layer = d * d * 2 + d * kv * 2 + 3 * d * f + 2 * d
        head = 0 if self.tie_word_embeddings else v * d
        return v * d + L * per_layer + d + head

    # ---- (de)serialisation ---------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        out = dict(self.__dict__)
        out["model_type"] = self.model_type
        return out

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LLaMAConfig":
        d = dict(d)
        d.pop("model_type", None)
        return cls(**d)

    def to_json_string(self) -> str:
        return json.dumps(self.to_dict(), indent=2, sort_keys=True)

    def save_pretrained(self, save_directory: str) -> None:
        os.makedirs(save_directory, exist_ok=True)
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            f.write(self.to_json_string())

    @classmethod
    def from_pretrained(cls, path: str) -> "LLaMAConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def __eq__(self, other: object) -> bool:
        return isinstance(other, LLaMAConfig) and self.to_dict() == other.to_dict()

    def __repr__(self) -> str:
        return f"LLaMAConfig {self.to_json_string()}"


# -------------------------------------------------------------------------------------
# Meta params.json handling (reference convert_weights.py:13-50)
# -------------------------------------------------------------------------------------
@dataclass
class ModelArgs:
    """Meta ``params.json`` schema. Constructing with unknown keys raises ``TypeError``
    exactly like the reference (``convert_weights.py:91``); ``from_params_json`` offers a
    tolerant path that also understands Llama-3.1 ``use_scaled_rope``."""

    dim: int = 512
    n_layers: int = 8
    n_heads: int = 8
    n_kv_heads: Optional[int] = None
    vocab_size: int = -1
    multiple_of: int = 256
    ffn_dim_multiplier: Optional[float] = None
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_batch_size: int = 32
    max_seq_len: int = 2048

    @classmethod
    def from_params_json(cls, params: Dict[str, Any], strict: bool = True) -> "ModelArgs":
        if strict:
            return cls(**params)
        names = {f.name for f in dataclasses.fields(cls)}
        return cls(**{k: v for k, v in params.items() if k in names})


def swiglu_hidden_size(dim: int, multiple_of: int, ffn_dim_multiplier: Optional[float] = None) -> int:
    """FFN width rule of Meta's FeedForward (reference ``convert_weights.py:36-39``)."""
    hidden = int(2 * (dim * 4) / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return multiple_of * ((hidden + multiple_of - 1) // multiple_of)


def config_from_params(args: ModelArgs) -> LLaMAConfig:
    return LLaMAConfig(
        vocab_size=args.vocab_size,
        hidden_size=args.dim,
        intermediate_size=swiglu_hidden_size(args.dim, args.multiple_of, args.ffn_dim_multiplier),
        num_hidden_layers=args.n_layers,
        num_attention_heads=args.n_heads,
        num_key_value_heads=args.n_kv_heads,
        max_sequence_length=args.max_seq_len,
        rms_norm_eps=args.norm_eps,
        rope_theta=args.rope_theta,
    )


# -------------------------------------------------------------------------------------
# Named presets (Meta params.json values; MODEL_CARD.md:82-91 for LLaMA-1 shapes).
# Used by the synthetic/random-init paths (bench.py, examples --synthetic).
# -------------------------------------------------------------------------------------
_META_PARAMS: Dict[str, Dict[str, Any]] = {
    "llama1-7b": dict(dim=4096, n_layers=32, n_heads=32, multiple_of=256, norm_eps=1e-6, vocab_size=32000),
    "llama1-13b": dict(dim=5120, n_layers=40, n_heads=40, multiple_of=256, norm_eps=1e-6, vocab_size=32000),
    "llama1-33b": dict(dim=6656, n_layers=60, n_heads=52, multiple_of=256, norm_eps=1e-6, vocab_size=32000),
    "llama1-65b": dict(dim=8192, n_layers=80, n_heads=64, multiple_of=256, norm_eps=1e-5, vocab_size=32000),
    "llama2-7b": dict(dim=4096, n_layers=32, n_heads=32, multiple_of=256, norm_eps=1e-5, vocab_size=32000),
    "llama2-13b": dict(dim=5120, n_layers=40, n_heads=40, multiple_of=256, norm_eps=1e-5, vocab_size=32000),
    "llama2-70b": dict(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, multiple_of=4096,
                       ffn_dim_multiplier=1.3, norm_eps=1e-5, vocab_size=32000),
    "llama3-8b": dict(dim=4096, n_layers=32, n_heads=32, n_kv_heads=8, multiple_of=1024,
                      ffn_dim_multiplier=1.3, norm_eps=1e-5, rope_theta=500000.0, vocab_size=128256),
    "llama3-70b": dict(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, multiple_of=4096,
                       ffn_dim_multiplier=1.3, norm_eps=1e-5, rope_theta=500000.0, vocab_size=128256),
    # The tiny fixture of jax_test.py:28-41 (dim 32, 4 layers, 4 heads, 2 kv heads, vocab 256).
    "tiny": dict(dim=32, n_layers=4, n_heads=4, n_kv_heads=2, multiple_of=2, norm_eps=1e-5,
                 vocab_size=256, max_seq_len=64),
}
_ALIASES = {"7b": "llama2-7b", "8b": "llama3-8b", "13b": "llama2-13b", "33b": "llama1-33b",
            "65b": "llama1-65b", "70b": "llama3-70b"}


def preset_names():
    return sorted(_META_PARAMS)


def get_preset(name: str, max_seq_len: Optional[int] = None, **overrides: Any) -> LLaMAConfig:
    name = _ALIASES.get(name.lower(), name.lower())
    if name not in _META_PARAMS:
        raise KeyError(f"unknown model preset {name!r}; known: {preset_names()}")
    p = dict(_META_PARAMS[name])
    if max_seq_len is not None:
        p["max_seq_len"] = max_seq_len
    cfg = config_from_params(ModelArgs(**p))
    for k, v in overrides.items():
        setattr(cfg, k, v)
    return cfg


# -------------------------------------------------------------------------------------
# Zavevik: a layer-list configuration (every layer names its mixer and its feed-forward)
# -------------------------------------------------------------------------------------
@dataclass
class MixerSpec:
    """One layer's sequence mixer. ``type`` ``"attention"``: softmax attention with RMS-normed q / k / v, an optional
    query temperature (``q_temp_coef`` / ``q_temp_every``), score ``scale``, optional ``softcap`` and an optional
    bucketed distance bias reaching ``bias_max``; ``kv_from``: the layer whose keys and values it reads instead of
    projecting its own. ``type`` ``"delta"``: the gated delta rule with ``conv``-tap short convolutions. ``type``
    ``"latent_attention"``: softmax attention whose keys and values are per-head linear maps of one cached vector of
    ``kv_rank`` numbers per token, without positions, with a learned per-head sink in the softmax denominator."""

    type: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int = 0
    scale: float = 1.0
    softcap: float = 0.0
    bias_max: int = 0
    q_temp_coef: float = 0.0
    q_temp_every: int = 1
    kv_from: Optional[int] = None
    kv_rank: int = 0

    @classmethod
    def from_dict(cls, type_: str, d: Dict[str, Any]) -> "MixerSpec":
        d = dict(d)
        qt = d.pop("q_temp", None) or {}
        heads, dim = int(d.pop("heads")), int(d.pop("dim"))
        known = dict(type=type_, heads=heads, kv_heads=int(d.pop("kv_heads", heads)), dim=dim,
                     vdim=int(d.pop("vdim", dim)), conv=int(d.pop("conv", 1 if type_ == "delta" else 0)),
                     scale=float(d.pop("scale", 1.0)),
                     softcap=float(d.pop("softcap", 0.0) or 0.0), bias_max=int(d.pop("bias_max", 0) or 0),
                     q_temp_coef=float(qt.get("coef", 0.0)), q_temp_every=int(qt.get("every", 1)),
                     kv_from=d.pop("kv_from", None), kv_rank=int(d.pop("kv_rank", 0) or 0))
        # (keys this family does not define are ignored, like HF configs keep unknown entries)
        if known["kv_from"] is not None:
            known["kv_from"] = int(known["kv_from"])
        if type_ not in ("attention", "delta", "latent_attention"):
            raise ValueError(f"unknown mixer type {type_!r}")
        if (type_ == "latent_attention") != (known["kv_rank"] > 0):
            raise ValueError("kv_rank belongs to latent_attention, which needs it")
        if known["heads"] % known["kv_heads"]:
            raise ValueError("heads must be divisible by kv_heads")
        return cls(**known)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim)
        if self.type == "delta":
            out["conv"] = self.conv
            return out
        if self.type == "latent_attention":
            return dict(heads=self.heads, dim=self.dim, vdim=self.vdim, kv_rank=self.kv_rank, scale=self.scale)
        out["scale"] = self.scale
        if self.softcap:
            out["softcap"] = self.softcap
        if self.bias_max:
            out["bias_max"] = self.bias_max
        if self.q_temp_coef:
            out["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass
class MoESpec:
    """Table-routed mixture of SwiGLU experts: ``experts`` experts of width ``ff``, ``top`` of them per token."""

    experts: int
    top: int
    ff: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MoESpec":
        if d.get("kind", "moe") != "moe":
            raise ValueError(f"unknown feed-forward kind {d.get('kind')!r}")
        return cls(experts=int(d["router"]["experts"]), top=int(d["router"]["top"]), ff=int(d["expert"]["ff"]))

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass
class DenseFFSpec:
    """Dense feed-forward of width ``ff``: ``W_down act(W_up h)``."""

    ff: int
    kind = "dense"

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass
class RoutedMoESpec:
    """Score-routed mixture: ``experts`` clamped-gate experts of width ``ff`` (clamp ``limit``), ``top`` of them per
    token by sigmoid score; an optional shared expert of width ``shared_ff`` (clamp ``shared_limit``) for every token."""

    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: int = 0
    shared_limit: float = 0.0
    kind = "moe"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "RoutedMoESpec":
        sh = d.get("shared") or {}
        out = cls(experts=int(d["router"]["experts"]), top=int(d["router"]["top"]), ff=int(d["expert"]["ff"]),
                  limit=float(d["expert"]["limit"]), shared_ff=int(sh.get("ff", 0)),
                  shared_limit=float(sh.get("limit", 0.0)))
        if not 1 <= out.top <= out.experts:
            raise ValueError(f"router: top {out.top} of {out.experts} experts")
        return out

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


@dataclass
class LayerSpec:
    mixer: MixerSpec
    mlp: Optional[Any]  # MoESpec (Zavevik), DenseFFSpec / RoutedMoESpec (Zasevik), or None


class ZavevikConfig:
    """Zavevik decoder: ``config.json`` with ``architecture: "Zavevik"``, ``vocab``, ``width``, ``norm.eps``,
    ``token_side.dim`` (optional) and a ``layers`` list of ``{type, mixer, mlp}`` entries."""

    model_type = "zavevik"
    architecture = "Zavevik"

    def __init__(self, vocab_size: int, hidden_size: int, layers, norm_eps: float = 1e-6, side_dim: int = 0,
                 pad_token_id: int = -1, eos_token_id: Optional[int] = None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.layers = list(layers)
        self.norm_eps = float(norm_eps)
        self.side_dim = int(side_dim)
        self.pad_token_id = pad_token_id
        self.eos_token_id = eos_token_id
        for i, ls in enumerate(self.layers):
            j = ls.mixer.kv_from
            if j is not None:
                src = self.layers[j].mixer if 0 <= j < i else None
                if src is None or src.type != "attention" or src.kv_from is not None:
                    raise ValueError(f"layer {i}: kv_from {j} is not an earlier attention layer with its own keys")
                if (src.kv_heads, src.dim, src.vdim) != (ls.mixer.kv_heads, ls.mixer.dim, ls.mixer.vdim):
                    raise ValueError(f"layer {i}: key / value geometry differs from layer {j}'s")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZavevikConfig":
        layers = [LayerSpec(MixerSpec.from_dict(e["type"], e["mixer"]),
                            MoESpec.from_dict(e["mlp"]) if e.get("mlp") is not None else None) for e in d["layers"]]
        side = d.get("token_side") or {}
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], layers=layers, norm_eps=d["norm"]["eps"],
                   side_dim=side.get("dim", 0), pad_token_id=d.get("pad_token_id", -1),
                   eos_token_id=d.get("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                               "norm": {"eps": self.norm_eps},
                               "layers": [{"type": ls.mixer.type, "mixer": ls.mixer.to_dict(),
                                           "mlp": ls.mlp.to_dict() if ls.mlp is not None else None}
                                          for ls in self.layers]}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out

    def save_pretrained(self, save_directory: str) -> None:
        os.makedirs(save_directory, exist_ok=True)
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=1, sort_keys=True)

    @classmethod
    def from_pretrained(cls, path: str) -> "ZavevikConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def __eq__(self, other: object) -> bool:
        return isinstance(other, ZavevikConfig) and self.to_dict() == other.to_dict()

    def __repr__(self) -> str:
        return f"ZavevikConfig {json.dumps(self.to_dict(), sort_keys=True)}"


class ZasevikConfig:
    """Zasevik decoder: ``config.json`` with ``architecture: "Zasevik"``, ``vocab``, ``width``, ``norm.eps``,
    ``embedding.scale`` and a ``layers`` list of ``{type, mixer, mlp}`` entries; ``mlp`` is null, ``{kind: dense, ff}``
    or ``{kind: moe, expert: {ff, limit}, router: {experts, top}, shared: {ff, limit}}``."""

    model_type = "zasevik"
    architecture = "Zasevik"

    def __init__(self, vocab_size: int, hidden_size: int, layers, norm_eps: float = 1e-6, embed_scale: float = 1.0,
                 pad_token_id: int = -1, eos_token_id: Optional[int] = None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.layers = list(layers)
        self.norm_eps = float(norm_eps)
        self.embed_scale = float(embed_scale)
        self.pad_token_id = pad_token_id
        self.eos_token_id = eos_token_id
        for i, ls in enumerate(self.layers):
            if ls.mixer.type != "latent_attention":
                raise ValueError(f"layer {i}: Zasevik has no mixer {ls.mixer.type!r}")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def _ff_from_dict(d: Optional[Dict[str, Any]]):
        if d is None:
            return None
        kind = d.get("kind")
        if kind == "dense":
            return DenseFFSpec(ff=int(d["ff"]))
        if kind == "moe":
            return RoutedMoESpec.from_dict(d)
        raise ValueError(f"unknown feed-forward kind {kind!r}")

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZasevikConfig":
        layers = [LayerSpec(MixerSpec.from_dict(e["type"], e["mixer"]), cls._ff_from_dict(e.get("mlp")))
                  for e in d["layers"]]
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], layers=layers, norm_eps=d["norm"]["eps"],
                   embed_scale=(d.get("embedding") or {}).get("scale", 1.0), pad_token_id=d.get("pad_token_id", -1),
                   eos_token_id=d.get("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embed_scale},
                "layers": [{"type": ls.mixer.type, "mixer": ls.mixer.to_dict(),
                            "mlp": ls.mlp.to_dict() if ls.mlp is not None else None} for ls in self.layers]}

    def save_pretrained(self, save_directory: str) -> None:
        os.makedirs(save_directory, exist_ok=True)
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=1, sort_keys=True)

    @classmethod
    def from_pretrained(cls, path: str) -> "ZasevikConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def __eq__(self, other: object) -> bool:
        return isinstance(other, ZasevikConfig) and self.to_dict() == other.to_dict()

    def __repr__(self) -> str:
        return f"ZasevikConfig {json.dumps(self.to_dict(), sort_keys=True)}"


# -------------------------------------------------------------------------------------
# Besulix: matrix-memory layers alternating with a chunked attention beside a time-mix recurrence
# -------------------------------------------------------------------------------------
@dataclass
class MLSTMSpec:
    """Matrix memory with exponential gates: ``heads`` heads of key size ``dim`` and value size ``vdim``; the gate
    pre-activations are capped at ``gate_cap`` by a tanh."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float
    type = "mlstm"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MLSTMSpec":
        heads, dim = int(d["heads"]), int(d["dim"])
        return cls(heads=heads, dim=dim, vdim=int(d.get("vdim", dim)), gate_cap=float(d["gate_cap"]))

    def to_dict(self) -> Dict[str, Any]:
        return dict(heads=self.heads, dim=self.dim, vdim=self.vdim, gate_cap=self.gate_cap)


@dataclass
class ChunkedAttentionSpec:
    """Softmax attention with projection biases, rotary positions on the first ``rot_dims`` numbers of each q / k head
    (and over the whole value head: values are cached rotated by their position and the sum is turned back), a
    temperature and a sink per head, and a mask that keeps a query inside its block of ``chunk`` positions."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    chunk: int
    type = "chunked_attention"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ChunkedAttentionSpec":
        heads, dim = int(d["heads"]), int(d["dim"])
        out = cls(heads=heads, kv_heads=int(d.get("kv_heads", heads)), dim=dim, vdim=int(d.get("vdim", dim)),
                  scale=float(d["scale"]), rot_base=float(d["rot"]["base"]), rot_dims=int(d["rot"]["dims"]),
                  chunk=int(d["mask"]["size"]))
        if out.heads % out.kv_heads:
            raise ValueError("heads must be divisible by kv_heads")
        if out.rot_dims % 2 or out.rot_dims > out.dim or out.vdim % 2:
            raise ValueError("rotary sizes: rot.dims even and at most dim, vdim even")
        if out.chunk < 1:
            raise ValueError("mask.size must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        return dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim, scale=self.scale,
                    rot={"base": self.rot_base, "dims": self.rot_dims}, mask={"size": self.chunk})


@dataclass
class TimeMixSpec:
    """Token-shifted linear recurrence with a decay per key channel: ``heads`` heads of size ``dim`` (keys and values)."""

    heads: int
    dim: int
    type = "timemix"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TimeMixSpec":
        return cls(heads=int(d["heads"]), dim=int(d["dim"]))

    def to_dict(self) -> Dict[str, Any]:
        return dict(heads=self.heads, dim=self.dim)


@dataclass
class ParallelSpec:
    """Two mixers reading the same input; their outputs are summed with fixed weights."""

    left: ChunkedAttentionSpec
    right: TimeMixSpec
    left_scale: float
    right_scale: float
    type = "parallel"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ParallelSpec":
        return cls(left=ChunkedAttentionSpec.from_dict(d["left"]), right=TimeMixSpec.from_dict(d["right"]),
                   left_scale=float(d["left_scale"]), right_scale=float(d["right_scale"]))

    def to_dict(self) -> Dict[str, Any]:
        return dict(left=self.left.to_dict(), right=self.right.to_dict(), left_scale=self.left_scale,
                    right_scale=self.right_scale)


@dataclass
class ClampedFFSpec:
    """Dense gated feed-forward of width ``ff`` whose gate and up pre-activations are clamped at ``limit``."""

    ff: int
    limit: float
    kind = "dense"

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


class BesulixConfig:
    """Besulix decoder: ``config.json`` with ``architecture: "Besulix"``, ``vocab``, ``width``, ``norm.eps``,
    ``logit_softcap`` and a ``layers`` list of ``{type, mixer, mlp}`` entries; ``type`` is ``mlstm`` or ``parallel``,
    ``mlp`` null or ``{kind: dense, ff, limit}``."""

    model_type = "besulix"
    architecture = "Besulix"
    MIXERS = {"mlstm": MLSTMSpec, "parallel": ParallelSpec}

    def __init__(self, vocab_size: int, hidden_size: int, layers, norm_eps: float = 1e-6, logit_softcap: float = 0.0,
                 pad_token_id: int = -1, eos_token_id: Optional[int] = None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.layers = list(layers)
        self.norm_eps = float(norm_eps)
        self.logit_softcap = float(logit_softcap or 0.0)
        self.pad_token_id = pad_token_id
        self.eos_token_id = eos_token_id

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "BesulixConfig":
        layers = []
        for i, e in enumerate(d["layers"]):
            if e["type"] not in cls.MIXERS:
                raise ValueError(f"layer {i}: Besulix has no mixer {e['type']!r}")
            f = e.get("mlp")
            if f is not None and f.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
            layers.append(LayerSpec(cls.MIXERS[e["type"]].from_dict(e["mixer"]),
                                    ClampedFFSpec(ff=int(f["ff"]), limit=float(f["limit"])) if f is not None else None))
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], layers=layers, norm_eps=d["norm"]["eps"],
                   logit_softcap=d.get("logit_softcap", 0.0), pad_token_id=d.get("pad_token_id", -1),
                   eos_token_id=d.get("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                "norm": {"eps": self.norm_eps}, "logit_softcap": self.logit_softcap,
                "layers": [{"type": ls.mixer.type, "mixer": ls.mixer.to_dict(),
                            "mlp": ls.mlp.to_dict() if ls.mlp is not None else None} for ls in self.layers]}

    def save_pretrained(self, save_directory: str) -> None:
        os.makedirs(save_directory, exist_ok=True)
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=1, sort_keys=True)

    @classmethod
    def from_pretrained(cls, path: str) -> "BesulixConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def __eq__(self, other: object) -> bool:
        return isinstance(other, BesulixConfig) and self.to_dict() == other.to_dict()

    def __repr__(self) -> str:
        return f"BesulixConfig {json.dumps(self.to_dict(), sort_keys=True)}"


# -------------------------------------------------------------------------------------
# Zifisun: windowed latent / normed attention, grouped routing with identity experts, several residual streams
# -------------------------------------------------------------------------------------
def _mask_from(d: Optional[Dict[str, Any]]):
    """``(window, keep_first)`` of a mixer's ``mask`` entry (absent: plain causal attention)."""
    d = d or {}
    window, keep = int(d.get("size") or 0), int(d.get("keep_first") or 0)
    if window < 0 or keep < 0:
        raise ValueError("mask.size and mask.keep_first must not be negative")
    return window, keep


def _mask_to(window: int, keep_first: int) -> Optional[Dict[str, Any]]:
    if not window:
        return None
    return {"size": window, "keep_first": keep_first} if keep_first else {"size": window}


@dataclass
class RotaryLatentSpec:
    """Latent attention with a query latent and one rotated key part: ``heads`` heads of ``dim`` plain and ``rot_dim``
    rotated query / key numbers and ``vdim`` value numbers; keys and values come from ``kv_rank`` cached numbers per
    token, queries from ``q_rank``; rotary base ``rot_base`` over ``rot_dims`` of the rotated part; a query sees the last
    ``window`` positions (0: all) and the first ``keep_first`` of the sequence."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: int = 0
    keep_first: int = 0
    type = "latent_attention"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "RotaryLatentSpec":
        dim, rot_dim = int(d["dim"]), int(d.get("rot_dim", 0) or 0)
        rot = d.get("rot") or {}
        window, keep = _mask_from(d.get("mask"))
        out = cls(heads=int(d["heads"]), dim=dim, rot_dim=rot_dim, vdim=int(d.get("vdim", dim)), kv_rank=int(d["kv_rank"]),
                  q_rank=int(d["q_rank"]), scale=float(d["scale"]), rot_base=float(rot.get("base", 10000.0)),
                  rot_dims=int(rot.get("dims", rot_dim)), window=window, keep_first=keep)
        if out.rot_dims % 2 or out.rot_dims > out.rot_dim:
            raise ValueError("rot.dims must be even and at most rot_dim")
        if min(out.heads, out.dim, out.vdim, out.kv_rank, out.q_rank) < 1:
            raise ValueError("latent_attention: sizes must be positive")
        return out

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = dict(heads=self.heads, dim=self.dim, rot_dim=self.rot_dim, vdim=self.vdim,
                                   kv_rank=self.kv_rank, q_rank=self.q_rank, scale=self.scale,
                                   rot={"base": self.rot_base, "dims": self.rot_dims})
        mask = _mask_to(self.window, self.keep_first)
        if mask:
            out["mask"] = mask
        return out


@dataclass
class NormedAttentionSpec:
    """Softmax attention without positions: ``heads`` query heads over ``kv_heads`` key / value heads, q and k RMS-normed
    per head with a weight, an output gate per head, a sliding window that may keep the sequence's first keys."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    keep_first: int = 0
    type = "attention"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "NormedAttentionSpec":
        heads, dim = int(d["heads"]), int(d["dim"])
        window, keep = _mask_from(d.get("mask"))
        out = cls(heads=heads, kv_heads=int(d.get("kv_heads", heads)), dim=dim, vdim=int(d.get("vdim", dim)),
                  scale=float(d["scale"]), window=window, keep_first=keep)
        if out.heads % out.kv_heads:
            raise ValueError("heads must be divisible by kv_heads")
        return out

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim, scale=self.scale)
        mask = _mask_to(self.window, self.keep_first)
        if mask:
            out["mask"] = mask
        return out


@dataclass
class GroupedMoESpec:
    """Softmax-routed mixture: ``experts`` squared-ReLU experts of width ``ff`` plus ``identity`` identity experts, ``top``
    of them per token, chosen inside the ``keep_groups`` best of ``groups`` equal groups; an optional shared expert of
    width ``shared_ff`` for every token."""

    experts: int
    identity: int
    top: int
    groups: int
    keep_groups: int
    ff: int
    shared_ff: int = 0
    kind = "moe"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GroupedMoESpec":
        if d.get("kind", "moe") != "moe":
            raise ValueError(f"unknown feed-forward kind {d.get('kind')!r}")
        r = d["router"]
        gr = r.get("groups") or {}
        out = cls(experts=int(r["experts"]), identity=int(r.get("identity", 0) or 0), top=int(r["top"]),
                  groups=int(gr.get("count", 1)), keep_groups=int(gr.get("keep", gr.get("count", 1))),
                  ff=int(d["expert"]["ff"]), shared_ff=int((d.get("shared") or {}).get("ff", 0)))
        total = out.experts + out.identity
        if out.groups < 1 or total % out.groups or not 1 <= out.keep_groups <= out.groups:
            raise ValueError(f"router: {total} experts do not form {out.groups} equal groups of which {out.keep_groups} are kept")
        if not 1 <= out.top <= out.keep_groups * (total // out.groups):
            raise ValueError(f"router: top {out.top} does not fit the kept groups")
        return out

    def to_dict(self) -> Dict[str, Any]:
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.identity:
            router["identity"] = self.identity
        if self.groups > 1:
            router["groups"] = {"count": self.groups, "keep": self.keep_groups}
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


class ZifisunConfig:
    """Zifisun decoder: ``config.json`` with ``architecture: "Zifisun"``, ``vocab``, ``width``, ``norm.eps``, ``streams``
    (residual streams of the hyper-connections; absent: one plain residual), ``loop`` (``{start, stop, times}``: layers
    ``start .. stop - 1`` run ``times`` times in a row with the same weights; absent: every layer once) and a ``layers``
    list of ``{type, mixer, mlp}`` entries; ``type`` is ``latent_attention`` or ``attention``, ``mlp`` null or a
    ``GroupedMoESpec`` entry."""

    model_type = "zifisun"
    architecture = "Zifisun"
    MIXERS = {"latent_attention": RotaryLatentSpec, "attention": NormedAttentionSpec}

    def __init__(self, vocab_size: int, hidden_size: int, layers, norm_eps: float = 1e-6, streams: int = 0,
                 loop_start: int = 0, loop_stop: int = 0, loop_times: int = 1, pad_token_id: int = -1,
                 eos_token_id: Optional[int] = None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.layers = list(layers)
        self.norm_eps = float(norm_eps)
        self.streams = int(streams or 0)  # 0: no hyper-connection tensors, a plain residual
        self.loop_start, self.loop_stop, self.loop_times = int(loop_start), int(loop_stop), int(loop_times)
        self.pad_token_id = pad_token_id
        self.eos_token_id = eos_token_id
        if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers) or self.loop_times < 1:
            raise ValueError(f"loop {self.loop_start}..{self.loop_stop} x {self.loop_times} does not fit "
                             f"{len(self.layers)} layers")

    def layer_runs(self) -> list:
        """The layer index of every layer run, in order (a looped layer appears once per pass; each run has its own
        cache)."""
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, len(self.layers)))

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layer_runs())

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZifisunConfig":
        layers = []
        for i, e in enumerate(d["layers"]):
            if e["type"] not in cls.MIXERS:
                raise ValueError(f"layer {i}: Zifisun has no mixer {e['type']!r}")
            f = e.get("mlp")
            layers.append(LayerSpec(cls.MIXERS[e["type"]].from_dict(e["mixer"]),
                                    GroupedMoESpec.from_dict(f) if f is not None else None))
        loop = d.get("loop") or {}
        return cls(vocab_size=d["vocab"], hidden_size=d["width"], layers=layers, norm_eps=d["norm"]["eps"],
                   streams=d.get("streams", 0), loop_start=loop.get("start", 0), loop_stop=loop.get("stop", 0),
                   loop_times=loop.get("times", 1), pad_token_id=d.get("pad_token_id", -1),
                   eos_token_id=d.get("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                               "norm": {"eps": self.norm_eps},
                               "layers": [{"type": ls.mixer.type, "mixer": ls.mixer.to_dict(),
                                           "mlp": ls.mlp.to_dict() if ls.mlp is not None else None} for ls in self.layers]}
        if self.streams:
            out["streams"] = self.streams
        if self.loop_stop > self.loop_start and self.loop_times != 1:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return out

    def save_pretrained(self, save_directory: str) -> None:
        os.makedirs(save_directory, exist_ok=True)
        with open(os.path.join(save_directory, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=1, sort_keys=True)

    @classmethod
    def from_pretrained(cls, path: str) -> "ZifisunConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def __eq__(self, other: object) -> bool:
        return isinstance(other, ZifisunConfig) and self.to_dict() == other.to_dict()

    def __repr__(self) -> str:
        return f"ZifisunConfig {json.dumps(self.to_dict(), sort_keys=True)}"
