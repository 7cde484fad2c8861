"""jax_llama_amd — an MI355X-native (gfx950 / CDNA4) LLaMA-1/2/3 inference framework with the
public API of LSaldyt/JAX_llama (reference ``jax_llama/__init__.py:4-10``), plus a model registry with a second
family (Zavevik: gated delta rule + biased attention + table-routed experts) and a third (Zasevik: latent attention
with a softmax sink + dense / score-routed feed-forwards) and a fourth (Besulix: matrix memories + block-local rotary
attention beside a time-mix recurrence) and a fifth (Zifisun: windowed latent / normed attention, grouped routing with
identity experts, several residual streams) on the same layer-list step function.

Framework layer: PyTorch-ROCm. Hot path: hand-written HIP kernels (``csrc/kernels``).
Multi-GPU: one process per GPU, RCCL + a custom xGMI all-reduce. Decode: hipGraph replay.
"""
from .config import BesulixConfig, LLaMAConfig, ModelArgs, ZasevikConfig, ZavevikConfig, ZifisunConfig, config_from_params, get_preset, swiglu_hidden_size
from .generation import LLaMA
from .models import (CausalLMOutput, FlaxLLaMAForCausalLM, FlaxLLaMAModel, KVCache, LLaMAForCausalLM,
                     LLaMAModel)
from .parallel.partition import (Mesh, P, PartitionSpec, get_llama_param_partition_spec,
                                 with_named_sharding_constraint, with_sharding_constraint)
from .models.registry import load_model
from .models.zasevik import ZasevikForCausalLM
from .models.besulix import BesulixForCausalLM
from .models.zifisun import ZifisunForCausalLM
from .models.zavevik import ZavevikForCausalLM
from .runtime.engine import GenerationConfig
from .runtime.stepper import SequenceStepper
from .tokenizer import ChatFormat, LLaMA2Tokenizer, LLaMA3Tokenizer
from .utils.checkpoint import convert_llama_weights

__version__ = "0.1.0"

__all__ = [
    "LLaMAConfig", "ModelArgs", "config_from_params", "get_preset", "swiglu_hidden_size",
    "LLaMA", "LLaMAForCausalLM", "LLaMAModel", "FlaxLLaMAForCausalLM", "FlaxLLaMAModel",
    "CausalLMOutput", "KVCache", "GenerationConfig",
    "Mesh", "P", "PartitionSpec", "get_llama_param_partition_spec", "with_named_sharding_constraint",
    "with_sharding_constraint", "LLaMA2Tokenizer", "LLaMA3Tokenizer", "ChatFormat", "convert_llama_weights",
    "ZavevikConfig", "ZavevikForCausalLM", "ZasevikConfig", "ZasevikForCausalLM", "BesulixConfig", "BesulixForCausalLM", "ZifisunConfig", "ZifisunForCausalLM", "SequenceStepper", "load_model",
]
