"""Model registry: HF `architectures[0]` -> implementation class."""

from __future__ import annotations

from ..config import ModelConfig
from .hybrid import HybridForCausalLM
from .llama_family import LlamaFamilyForCausalLM

_REGISTRY = {
    "Qwen2ForCausalLM": LlamaFamilyForCausalLM,
    "LlamaForCausalLM": LlamaFamilyForCausalLM,
    "MixtralForCausalLM": LlamaFamilyForCausalLM,  # sparse MoE MLP branch
    # Mistral v0.3+ ships sliding_window=null -> plain llama arch; models
    # that DO set a window are rejected at config load (no SWA kernels yet)
    "MistralForCausalLM": LlamaFamilyForCausalLM,
    "Qwen3ForCausalLM": LlamaFamilyForCausalLM,  # + per-head q/k RMSNorm
    "Qwen3MoeForCausalLM": LlamaFamilyForCausalLM,  # qk-norm + sparse MoE
    "Qwen2MoeForCausalLM": LlamaFamilyForCausalLM,  # MoE + shared expert
    # llama arch + NoPE every no_rope_layer_interval-th layer + tied embeds
    "SmolLM3ForCausalLM": LlamaFamilyForCausalLM,
    # layer-list decoder: attention / lightning / mamba1 mixers, fp32
    # residual, token shift + gated residual (models/hybrid.py)
    "Gagorax": HybridForCausalLM,
    # layer-list decoder: residual in weighted copies, layer norm + short
    # input convolution, window/pooled attention beside retention, clamped
    # GLU or group-routed experts (models/hybrid.py StreamBlock)
    "Fusolix": HybridForCausalLM,
    # layer-list decoder: one tanh norm per layer in front of a mixer and a
    # GELU GLU side by side; capped window attention that keeps the first
    # tokens, latent attention, mamba2; a looped run of layers
    # (models/hybrid.py SharedNormBlock)
    "Legalix": HybridForCausalLM,
    # layer-list decoder: two RMS norms of one residual in front of a mixer
    # and routed experts side by side, each result scaled per channel;
    # two-map difference attention behind short convolutions (optionally on
    # an earlier layer's keys and values), attention whose values are its
    # keys; logits through the embedding table (models/hybrid.py
    # DualNormBlock)
    "Rivolix": HybridForCausalLM,
}


def create_model(cfg, dtype=None):
    import torch

    cls = _REGISTRY.get(cfg.architecture)
    if cls is None:
        raise ValueError(
            f"unsupported architecture {cfg.architecture!r}; known: {sorted(_REGISTRY)}"
        )
    return cls(cfg, dtype=dtype or torch.bfloat16)
