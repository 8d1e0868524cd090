"""Seeded synthetic inputs for the five benchmark configurations of the backbone kernel path.

All tensors are drawn on the CPU from a ``torch.Generator`` with a fixed seed and moved to the target device by the
caller, the practice of the reference's operator benchmark
(src/taac2026/application/benchmarking/pcvr_tilelang_ops_benchmark.py:433-462, seed 42). Every generator takes the
shape parameters as arguments so that tests can draw small instances of the same distributions.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

SEED = 42


def _generator(seed: int) -> torch.Generator:
    generator = torch.Generator(device="cpu")
    generator.manual_seed(seed)
    return generator


def rmsnorm_fp32_inputs(batch: int = 1024, tokens: int = 64, dim: int = 128, *, seed: int = SEED):
    """Config 1: x ~ N(0,1) [B, T, D] fp32, weight ~ N(1, 0.1), eps 1e-6."""
    g = _generator(seed)
    x = torch.randn(batch, tokens, dim, generator=g)
    weight = 1.0 + 0.1 * torch.randn(dim, generator=g)
    return x, weight, 1e-6


def norm_bf16_inputs(batch: int = 4096, tokens: int = 256, dim: int = 256, *, outlier_fraction: float = 0.01,
                     outlier_scale: float = 50.0, seed: int = SEED):
    """Config 2: x ~ N(0,1) with 1 % of the rows scaled x50, gamma ~ N(1, 0.1), beta ~ N(0, 0.02), all bf16."""
    g = _generator(seed)
    x = torch.randn(batch, tokens, dim, generator=g)
    rows = batch * tokens
    picked = torch.randperm(rows, generator=g)[: max(1, int(rows * outlier_fraction))]
    x.view(rows, dim)[picked] *= outlier_scale
    gamma = 1.0 + 0.1 * torch.randn(dim, generator=g)
    beta = 0.02 * torch.randn(dim, generator=g)
    return x.to(torch.bfloat16), gamma.to(torch.bfloat16), beta.to(torch.bfloat16)


def attention_inputs(batch: int = 2048, heads: int = 4, tokens: int = 256, head_dim: int = 64, *, min_len: int = 16,
                     seed: int = SEED, dtype: torch.dtype = torch.bfloat16):
    """Config 3: q, k, v ~ N(0,1) [B, H, T, d]; valid length ~ U{min_len..T} per sample (right padding)."""
    g = _generator(seed)
    q = torch.randn(batch, heads, tokens, head_dim, generator=g).to(dtype)
    k = torch.randn(batch, heads, tokens, head_dim, generator=g).to(dtype)
    v = torch.randn(batch, heads, tokens, head_dim, generator=g).to(dtype)
    lengths = torch.randint(min_len, tokens + 1, (batch,), generator=g, dtype=torch.int32)
    return q, k, v, lengths


@dataclass
class BackboneInputs:
    emb: torch.Tensor  # [B, T, D] bf16
    key_lengths: torch.Tensor  # [B] int32, n_feature_tokens + sequence length
    blocks: list[dict[str, torch.Tensor]]  # bf16 weights, reference parameter names
    head_weight: torch.Tensor  # [1, D] bf16
    head_bias: torch.Tensor  # [1] bf16
    num_heads: int
    d_ff: int


def _xavier_uniform(out_features: int, in_features: int, g: torch.Generator) -> torch.Tensor:
    bound = (6.0 / (in_features + out_features)) ** 0.5
    return (torch.rand(out_features, in_features, generator=g) * 2.0 - 1.0) * bound


def backbone_inputs(batch: int = 1024, n_feature_tokens: int = 32, n_sequence_tokens: int = 480, d_model: int = 256,
                    num_heads: int = 8, d_ff: int = 1024, n_blocks: int = 4, *, min_sequence_len: int = 32,
                    seed: int = SEED, qk_norm: bool = False) -> BackboneInputs:
    """Config 4: emb ~ N(0, 0.02) [B, 32 + 480, 256] bf16; sequence valid length ~ U{32..480}; Xavier-uniform
    weights, zero biases, unit norm weights. ``qk_norm`` adds the (unit) weights of the reference layer's query / key
    RMSNorm, which the benchmark recipe leaves out."""
    g = _generator(seed)
    tokens = n_feature_tokens + n_sequence_tokens
    emb = (0.02 * torch.randn(batch, tokens, d_model, generator=g)).to(torch.bfloat16)
    seq_len = torch.randint(min_sequence_len, n_sequence_tokens + 1, (batch,), generator=g, dtype=torch.int32)
    key_lengths = (n_feature_tokens + seq_len).to(torch.int32)
    blocks = []
    for _ in range(n_blocks):
        blocks.append(
            {
                "attn_norm.weight": torch.ones(d_model, dtype=torch.bfloat16),
                "qkv.weight": _xavier_uniform(3 * d_model, d_model, g).to(torch.bfloat16),
                "qkv.bias": torch.zeros(3 * d_model, dtype=torch.bfloat16),
                "out.weight": _xavier_uniform(d_model, d_model, g).to(torch.bfloat16),
                "out.bias": torch.zeros(d_model, dtype=torch.bfloat16),
                "ffn_norm.weight": torch.ones(d_model, dtype=torch.bfloat16),
                "up.weight": _xavier_uniform(2 * d_ff, d_model, g).to(torch.bfloat16),
                "up.bias": torch.zeros(2 * d_ff, dtype=torch.bfloat16),
                "down.weight": _xavier_uniform(d_model, d_ff, g).to(torch.bfloat16),
                "down.bias": torch.zeros(d_model, dtype=torch.bfloat16),
            }
        )
    if qk_norm:
        for weights in blocks:
            weights["query_norm.weight"] = torch.ones(d_model, dtype=torch.bfloat16)
            weights["key_norm.weight"] = torch.ones(d_model, dtype=torch.bfloat16)
    head_weight = _xavier_uniform(1, d_model, g).to(torch.bfloat16)
    head_bias = torch.zeros(1, dtype=torch.bfloat16)
    return BackboneInputs(emb, key_lengths, blocks, head_weight, head_bias, num_heads, d_ff)


def load_backbone_state(model, inputs: BackboneInputs) -> None:
    """Copy a ``BackboneInputs`` weight set into a ``PCVRBackbone`` (parameter names match)."""
    with torch.no_grad():
        for block, weights in zip(model.blocks, inputs.blocks):
            for name, value in weights.items():
                module_name, parameter_name = name.split(".")
                getattr(getattr(block, module_name), parameter_name).copy_(value)
        model.head.weight.copy_(inputs.head_weight)
        model.head.bias.copy_(inputs.head_bias)


__all__ = [
    "BackboneInputs",
    "SEED",
    "attention_inputs",
    "backbone_inputs",
    "load_backbone_state",
    "norm_bf16_inputs",
    "rmsnorm_fp32_inputs",
]
