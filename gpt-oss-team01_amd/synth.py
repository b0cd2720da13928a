"""Synthetic, seeded GPT-OSS-architecture checkpoints and inputs (random-init, bf16-representable
values stored as fp32 like the reference's exporters do)."""
from __future__ import annotations

import numpy as np

from .binfmt import Config, tensor_shapes


def bf16_round(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16, returned as fp32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return u.astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def tiny_config(max_seq_len: int = 2048) -> Config:
    """The tiny end-to-end configuration: 4 blocks, hidden 256, 8 query / 2 KV heads of 32,
    8 experts top-4, intermediate 256, vocab 4096, theta 150000, window 128.  RoPE scaling 32 and
    initial context 4096 as in the reference's 20B config.json."""
    return Config(vocab_size=4096, hidden_dim=256, n_experts=8, experts_per_token=4,
                  intermediate_dim=256, n_layers=4, head_dim=32, n_attn_heads=8, n_kv_heads=2,
                  seq_len=max_seq_len, initial_context_length=4096, rope_theta=150000.0,
                  rope_scaling_factor=32.0, sliding_window=128, swiglu_limit=7.0)


def gptoss20b_config(max_seq_len: int = 1024) -> Config:
    return Config(vocab_size=201088, hidden_dim=2880, n_experts=32, experts_per_token=4,
                  intermediate_dim=2880, n_layers=24, head_dim=64, n_attn_heads=64, n_kv_heads=8,
                  seq_len=max_seq_len, initial_context_length=4096, rope_theta=150000.0,
                  rope_scaling_factor=32.0, sliding_window=128, swiglu_limit=7.0)


def random_tensors(c: Config, seed: int, std: float = 0.02, gate_scale: float = 1.0) -> dict:
    """bf16-rounded N(0, std) for every tensor; norm scales are 1 + N(0, std).  gate_scale (a power
    of two, so the values stay bf16) multiplies the router's weight and bias: wider router scores,
    fewer near-ties between the k-th and (k+1)-th expert."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(c).items():
        t = rng.standard_normal(size=shape, dtype=np.float32) * np.float32(std)
        if name in ("attn_norm", "mlp_norm", "final_norm"):
            t = t + np.float32(1.0)
        if name in ("gate_weight", "gate_bias"):
            t = t * np.float32(gate_scale)
        out[name] = bf16_round(t)
    return out


def random_prompts(c: Config, n_req: int, n_tokens: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.integers(0, c.vocab_size, size=(n_req, n_tokens), dtype=np.int32)
