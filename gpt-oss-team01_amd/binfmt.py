"""Flat ``.bin`` checkpoint format of the reference, unchanged.

Header: 15 little-endian 4-byte fields (reference ``run.cpp:25-45``,
``export_model_bin/gpt-oss-7m/generate_bin.py:15-21,46-57``), then fp32 tensors in the order the
reference's loader walks them (``run.cpp:194-233``).
"""
from __future__ import annotations

import struct
from collections import OrderedDict
from dataclasses import dataclass, asdict

import numpy as np

HEADER_FIELDS = (
    ("vocab_size", "i"), ("hidden_dim", "i"), ("n_experts", "i"), ("experts_per_token", "i"),
    ("intermediate_dim", "i"), ("n_layers", "i"), ("head_dim", "i"), ("n_attn_heads", "i"),
    ("n_kv_heads", "i"), ("seq_len", "i"), ("initial_context_length", "i"),
    ("rope_theta", "f"), ("rope_scaling_factor", "f"), ("sliding_window", "i"),
    ("swiglu_limit", "f"),
)
HEADER_STRUCT = struct.Struct("<" + "".join(f for _, f in HEADER_FIELDS))
HEADER_BYTES = HEADER_STRUCT.size  # 60


@dataclass
class Config:
    vocab_size: int
    hidden_dim: int
    n_experts: int
    experts_per_token: int
    intermediate_dim: int
    n_layers: int
    head_dim: int
    n_attn_heads: int
    n_kv_heads: int
    seq_len: int
    initial_context_length: int
    rope_theta: float
    rope_scaling_factor: float
    sliding_window: int
    swiglu_limit: float

    def pack(self) -> bytes:
        return HEADER_STRUCT.pack(*[getattr(self, n) for n, _ in HEADER_FIELDS])

    @classmethod
    def unpack(cls, raw: bytes) -> "Config":
        return cls(*HEADER_STRUCT.unpack(raw[:HEADER_BYTES]))

    def as_dict(self):
        return asdict(self)


def tensor_shapes(c: Config) -> "OrderedDict[str, tuple]":
    """Tensor names and shapes in file order (``run.cpp:194-233``)."""
    H, V, L, E = c.hidden_dim, c.vocab_size, c.n_layers, c.n_experts
    D, nq, nkv, I = c.head_dim, c.n_attn_heads, c.n_kv_heads, c.intermediate_dim
    qkv = D * (nq + 2 * nkv)
    return OrderedDict([
        ("embedding", (V, H)), ("unembedding", (V, H)),
        ("attn_norm", (L, H)), ("mlp_norm", (L, H)), ("final_norm", (H,)),
        ("qkv_weight", (L, qkv, H)), ("qkv_bias", (L, qkv)),
        ("out_weight", (L, H, nq * D)), ("out_bias", (L, H)),
        ("sinks", (L, nq)),
        ("gate_weight", (L, E, H)), ("gate_bias", (L, E)),
        ("mlp1_weight", (L, E, 2 * I, H)), ("mlp1_bias", (L, E, 2 * I)),
        ("mlp2_weight", (L, E, H, I)), ("mlp2_bias", (L, E, H)),
    ])


def n_weight_floats(c: Config) -> int:
    return int(sum(int(np.prod(s)) for s in tensor_shapes(c).values()))


def write_bin(path: str, c: Config, tensors: dict) -> None:
    with open(path, "wb") as f:
        f.write(c.pack())
        for name, shape in tensor_shapes(c).items():
            t = np.ascontiguousarray(tensors[name], dtype="<f4")
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {t.shape} != {shape}")
            f.write(t.tobytes())


def read_bin(path: str, mmap: bool = True):
    """Returns (Config, dict name -> float32 array view)."""
    with open(path, "rb") as f:
        c = Config.unpack(f.read(HEADER_BYTES))
    data = np.memmap(path, dtype="<f4", mode="r", offset=HEADER_BYTES) if mmap else \
        np.fromfile(path, dtype="<f4", offset=HEADER_BYTES)
    need = n_weight_floats(c)
    if data.size < need:
        raise ValueError(f"{path}: {data.size} floats, need {need}")
    out, off = OrderedDict(), 0
    for name, shape in tensor_shapes(c).items():
        n = int(np.prod(shape))
        out[name] = data[off:off + n].reshape(shape)
        off += n
    return c, out
