#!/usr/bin/env python3
"""Writes tests/golden/synthetic_qwen3moe.gguf: the synthetic one-layer MoE model file that the reference's loader test
assembles field by field (write_synthetic_qwen3moe_gguf, tests/graph/test_gguf_loader.c:171-256), in that test's
order: header (magic, version 3, tensor count, 16 key/value pairs), the key/value pairs, the tensor infos with
offsets that simply accumulate the tensors' sizes (no per-tensor alignment: the 16-byte norm weights leave later
offsets at 16 modulo 32), zero padding to the 32-byte alignment, then the FLOAT32 data.

The reference's test leaves the data zero; here tensor t holds the values t + j / 1024 (j its element index in file
order) so that a reader that resolves an offset or a size wrongly shows up. Everything else follows the test."""
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
GGUF_TYPE_UINT32, GGUF_TYPE_FLOAT32, GGUF_TYPE_STRING = 4, 6, 8

TENSORS = [
    ("output_norm.weight", (8,)),
    ("output.weight", (8, 16)),
    ("blk.0.attn_norm.weight", (8,)),
    ("blk.0.attn_q.weight", (8, 8)),
    ("blk.0.attn_k.weight", (8, 4)),
    ("blk.0.attn_v.weight", (8, 4)),
    ("blk.0.attn_output.weight", (8, 8)),
    ("blk.0.attn_q_norm.weight", (4,)),
    ("blk.0.attn_k_norm.weight", (4,)),
    ("blk.0.ffn_norm.weight", (8,)),
    ("blk.0.ffn_gate_inp.weight", (8, 2)),
    ("blk.0.ffn_gate_exps.weight", (8, 6, 2)),
    ("blk.0.ffn_up_exps.weight", (8, 6, 2)),
    ("blk.0.ffn_down_exps.weight", (6, 8, 2)),
    ("blk.0.ffn_gate_shexp.weight", (8, 6)),
    ("blk.0.ffn_up_shexp.weight", (8, 6)),
    ("blk.0.ffn_down_shexp.weight", (6, 8)),
]

KV = [
    ("general.architecture", GGUF_TYPE_STRING, "qwen3moe"),
    ("general.alignment", GGUF_TYPE_UINT32, 32),
    ("qwen3moe.context_length", GGUF_TYPE_UINT32, 32),
    ("qwen3moe.embedding_length", GGUF_TYPE_UINT32, 8),
    ("qwen3moe.block_count", GGUF_TYPE_UINT32, 1),
    ("qwen3moe.attention.head_count", GGUF_TYPE_UINT32, 2),
    ("qwen3moe.attention.head_count_kv", GGUF_TYPE_UINT32, 1),
    ("qwen3moe.feed_forward_length", GGUF_TYPE_UINT32, 6),
    ("qwen3moe.rope.dimension_count", GGUF_TYPE_UINT32, 4),
    ("qwen3moe.attention.key_length", GGUF_TYPE_UINT32, 4),
    ("qwen3moe.attention.layer_norm_rms_epsilon", GGUF_TYPE_FLOAT32, 1.0e-5),
    ("qwen3moe.rope.freq_base", GGUF_TYPE_FLOAT32, 10000.0),
    ("qwen3moe.expert_count", GGUF_TYPE_UINT32, 2),
    ("qwen3moe.expert_used_count", GGUF_TYPE_UINT32, 1),
    ("qwen3moe.expert_shared_count", GGUF_TYPE_UINT32, 1),
    ("qwen3moe.expert_weights_scale", GGUF_TYPE_FLOAT32, 1.25),
]


def string(s: str) -> bytes:
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def tensor_values(t: int, dims) -> np.ndarray:
    n = int(np.prod(dims))
    return (np.float32(t) + np.arange(n, dtype=np.float32) / np.float32(1024.0)).astype(np.float32)


def build() -> bytes:
    out = bytearray()
    out += struct.pack("<IIQQ", 0x46554747, 3, len(TENSORS), len(KV))
    for key, typ, value in KV:
        out += string(key) + struct.pack("<I", typ)
        out += string(value) if typ == GGUF_TYPE_STRING else struct.pack("<I" if typ == GGUF_TYPE_UINT32 else "<f", value)
    offset = 0
    for name, dims in TENSORS:
        out += string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", 0, offset)  # ggml type 0 = FLOAT32
        offset += int(np.prod(dims)) * 4
    out += bytes(-len(out) % 32)
    for t, (_, dims) in enumerate(TENSORS):
        out += tensor_values(t, dims).tobytes()
    return bytes(out)


if __name__ == "__main__":
    path = os.path.join(HERE, "synthetic_qwen3moe.gguf")
    with open(path, "wb") as f:
        f.write(build())
    print("wrote", path, os.path.getsize(path), "bytes")
