"""CPU: the library's GGUF reader (host code, no GPU call) against files written by tests/gguf_writer.py: header and
key/value skipping, general.alignment, the loader's shape convention ([rows, cols] for matrices, file order for
expert stacks), the ggml-type mapping of every weight format, views that alias the file's bytes, error paths; and
against a committed file laid out like the synthetic MoE model of the reference's own loader test."""
import os
import struct

import numpy as np
import pytest

from marmot_amd import capi
from marmot_amd.gguf import GgufFile
from oracle.pyoracle import BLOCK_BYTES, BLOCK_VALUES, KINDS
from tests.gguf_writer import write_gguf
from tests.util import gaussian, random_valid_blocks

WEIGHT_KINDS = ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q8_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"]


def test_every_weight_format_round_trips(tmp_path, oracle):
    rng = np.random.default_rng(1)
    tensors, want = [], {}
    for name in WEIGHT_KINDS:
        kind = KINDS[name]
        rows, cols = 6, 512
        blocks = random_valid_blocks(rng, kind, rows, cols)
        tensors.append((f"blk.0.{name}.weight", name, (cols, rows), blocks))
        want[f"blk.0.{name}.weight"] = (kind, (rows, cols), blocks)
    norm = gaussian(2, (512,))
    tensors.append(("output_norm.weight", "f32", (512,), norm))
    experts = random_valid_blocks(rng, KINDS["q4_k"], 3 * 8, 256)  # [cols=256, rows=8, experts=3]
    tensors.append(("blk.0.ffn_gate_exps.weight", "q4_k", (256, 8, 3), experts))
    path = write_gguf(str(tmp_path / "m.gguf"), tensors,
                      kv={"general.architecture": "llama", "llama.block_count": 1, "tokenizer.ggml.tokens": ["a", "bc"],
                          "llama.rope.freq_base": 10000.0, "some.flag": True, "some.ints": [1, 2, 3]})
    with GgufFile(path) as g:
        assert g.alignment == 32 and len(g.tensors) == len(tensors)
        for name, (kind, shape, blocks) in want.items():
            t = g.find(name)
            assert (t.kind, t.shape, t.dtype) == (kind, shape, 6)
            assert t.nbytes == shape[0] * (shape[1] // BLOCK_VALUES[kind]) * BLOCK_BYTES[kind]
            assert t.address % 32 == 0
            assert np.array_equal(g.array(t), blocks.reshape(-1))
        t = g.find("output_norm.weight")
        assert t.kind == 0 and t.dtype == capi.DT_F32 and t.shape == (512,) and np.array_equal(g.array(t), norm)
        e = g.find("blk.0.ffn_gate_exps.weight")
        assert e.shape == (256, 8, 3) and e.nbytes == 3 * 8 * 144  # the file's order is kept for rank 3
        with pytest.raises(capi.MarmotHipError):
            g.find("missing")
        # key/value metadata: every value kind the writer produces, typed readers, file order
        md = g.metadata()
        assert list(md)[:6] == ["general.architecture", "llama.block_count", "tokenizer.ggml.tokens",
                                "llama.rope.freq_base", "some.flag", "some.ints"]
        assert md["general.architecture"] == "llama" and md["llama.block_count"] == 1
        assert md["tokenizer.ggml.tokens"] == ["a", "bc"] and md["llama.rope.freq_base"] == 10000.0
        assert md["some.flag"] is True and md["some.ints"] == [1, 2, 3] and md["general.alignment"] == 32
        assert g.get("llama.block_count") == 1
        with pytest.raises(capi.MarmotHipError):
            g.get("llama.missing")
        import ctypes as C
        kv = capi.GgufKv()
        capi.check(g.lib.marmot_hip_gguf_find_kv(g.handle, b"tokenizer.ggml.tokens", C.byref(kv)))
        assert (kv.type, kv.elem_type, kv.count) == (9, 8, 2) and kv.nbytes == 8 + 1 + 8 + 2
        v, f = C.c_int64(), C.c_double()
        assert g.lib.marmot_hip_gguf_kv_int(C.byref(kv), 0, C.byref(v)) != 0       # a string is no integer
        p, n = C.c_char_p(), C.c_size_t()
        assert g.lib.marmot_hip_gguf_kv_string(C.byref(kv), 2, C.byref(p), C.byref(n)) != 0   # past the end
        capi.check(g.lib.marmot_hip_gguf_find_kv(g.handle, b"llama.rope.freq_base", C.byref(kv)))
        assert g.lib.marmot_hip_gguf_kv_int(C.byref(kv), 0, C.byref(v)) != 0       # a float is no integer
        capi.check(g.lib.marmot_hip_gguf_kv_float(C.byref(kv), 0, C.byref(f)))
        assert f.value == 10000.0 and g.lib.marmot_hip_gguf_kv_float(C.byref(kv), 1, C.byref(f)) != 0


def test_alignment_and_version(tmp_path):
    w = np.arange(64, dtype=np.float32).reshape(4, 16)
    b = np.arange(10, dtype=np.float16)
    p = write_gguf(str(tmp_path / "a.gguf"), [("w", "f32", (16, 4), w), ("b", "f16", (10,), b)], alignment=64)
    with GgufFile(p) as g:
        assert g.alignment == 64
        assert all(t.address % 64 == 0 for t in g.tensors)
        assert np.array_equal(g.array(g.find("w")), w) and g.find("w").shape == (4, 16)
        assert np.array_equal(g.array(g.find("b")), b)
    p = write_gguf(str(tmp_path / "v2.gguf"), [("w", "f32", (16, 4), w)], version=2, declare_alignment=False)
    with GgufFile(p) as g:
        assert g.alignment == 32 and np.array_equal(g.array(g.tensors[0]), w)


def test_malformed_files_are_rejected(tmp_path):
    w = np.zeros((4, 32), np.float32)
    good = write_gguf(str(tmp_path / "g.gguf"), [("w", "f32", (32, 4), w)])
    raw = open(good, "rb").read()

    def opens(data, name):
        p = str(tmp_path / name)
        open(p, "wb").write(data)
        try:
            GgufFile(p).close()
            return None
        except capi.MarmotHipError as e:
            return e.code

    assert opens(raw, "ok.gguf") is None
    assert opens(b"GGML" + raw[4:], "magic.gguf") == -1
    assert opens(raw[:4] + struct.pack("<I", 1) + raw[8:], "v1.gguf") == -8
    assert opens(raw[:40], "cut_header.gguf") == -1
    assert opens(raw[:-64], "cut_data.gguf") == -1           # tensor storage beyond the end of the file
    bad_type = write_gguf(str(tmp_path / "t.gguf"), [("w", "f32", (32, 4), w)])
    data = bytearray(open(bad_type, "rb").read())
    at = data.index(b"w" + struct.pack("<I", 2)) + 1 + 4 + 16   # name, rank, two dimensions -> the type field
    data[at:at + 4] = struct.pack("<I", 99)
    assert opens(bytes(data), "type.gguf") == -8
    # dimensions whose product wraps around 64 bits to the size of the stored payload (2^62 * 4 * 4 bytes = 2^66,
    # plus a row count chosen so that the wrapped byte count equals the real one) must not pass the size check
    at_dims = data.index(b"w" + struct.pack("<I", 2)) + 1 + 4
    for dims in ((1 << 62, 4), (32, (1 << 62) + 4), ((1 << 63) + 32, 2), (0xFFFFFFFFFFFFFFFF, 0xFFFFFFFFFFFFFFFF)):
        wrapped = bytearray(raw)
        wrapped[at_dims:at_dims + 16] = struct.pack("<QQ", *dims)
        assert opens(bytes(wrapped), "overflow.gguf") == -1, dims
    blocks = np.zeros((4, 144), np.uint8)
    q = bytearray(open(write_gguf(str(tmp_path / "q.gguf"), [("w", "q4_k", (256, 4), blocks)]), "rb").read())
    at_q = q.index(b"w" + struct.pack("<I", 2)) + 1 + 4
    for dims in ((0xFFFFFFFFFFFFFFFF, 4), (256, (1 << 64) // 144 + 4), ((1 << 63), 1 << 40)):
        wrapped = bytearray(q)
        wrapped[at_q:at_q + 16] = struct.pack("<QQ", *dims)
        assert opens(bytes(wrapped), "overflow_q.gguf") == -1, dims
    with pytest.raises(capi.MarmotHipError):
        GgufFile(str(tmp_path / "does_not_exist.gguf"))
    assert not os.path.exists(str(tmp_path / "does_not_exist.gguf"))


def test_synthetic_moe_file_of_the_reference_loader_test():
    """tests/golden/synthetic_qwen3moe.gguf follows write_synthetic_qwen3moe_gguf (the reference's
    tests/graph/test_gguf_loader.c:171-256) field by field: 16 key/value pairs, 17 FLOAT32 tensors whose offsets
    accumulate the sizes without per-tensor alignment, 32-byte alignment of the data section only. Expectations below
    are written down from that test, not from the generator."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "synthetic_qwen3moe.gguf")
    raw = open(path, "rb").read()
    # the committed bytes are what the committed generator writes
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_synthetic_gguf", os.path.join(os.path.dirname(path),
                                                                                      "make_synthetic_gguf.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert mod.build() == raw
    assert struct.unpack_from("<IIQQ", raw, 0) == (0x46554747, 3, 17, 16)
    expect_kv = [("general.architecture", "qwen3moe"), ("general.alignment", 32), ("qwen3moe.context_length", 32),
                 ("qwen3moe.embedding_length", 8), ("qwen3moe.block_count", 1), ("qwen3moe.attention.head_count", 2),
                 ("qwen3moe.attention.head_count_kv", 1), ("qwen3moe.feed_forward_length", 6),
                 ("qwen3moe.rope.dimension_count", 4), ("qwen3moe.attention.key_length", 4),
                 ("qwen3moe.attention.layer_norm_rms_epsilon", float(np.float32(1.0e-5))),
                 ("qwen3moe.rope.freq_base", 10000.0), ("qwen3moe.expert_count", 2), ("qwen3moe.expert_used_count", 1),
                 ("qwen3moe.expert_shared_count", 1), ("qwen3moe.expert_weights_scale", 1.25)]
    # name, dimensions as the file lists them (innermost first)
    expect_tensors = [("output_norm.weight", (8,)), ("output.weight", (8, 16)), ("blk.0.attn_norm.weight", (8,)),
                      ("blk.0.attn_q.weight", (8, 8)), ("blk.0.attn_k.weight", (8, 4)), ("blk.0.attn_v.weight", (8, 4)),
                      ("blk.0.attn_output.weight", (8, 8)), ("blk.0.attn_q_norm.weight", (4,)),
                      ("blk.0.attn_k_norm.weight", (4,)), ("blk.0.ffn_norm.weight", (8,)),
                      ("blk.0.ffn_gate_inp.weight", (8, 2)), ("blk.0.ffn_gate_exps.weight", (8, 6, 2)),
                      ("blk.0.ffn_up_exps.weight", (8, 6, 2)), ("blk.0.ffn_down_exps.weight", (6, 8, 2)),
                      ("blk.0.ffn_gate_shexp.weight", (8, 6)), ("blk.0.ffn_up_shexp.weight", (8, 6)),
                      ("blk.0.ffn_down_shexp.weight", (6, 8))]
    with GgufFile(path) as g:
        assert g.alignment == 32
        assert list(g.metadata().items()) == expect_kv  # file order, types resolved (uint32, float32, string)
        assert g.get("qwen3moe.expert_weights_scale") == 1.25 and g.get("general.architecture") == "qwen3moe"
        assert [t.name for t in g.tensors] == [n for n, _ in expect_tensors]
        data_start = None
        offset = 0
        for t, (info, (name, dims)) in enumerate(zip(g.tensors, expect_tensors)):
            n = int(np.prod(dims))
            assert info.ggml_type == 0 and info.kind == 0 and info.dtype == capi.DT_F32 and info.nbytes == 4 * n
            # matrices are [rows, cols] (the file's two dimensions reversed), vectors and expert stacks keep file order
            assert info.shape == (tuple(reversed(dims)) if len(dims) == 2 else dims), name
            data_start = info.address - offset if data_start is None else data_start
            assert info.address == data_start + offset, name  # offsets accumulate sizes: no per-tensor alignment
            offset += 4 * n
            want = np.float32(t) + np.arange(n, dtype=np.float32) / np.float32(1024.0)
            assert np.array_equal(g.array(info).ravel(), want), name
            assert g.find(name) == info
        # the norm weights of 16 bytes leave the tensors behind them 16 bytes off the 32-byte alignment
        assert (g.find("blk.0.attn_k_norm.weight").address - data_start) % 32 == 16
        assert data_start % 32 == g.tensors[0].address % 32
        # the data section starts at the first multiple of 32 behind the tensor infos and runs to the end of the file
        assert offset == 4 * sum(int(np.prod(d)) for _, d in expect_tensors) and len(raw) - offset == (len(raw) - offset) // 32 * 32
