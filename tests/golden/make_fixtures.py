#!/usr/bin/env python3
"""Regenerates the committed fixtures under tests/golden/ (data only).

Needs the reference checkout (default /root/reference) and, for the second file, the
reference-built leaf library (``make -C oracle ref``). Neither is needed to *use* the fixtures.

  reference_goldens.npz   the golden vectors the reference's own tests hold for this path
                          (quantizer bytes, dequantized values, block dots, whole matmuls),
                          transcribed by compiling dump_reference_goldens.c against the
                          reference's headers.
  ref_gaussian.npz        outputs of the reference's own quantize / dequantize / pack / block-dot
                          code (scalar build) on seeded Gaussian rows: what the reference's
                          golden vectors leave open for N(0, 0.02) weights and N(0, 1) activations.
"""
import io
import os
import struct
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = os.environ.get("MARMOT_REFERENCE", "/root/reference")
CLANG = os.environ.get("REFCC", "/opt/rocm/llvm/bin/clang")


def dump_reference_goldens():
    with tempfile.TemporaryDirectory() as td:
        exe = os.path.join(td, "dump")
        subprocess.check_call([
            CLANG, "-std=c2x", "-O0", "-w", f"-I{REF}/include", f"-I{REF}/tests", f"-I{REF}/src",
            os.path.join(HERE, "dump_reference_goldens.c"), "-o", exe,
        ])
        raw = subprocess.check_output([exe])
    arrays = {}
    f = io.BytesIO(raw)
    while True:
        hdr = f.read(4)
        if not hdr:
            break
        (nl,) = struct.unpack("<I", hdr)
        name = f.read(nl).decode()
        (dl,) = struct.unpack("<I", f.read(4))
        dtype = f.read(dl).decode()
        (nb,) = struct.unpack("<Q", f.read(8))
        arrays[name] = np.frombuffer(f.read(nb), dtype=np.dtype("<" + dtype)).copy()
    np.savez_compressed(os.path.join(HERE, "reference_goldens.npz"), **arrays)
    print("reference_goldens.npz:", len(arrays), "arrays")


def dump_ref_gaussian():
    sys.path.insert(0, ROOT)
    from oracle.pyoracle import (BLOCK_VALUES, KIND_Q2_K, KIND_Q3_K, KIND_Q4_0, KIND_Q4_1, KIND_Q4_K, KIND_Q5_0,
                                 KIND_Q5_1, KIND_Q5_K, KIND_Q6_K, KIND_Q8_0, KIND_Q8_1, KIND_Q8_K, RefLib)

    ref = RefLib()
    out = {}
    K = 1024
    for name, kind, seed in (("q8_0", KIND_Q8_0, 100), ("q4_0", KIND_Q4_0, 101), ("q4_k", KIND_Q4_K, 102),
                             ("q6_k", KIND_Q6_K, 103), ("q5_k", KIND_Q5_K, 105),
                             ("q4_1", KIND_Q4_1, 106), ("q5_0", KIND_Q5_0, 107), ("q5_1", KIND_Q5_1, 108),
                             ("q2_k", KIND_Q2_K, 109), ("q3_k", KIND_Q3_K, 110), ("q8_1", KIND_Q8_1, 111)):
        rng = np.random.default_rng(seed)
        rows = 16  # 16 rows x 1024 -> 64 K-quant super-blocks (512 legacy blocks) per format
        w = (rng.standard_normal((rows, K), dtype=np.float32) * np.float32(0.02)).astype(np.float32)
        # a few adversarial rows: all-zero, one spike, constant, tiny magnitudes
        w[0, :256] = 0.0
        w[1, :256] = 0.0
        w[1, 17] = 0.5
        w[2, :256] = 0.0123
        w[3, :256] *= np.float32(1e-6)
        x = rng.standard_normal(K, dtype=np.float32)
        blocks = ref.quantize(kind, w)
        deq = ref.dequantize(kind, blocks, K)
        act_kind = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
        act = ref.pack(act_kind, x)
        act16 = ref.pack(act_kind, x.astype(np.float16))
        nb = K // BLOCK_VALUES[kind]
        dots = np.array([ref.vec_dot(kind, blocks[r], act, nb) for r in range(rows)], dtype=np.float32)
        dots16 = np.array([ref.vec_dot_f16(kind, blocks[r], x.astype(np.float16), K) for r in range(rows)],
                          dtype=np.float32)
        out[f"{name}_w"] = w
        out[f"{name}_x"] = x
        out[f"{name}_blocks"] = blocks
        out[f"{name}_dequant"] = deq
        out[f"{name}_act"] = act
        out[f"{name}_act_from_f16"] = act16
        out[f"{name}_dots"] = dots
        out[f"{name}_dots_f16"] = dots16
    # ragged tail: K not a multiple of the block
    rng = np.random.default_rng(104)
    for name, kind, k in (("q8_0", KIND_Q8_0, 70), ("q4_0", KIND_Q4_0, 70), ("q4_k", KIND_Q4_K, 300),
                          ("q6_k", KIND_Q6_K, 300), ("q5_k", KIND_Q5_K, 300),
                          ("q4_1", KIND_Q4_1, 70), ("q5_0", KIND_Q5_0, 70), ("q5_1", KIND_Q5_1, 70),
                          ("q2_k", KIND_Q2_K, 300), ("q3_k", KIND_Q3_K, 300), ("q8_1", KIND_Q8_1, 70)):
        w = (rng.standard_normal((2, k), dtype=np.float32) * np.float32(0.02)).astype(np.float32)
        blocks = ref.quantize(kind, w)
        out[f"{name}_tail_w"] = w
        out[f"{name}_tail_blocks"] = blocks
        out[f"{name}_tail_dequant"] = ref.dequantize(kind, blocks, k)
        x = rng.standard_normal(k, dtype=np.float32)
        act_kind = KIND_Q8_K if BLOCK_VALUES[kind] == 256 else KIND_Q8_0
        out[f"{name}_tail_x"] = x
        out[f"{name}_tail_act"] = ref.pack(act_kind, x)
    np.savez_compressed(os.path.join(HERE, "ref_gaussian.npz"), **out)
    print("ref_gaussian.npz:", len(out), "arrays")


if __name__ == "__main__":
    dump_reference_goldens()
    dump_ref_gaussian()
