#!/usr/bin/env python3
"""Writes the golden fixtures in this directory.  Nothing here imports the oracle or the product: the expected values
come from Python integers and from numpy / torch library routines, so they pin the oracle independently.

    python tests/golden/make_golden.py

pcg3d_vectors.json  the integer hash of gemm/gemm_test.cu:34-53 evaluated with Python big integers
gemm_small.npz      48x40x80 fp16 and bf16 operands (raw bits) in all four A/B storage layouts and C = A B in fp64
                    from numpy.matmul on the numpy/torch-widened values
random_style_vectors.json
                    elements of the reference's sparse random style (gemm/gemm_test.cu:73-91) worked out by hand from
                    the Python-integer hash: zeros, fourth powers (numpy float32 arithmetic in the reference's order of
                    operations) and every 1-in-100000 spike of 1000 among the first 1024 x 1024 coordinates, with the
                    fp16 / bf16 bit patterns from numpy / torch casts
"""
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
MASK = (1 << 32) - 1


def pcg3d_xyz(x: int, y: int, z: int):
    """Jarzynski & Olano's pcg3d on unbounded Python ints, wrapped to 32 bits after every operation."""
    v = [x & MASK, y & MASK, z & MASK]
    v = [(e * 1664525 + 1013904223) & MASK for e in v]
    for _ in range(2):
        v[0] = (v[0] + v[1] * v[2]) & MASK
        v[1] = (v[1] + v[2] * v[0]) & MASK
        v[2] = (v[2] + v[0] * v[1]) & MASK
        if _ == 0:
            v = [e ^ (e >> 16) for e in v]
    return v


def pcg3d_python(x: int, y: int, z: int) -> int:
    """The three outputs packed the way the reference packs them (gemm/gemm_test.cu:52): x in bits 0..31, y shifted up
    by 12, z shifted up by 24, combined with xor."""
    v = pcg3d_xyz(x, y, z)
    return v[0] ^ (v[1] << 12) ^ (v[2] << 24)


def main():
    vecs = []
    rng = np.random.default_rng(20250101)
    pts = [(0, 0, 0), (1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 2, 3), (8191, 8191, 20010106), (65535, 0, 19980724),
           (MASK, MASK, MASK), (123456789, 987654321, 0x9E3779B9)]
    pts += [tuple(int(v) for v in rng.integers(0, 1 << 32, 3)) for _ in range(23)]
    for x, y, z in pts:
        vecs.append({"x": x, "y": y, "z": z, "h": pcg3d_python(x, y, z)})
    with open(os.path.join(HERE, "pcg3d_vectors.json"), "w") as f:
        json.dump(vecs, f, indent=0)

    M, N, K = 48, 40, 80
    out = {}
    for name in ("f16", "bf16"):
        a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        if name == "f16":
            a16, b16 = a.astype(np.float16), b.astype(np.float16)
            a_bits, b_bits = a16.view(np.uint16), b16.view(np.uint16)
            aw, bw = a16.astype(np.float64), b16.astype(np.float64)
        else:
            ta, tb = torch.from_numpy(a).to(torch.bfloat16), torch.from_numpy(b).to(torch.bfloat16)
            a_bits = ta.view(torch.int16).numpy().view(np.uint16)
            b_bits = tb.view(torch.int16).numpy().view(np.uint16)
            aw, bw = ta.to(torch.float64).numpy(), tb.to(torch.float64).numpy()
        out[f"{name}_a_rowmajor"] = np.ascontiguousarray(a_bits)          # M x K
        out[f"{name}_a_colmajor"] = np.ascontiguousarray(a_bits.T)        # stored K x M
        out[f"{name}_b_rowmajor"] = np.ascontiguousarray(b_bits)          # K x N
        out[f"{name}_b_colmajor"] = np.ascontiguousarray(b_bits.T)        # stored N x K
        out[f"{name}_c_f64"] = aw @ bw
        out[f"{name}_abs_c_f64"] = np.abs(aw) @ np.abs(bw)
    np.savez_compressed(os.path.join(HERE, "gemm_small.npz"), **out)

    # gemm/gemm_test.cu:76-89: randbits = pcg3d(x, y, 20010106); 1000 if randbits % 100000 == 0; else 0 unless
    # randbits % 4 == 0; else v = (pcg3d(x, y, 19980724) % 1000000) * 1e-6f in fp32, value (v * v) * (v * v)
    def random_style(x, y):
        randbits = pcg3d_python(x, y, 20010106)
        if randbits % 100000 == 0:
            return "spike", np.float32(1000.0)
        if randbits % 4 != 0:
            return "zero", np.float32(0.0)
        v = np.float32(pcg3d_python(x, y, 19980724) % 1000000) * np.float32(1e-6)
        return "fourth_power", (v * v) * (v * v)

    picked, seen = [], {"spike": 0, "zero": 0, "fourth_power": 0}
    for y in range(1024):
        for x in range(1024):
            kind, val = random_style(x, y)
            want = 64 if kind == "spike" else 12
            if seen[kind] < want and (kind == "spike" or (x * 7 + y * 13) % 97 == 0):
                seen[kind] += 1
                f16 = int(np.float32(val).astype(np.float16).view(np.uint16))
                bf16 = int(torch.tensor(float(val), dtype=torch.float32).to(torch.bfloat16).view(torch.int16).item()) & 0xFFFF
                picked.append({"x": x, "y": y, "kind": kind, "f32_bits": int(np.float32(val).view(np.uint32)),
                               "f16_bits": f16, "bf16_bits": bf16})
    assert seen["spike"] >= 4 and seen["zero"] == 12 and seen["fourth_power"] == 12, seen
    with open(os.path.join(HERE, "random_style_vectors.json"), "w") as f:
        json.dump(picked, f, indent=0)


if __name__ == "__main__":
    main()
