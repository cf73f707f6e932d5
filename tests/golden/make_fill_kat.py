"""Writes fill_random_kat.json: known answers for the reference's input generators.

The values are derived here from the published formula alone
(quantization/GEMM_fp32.cu:13-16, GEMM_bf16.cu:14-18, GEMM_fp16.cu:14-18,
GEMM_int8.cu:14-18) with Python integers and numpy scalar float32 arithmetic, i.e. by a
second implementation that shares no code with oracle/oracle.c.  Nothing from the
reference is imported or executed.

    python tests/golden/make_fill_kat.py
"""
import json
import os

import numpy as np

MASK = (1 << 64) - 1


def hash64(idx, seed):
    return ((idx ^ seed) * 2862933555777941757 + 3037000493) & MASK


def as_f32(idx, seed, lo=-1.0, hi=1.0):
    r = np.float32((hash64(idx, seed) >> 11) & 0xFFFFFF) / np.float32(16777215.0)
    return np.float32(lo) + r * (np.float32(hi) - np.float32(lo))


def bf16_bits(f):
    u = int(np.float32(f).view(np.uint32))
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF


def f16_bits(f):
    return int(np.float32(f).astype(np.float16).view(np.uint16))


def as_i8(idx, seed, lo=-127, hi=127):
    r = (hash64(idx, seed) >> 11) & 0xFFFF
    return lo + r % (hi - lo + 1)


LAST = (1 << 24) - 1  # last element of a 4096 x 4096 operand
IDX = [0, 1, 2, 3, 4, 5, 6, 7, 255, 256, 4095, 4096, 65535, 65536, 1000003, LAST]

kat = {
    "comment": "idx -> value for the seeds the reference uses; floats as uint32/uint16 bit patterns",
    "idx": IDX,
    "hash64": {hex(s): [hex(hash64(i, s)) for i in IDX] for s in (0x1234, 0x4234)},
    "f32": {hex(s): [int(as_f32(i, s).view(np.uint32)) for i in IDX] for s in (0x3234, 0x7776)},
    "bf16": {hex(s): [bf16_bits(as_f32(i, s)) for i in IDX] for s in (0x1234, 0x9876)},
    "f16": {hex(s): [f16_bits(as_f32(i, s)) for i in IDX] for s in (0x2234, 0x8876)},
    "i8": {hex(s): [as_i8(i, s) for i in IDX] for s in (0x4234, 0x6676)},
}
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fill_random_kat.json")
with open(path, "w") as f:
    json.dump(kat, f, indent=1)
print("wrote", path)
