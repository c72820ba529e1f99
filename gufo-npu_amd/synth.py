"""Seeded synthetic K-quant weights and activations.

One generator feeds the GPU path, the CPU checker and the bench, so all of them see
identical bytes.  Distributions:

* Q4_K block (144 B): d, dmin = fp16(|N(0, 0.02)|); eight 6-bit scales and eight
  6-bit mins uniform on 0..63; 256 quants uniform on 0..15.  The 12 scale bytes and
  the 128 quant bytes are bijections of those values, so this is exactly "two fp16
  values followed by 140 uniform random bytes" - how the reference's own test
  builds rows (tests/models/qwen35/gguf_dot_test.cpp:61-70).
* Q5_K block (176 B): the same plus 32 uniform high-bit bytes.
* Q6_K block (210 B): 128 + 64 uniform quant bytes, 16 int8 scales uniform over all
  byte values, d = fp16(|N(0, 0.02)|) at byte 208.
* activations: fp32 N(0, 1); router logits: fp32 N(0, 1).

numpy's Philox bit generator is counter based and gives the same stream on every
platform for a given seed.
"""
from __future__ import annotations

import numpy as np

F32, Q8_0, Q4_K, Q5_K, Q6_K = 0, 8, 12, 13, 14
BLOCK_BYTES = {Q4_K: 144, Q5_K: 176, Q6_K: 210}
TYPE_NAMES = {F32: "F32", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K"}
SUPER_BLOCK = 256
# The reference's own test seed (tests/models/qwen35/gguf_dot_test.cpp:91).
BASE_SEED = 20261105


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(seed))


def row_bytes(ggml_type: int, cols: int) -> int:
    if cols % SUPER_BLOCK != 0:
        raise ValueError("row is not a whole number of blocks")
    return cols // SUPER_BLOCK * BLOCK_BYTES[ggml_type]


def _half_scales(gen: np.random.Generator, n: int) -> np.ndarray:
    """n fp16 values |N(0, 0.02)| as their two little-endian bytes."""
    values = np.abs(gen.standard_normal(n, dtype=np.float32) * np.float32(0.02))
    return values.astype(np.float16).view(np.uint8).reshape(n, 2)


def kquant_matrix(ggml_type: int, rows: int, cols: int, seed: int) -> np.ndarray:
    """rows x row_bytes uint8: a row-major matrix of GGUF blocks, as a file stores it."""
    block = BLOCK_BYTES[ggml_type]
    n_blocks = rows * (cols // SUPER_BLOCK)
    if cols % SUPER_BLOCK != 0:
        raise ValueError("row is not a whole number of blocks")
    gen = rng(seed)
    data = gen.integers(0, 256, size=(n_blocks, block), dtype=np.uint8)
    if ggml_type in (Q4_K, Q5_K):
        data[:, 0:2] = _half_scales(gen, n_blocks)
        data[:, 2:4] = _half_scales(gen, n_blocks)
    else:
        data[:, 208:210] = _half_scales(gen, n_blocks)
    return data.reshape(rows, -1)


def q8_0_matrix(rows: int, cols: int, seed: int) -> np.ndarray:
    """rows x (cols/32*34) uint8 of Q8_0 blocks: d = fp16(|N(0, 0.02)|), 32 uniform int8
    (how the reference's own test builds such rows, tests/models/qwen35/gguf_dot_test.cpp:61-70)."""
    if cols % 32 != 0:
        raise ValueError("row is not a whole number of blocks")
    n_blocks = rows * (cols // 32)
    gen = rng(seed)
    data = gen.integers(0, 256, size=(n_blocks, 34), dtype=np.uint8)
    data[:, 0:2] = _half_scales(gen, n_blocks)
    return data.reshape(rows, -1)


def f32_matrix(rows: int, cols: int, seed: int) -> np.ndarray:
    """rows x (cols*4) uint8: fp32 N(0, 0.05) weights as a file stores them."""
    w = rng(seed).standard_normal((rows, cols), dtype=np.float32) * np.float32(0.05)
    return np.ascontiguousarray(w).view(np.uint8).reshape(rows, cols * 4)


def matrix(ggml_type: int, rows: int, cols: int, seed: int) -> np.ndarray:
    """A synthetic matrix of any row type the backend takes."""
    if ggml_type == F32:
        return f32_matrix(rows, cols, seed)
    if ggml_type == Q8_0:
        return q8_0_matrix(rows, cols, seed)
    return kquant_matrix(ggml_type, rows, cols, seed)


def activations(tokens: int, cols: int, seed: int) -> np.ndarray:
    return rng(seed).standard_normal((tokens, cols), dtype=np.float32)


def router_logits(tokens: int, experts: int, seed: int) -> np.ndarray:
    return rng(seed).standard_normal((tokens, experts), dtype=np.float32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bits (round to nearest even) as uint16."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def bf16_to_float(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def pack_scales_k4(scales: np.ndarray, mins: np.ndarray) -> np.ndarray:
    """The 12 packed bytes for eight 6-bit scales and mins (the packer that
    quant::ScaleMinK4, src/core/quant.cpp:158-167 of the reference, undoes)."""
    sc = np.asarray(scales, dtype=np.uint8)
    m = np.asarray(mins, dtype=np.uint8)
    out = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        out[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        out[j + 4] = (m[j] & 63) | ((m[j + 4] >> 4) << 6)
        out[j + 8] = (sc[j + 4] & 15) | ((m[j + 4] & 15) << 4)
    return out
