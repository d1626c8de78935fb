"""Shared pieces of the parity tests: seeded inputs and closed-form patterns
the reference's own tests use."""

from __future__ import annotations

import numpy as np


def kernel_test_pattern(total: int) -> np.ndarray:
    """byte i = (i*31+7) & 0xFF (transfer/kernel.rs:221 of the reference)."""
    i = np.arange(total, dtype=np.uint64)
    return ((i * 31 + 7) & 0xFF).astype(np.uint8)


def block_fill_pattern(num_blocks: int, block_bytes: int) -> np.ndarray:
    """block i filled with byte (i % 251) + 1 (tests/common/helpers.rs:79-89)."""
    fills = ((np.arange(num_blocks) % 251) + 1).astype(np.uint8)
    return np.repeat(fills, block_bytes)


def split_fill_pattern(num_blocks: int, segment: int, kv_stride: int) -> np.ndarray:
    """K and V regions both carry the block fill (tests/common/harness.rs:53-80)."""
    size = (num_blocks - 1) * segment + kv_stride + segment
    out = np.zeros(size, dtype=np.uint8)
    fills = ((np.arange(num_blocks) % 251) + 1).astype(np.uint8)
    out[: num_blocks * segment] = np.repeat(fills, segment)
    out[kv_stride: kv_stride + num_blocks * segment] = np.repeat(fills, segment)
    return out


def xorshift_shuffle(n: int, seed: int = 0x9E3779B97F4A7C15) -> list[int]:
    """Deterministic permutation of the reference's transfer bench
    (benches/transfer_h2d.rs:301-315): xorshift64 Fisher-Yates."""
    mask = (1 << 64) - 1
    state = seed

    def nxt():
        nonlocal state
        state ^= (state << 13) & mask
        state ^= state >> 7
        state ^= (state << 17) & mask
        return state

    perm = list(range(n))
    for i in range(n - 1, 0, -1):
        j = nxt() % (i + 1)
        perm[i], perm[j] = perm[j], perm[i]
    return perm


def random_bytes(rng: np.random.Generator, n: int) -> np.ndarray:
    return rng.integers(0, 256, size=n, dtype=np.uint8)


def bf16_normal_bytes(rng: np.random.Generator, n_elems: int) -> np.ndarray:
    """N(0,1) samples truncated to bf16, as raw bytes (2 per element)."""
    f = rng.standard_normal(n_elems, dtype=np.float32)
    hi = (f.view(np.uint32) >> 16).astype(np.uint16)
    return hi.view(np.uint8)


def fp8_e4m3_bytes(rng: np.random.Generator, n: int) -> np.ndarray:
    """Random bytes with the e4m3fn NaN encodings (0x7F, 0xFF) remapped."""
    b = rng.integers(0, 256, size=n, dtype=np.uint8)
    b[b == 0x7F] = 0x7E
    b[b == 0xFF] = 0xFE
    return b
