"""The AICI logit-mask step on the CPU.  TEST INFRASTRUCTURE (see
oracle/__init__.py): never imported by the product.
"""
from __future__ import annotations

import numpy as np
import torch


def mask_bytes_for(vocab_size: int) -> int:
    """aicirt/src/api.rs:216-221 `BiasType::Bool.size_in_bytes`: 4 * ceil(vocab/32)."""
    return 4 * ((vocab_size + 31) // 32)


def pack_allowed(allowed: np.ndarray) -> np.ndarray:
    """allowed: bool [V] -> u8 [4*ceil(V/32)], bit k of byte i (LSB first) <-> token 8i+k
    (aicirt/src/api.rs:278-292 read backwards)."""
    V = allowed.shape[0]
    out = np.zeros((mask_bytes_for(V),), dtype=np.uint8)
    idx = np.nonzero(allowed)[0]
    np.bitwise_or.at(out, idx >> 3, (1 << (idx & 7)).astype(np.uint8))
    return out


def apply_to_slice(src: np.ndarray, row_len: int) -> np.ndarray:
    """aicirt/src/api.rs:278-292 `apply_to_slice` for BiasType::F32: bit set -> 0.0,
    clear -> -inf, everything past 8*len(src) -> -inf."""
    dst = np.full((row_len,), -np.inf, dtype=np.float32)
    dp = 0
    for sb in src.tolist():
        for bit in range(8):
            dst[dp] = 0.0 if (sb >> bit) & 1 else -np.inf
            dp += 1
    return dst


def apply_to_slice_fast(src: np.ndarray, row_len: int) -> np.ndarray:
    """Vectorised `apply_to_slice` (checked against it in the tests)."""
    bits = np.unpackbits(src, bitorder="little")
    dst = np.full((row_len,), -np.inf, dtype=np.float32)
    n = min(row_len, bits.shape[0])
    dst[:n] = np.where(bits[:n] != 0, np.float32(0.0), np.float32(-np.inf))
    return dst


def bias_row_len(vocab_size: int) -> int:
    """aicirt/src/main.rs:1303-1309: rows are (vocab + 1000) & !63 floats long."""
    return (vocab_size + 1000) & ~63


def biased_argmax(logits: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """tmodel.rs:277-283 + 234-236: logits_row + bias_row[0..V] (promotes to f32), argmax."""
    V = logits.shape[1]
    return (logits.float() + bias[:, :V]).argmax(dim=1)
