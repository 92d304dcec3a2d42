"""Seeded synthetic inputs in the shapes of the benchmark configurations.

Everything is generated on the CPU from `torch.Generator().manual_seed(seed)` /
`numpy.random.default_rng(seed)` so that the CPU oracle and the GPU kernels see
identical bits, except `decode_inputs(..., device=...)`, which can fill the
(large) KV cache directly on the GPU for throughput runs.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

BLOCK_SIZE = 16


def cache_shapes(num_blocks: int, num_kv_heads: int, head_size: int, block_size: int, dtype: torch.dtype):
    x = 16 // torch.empty((), dtype=dtype).element_size()
    return ((num_blocks, num_kv_heads, head_size // x, block_size, x),
            (num_blocks, num_kv_heads, head_size, block_size))


def offsets(lens: Sequence[int]) -> torch.Tensor:
    out = [0]
    for l in lens:
        out.append(out[-1] + int(l))
    return torch.tensor(out, dtype=torch.int32)


def slots_for(blocks: Sequence[int], length: int, block_size: int = BLOCK_SIZE) -> List[int]:
    return [int(blocks[t // block_size]) * block_size + t % block_size for t in range(length)]


@dataclass
class DecodeInputs:
    q: torch.Tensor             # [S, Hq, d]
    key_cache: torch.Tensor     # [nb, Hkv, d/8, 16, 8]
    value_cache: torch.Tensor   # [nb, Hkv, d, 16]
    block_tables: torch.Tensor  # int32 [S, max_blocks]
    context_lens: torch.Tensor  # int32 [S]
    max_ctx: int
    scale: float
    num_kv_heads: int

    def algorithmic_bytes(self) -> int:
        """K and V read once per kv head, q in, out written, tables and lengths read."""
        S, Hq, d = self.q.shape
        elt = self.q.element_size()
        ctx = self.context_lens.cpu().numpy().astype(np.int64)
        kv = int(ctx.sum()) * 2 * self.num_kv_heads * d * elt
        qo = 2 * S * Hq * d * elt
        tbl = 4 * int(((ctx + BLOCK_SIZE - 1) // BLOCK_SIZE).sum()) + 4 * S
        return kv + qo + tbl

    def to(self, device) -> "DecodeInputs":
        return DecodeInputs(self.q.to(device), self.key_cache.to(device), self.value_cache.to(device),
                            self.block_tables.to(device), self.context_lens.to(device), self.max_ctx, self.scale,
                            self.num_kv_heads)


def decode_inputs(seed: int, S: int, ctx_lo: int, ctx_hi: int, Hq: int, Hkv: int, d: int, dtype: torch.dtype,
                  pool_blocks: int, device=None, block_size: int = BLOCK_SIZE) -> DecodeInputs:
    """One query token per sequence; contexts uniform in [ctx_lo, ctx_hi]; block tables are
    consecutive slices of a seeded permutation of the pool (no block reused); K/V/Q ~ N(0,1).
    With `device`, the cache is filled there (seeded) instead of on the CPU."""
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    ctx = rng.integers(ctx_lo, ctx_hi + 1, size=S).astype(np.int32)
    nblk = (ctx.astype(np.int64) + block_size - 1) // block_size
    assert int(nblk.sum()) <= pool_blocks, "block pool too small for the drawn contexts"
    perm = torch.randperm(pool_blocks, generator=g).numpy()
    width = int(nblk.max())
    tables = np.zeros((S, width), dtype=np.int32)
    pos = 0
    for s in range(S):
        tables[s, :nblk[s]] = perm[pos:pos + nblk[s]]
        pos += int(nblk[s])
    kshape, vshape = cache_shapes(pool_blocks, Hkv, d, block_size, dtype)
    if device is None:
        kc = torch.randn(kshape, generator=g, dtype=torch.float32).to(dtype)
        vc = torch.randn(vshape, generator=g, dtype=torch.float32).to(dtype)
    else:
        gd = torch.Generator(device=device).manual_seed(seed)
        kc = torch.randn(kshape, generator=gd, dtype=dtype, device=device)
        vc = torch.randn(vshape, generator=gd, dtype=dtype, device=device)
    q = torch.randn((S, Hq, d), generator=g, dtype=torch.float32).to(dtype)
    out = DecodeInputs(q, kc, vc, torch.from_numpy(tables), torch.from_numpy(ctx), int(ctx.max()),
                       1.0 / math.sqrt(d), Hkv)
    return out.to(device) if device is not None else out


def config2(device=None, S: int = 64, pool_blocks: int = 20000) -> DecodeInputs:
    """Paged decode: 64 sequences, contexts U[512,4096], 32 q / 8 kv heads, d 128, bf16,
    tables from a shuffled 20k-block pool (seed 2)."""
    return decode_inputs(2, S, 512, 4096, 32, 8, 128, torch.bfloat16, pool_blocks, device)


@dataclass
class PrefillInputs:
    q: torch.Tensor          # [T, Hq, d]
    k: torch.Tensor          # [T, Hkv, d]
    v: torch.Tensor
    cu_q: torch.Tensor       # int32 [b+1]
    cu_k: torch.Tensor
    max_q: int
    max_k: int
    scale: float
    lens_q: List[int]
    lens_k: List[int]

    def flops(self) -> float:
        """4*d*Hq * sum over sequences of the unmasked (query, key) pairs."""
        d, Hq = self.q.shape[2], self.q.shape[1]
        pairs = sum(lq * (lk - lq) + lq * (lq + 1) // 2 for lq, lk in zip(self.lens_q, self.lens_k))
        return 4.0 * d * Hq * pairs

    def to(self, device) -> "PrefillInputs":
        return PrefillInputs(self.q.to(device), self.k.to(device), self.v.to(device), self.cu_q.to(device),
                             self.cu_k.to(device), self.max_q, self.max_k, self.scale, self.lens_q, self.lens_k)


def prefill_inputs(seed: int, lens: Sequence[int], Hq: int, Hkv: int, d: int, dtype: torch.dtype, sigma: float = 1.0,
                   device=None) -> PrefillInputs:
    """Self-attention prefill (Lq = Lk per sequence); Q/K/V ~ N(0, sigma^2) rounded to dtype."""
    lens = [int(l) for l in lens]
    T = sum(lens)
    if device is None:
        g = torch.Generator().manual_seed(seed)
        q, k, v = (torch.randn((T, h, d), generator=g, dtype=torch.float32).mul_(sigma).to(dtype)
                   for h in (Hq, Hkv, Hkv))
    else:
        gd = torch.Generator(device=device).manual_seed(seed)
        q, k, v = (torch.randn((T, h, d), generator=gd, dtype=torch.float32, device=device).mul_(sigma).to(dtype)
                   for h in (Hq, Hkv, Hkv))
    c = offsets(lens)
    if device is not None:
        c = c.to(device)
    return PrefillInputs(q, k, v, c, c.clone(), max(lens), max(lens), 1.0 / math.sqrt(d), lens, list(lens))


def config1() -> Tuple[PrefillInputs, Dict[str, torch.Tensor]]:
    """4 sequences of 128/256/384/512 tokens, 32 = 32 heads, d 128, fp16 on the GPU (seed 0);
    blocks handed out from a random permutation of a 128-block pool."""
    p = prefill_inputs(0, [128, 256, 384, 512], 32, 32, 128, torch.float16)
    g = torch.Generator().manual_seed(0)
    perm = torch.randperm(128, generator=g).tolist()
    slots, pos = [], 0
    for L in p.lens_q:
        n = (L + BLOCK_SIZE - 1) // BLOCK_SIZE
        slots += slots_for(perm[pos:pos + n], L)
        pos += n
    return p, {"slot_mapping": torch.tensor(slots, dtype=torch.int32), "pool_blocks": 128}


def config3(sigma: float = 1.0, device=None, batch: int = 8, L: int = 4096) -> PrefillInputs:
    """Long GQA prefill, Llama-3-8B attention shape: 8 x 4096 tokens, 32 q / 8 kv heads, d 128, bf16 (seed 3)."""
    return prefill_inputs(3, [L] * batch, 32, 8, 128, torch.bfloat16, sigma, device)


def allow_mask(seed: int, S: int, vocab: int, frac: float = 0.05) -> np.ndarray:
    """Per sequence a seeded random `frac` of the vocabulary allowed; bool [S, vocab]."""
    rng = np.random.default_rng(seed)
    return rng.random((S, vocab)) < frac
