"""Shared helpers of the test-suite: seeded input builders for the benchmark
configurations and small utilities.  CPU tensors only; GPU tests move them."""
from __future__ import annotations

import json
import os
from typing import List, Tuple

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# Parity gates: max-abs error of the attention output against the fp32 oracle
# evaluated on the same rounded inputs.
TOL = {torch.float16: 5e-3, torch.bfloat16: 2e-2}


def load_kat():
    with open(os.path.join(GOLDEN, "flash_attn_varlen_kat.json")) as f:
        return json.load(f)


def kat_inputs():
    """q, k, v as the reference test builds them: [total=2, heads=3, d=8] bf16 views."""
    base = torch.arange(48, dtype=torch.bfloat16).reshape(3, 2, 8)
    k = base / 40.0
    v = base / 50.0
    q = base / 30.0
    return q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)


def round4(t: torch.Tensor) -> torch.Tensor:
    """f32::round(x * 10^4) / 10^4 in f32, as the reference test does (round half away from zero)."""
    b = torch.tensor(10.0 ** 4, dtype=torch.float32)
    x = t.float() * b
    r = torch.where(x >= 0, torch.floor(x + 0.5), torch.ceil(x - 0.5))
    return r / b


def make_cache(num_blocks: int, num_kv_heads: int, head_size: int, block_size: int, dtype: torch.dtype,
               fill=None, gen=None) -> Tuple[torch.Tensor, torch.Tensor]:
    x = 16 // torch.tensor([], dtype=dtype).element_size()
    kshape = (num_blocks, num_kv_heads, head_size // x, block_size, x)
    vshape = (num_blocks, num_kv_heads, head_size, block_size)
    if fill is not None:
        return torch.full(kshape, fill, dtype=dtype), torch.full(vshape, fill, dtype=dtype)
    return (torch.randn(kshape, generator=gen, dtype=torch.float32).to(dtype),
            torch.randn(vshape, generator=gen, dtype=torch.float32).to(dtype))


def slots_for(blocks: List[int], length: int, block_size: int) -> List[int]:
    return [blocks[t // block_size] * block_size + t % block_size for t in range(length)]


def cu(lens) -> torch.Tensor:
    out = [0]
    for l in lens:
        out.append(out[-1] + int(l))
    return torch.tensor(out, dtype=torch.int32)


def decode_case(seed: int, S: int, ctx_lo: int, ctx_hi: int, Hq: int, Hkv: int, d: int, dtype: torch.dtype,
                pool_blocks: int, block_size: int = 16):
    """Paged-decode inputs in the shape of the benchmark's decode configuration: contexts
    uniform in [ctx_lo, ctx_hi], block tables = consecutive slices of a permutation of the pool."""
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    ctx = rng.integers(ctx_lo, ctx_hi + 1, size=S).astype(np.int32)
    nblk = (ctx + block_size - 1) // block_size
    assert int(nblk.sum()) <= pool_blocks
    perm = torch.randperm(pool_blocks, generator=g).numpy()
    width = int(nblk.max())
    tables = np.zeros((S, width), dtype=np.int32)
    pos = 0
    for s in range(S):
        tables[s, :nblk[s]] = perm[pos:pos + nblk[s]]
        pos += nblk[s]
    kc, vc = make_cache(pool_blocks, Hkv, d, block_size, dtype, gen=g)
    q = torch.randn((S, Hq, d), generator=g, dtype=torch.float32).to(dtype)
    return dict(q=q, key_cache=kc, value_cache=vc, block_tables=torch.from_numpy(tables),
                context_lens=torch.from_numpy(ctx), max_ctx=int(ctx.max()), scale=1.0 / float(np.sqrt(d)))
