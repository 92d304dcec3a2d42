"""One layer's attention as rLLM composes it (llm/mod.rs:318-354), driven by the C++ batch
builder: a mixed continuous-batching step with prefill chunks that have prior context in the
paged cache plus single-token decode rows, against the oracle pipeline that rLLM's CPU build
runs (scatter -> gather -> repeat_kv -> varlen SDPA for every row)."""
import math

import numpy as np
import pytest
import torch

from aici_amd import attn, paged
from aici_amd import workloads as W
from oracle import refkernels as ref
from tests.common import TOL, make_cache

pytestmark = pytest.mark.gpu


def mixed_step(seed, chunk_priors, chunk_len, n_decode, ctx_lo, ctx_hi, Hq, Hkv, d, dtype, pool, fused_qkv, device,
               paged_prefill=False, bs=16):
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    alloc = paged.BlockAllocator(bs, pool)
    builder = paged.BatchInfoBuilder(bs, 1 << 20, paged_attn_kernel_v=1)
    kc, vc = make_cache(pool, Hkv, d, bs, dtype, fill=float("nan"))  # uninitialised cache
    seqs = []
    sid = 1
    decode_ctx = rng.integers(ctx_lo, ctx_hi + 1, size=n_decode).tolist()
    order = [("chunk", pr) for pr in chunk_priors] + [("decode", c) for c in decode_ctx]
    perm = rng.permutation(len(order))  # interleave: the builder must sort multi-token entries first
    for idx in perm:
        kind, n = order[idx]
        total = n + chunk_len if kind == "chunk" else n
        computed = n if kind == "chunk" else total - 1
        alloc.alloc_seq(sid, total)
        slots = alloc.get_block_idxes(sid, total)
        # the prior context is already in the cache
        kprior = torch.randn((computed, Hkv, d), generator=g).to(dtype)
        vprior = torch.randn((computed, Hkv, d), generator=g).to(dtype)
        ref.reshape_and_cache(kprior, vprior, kc, vc, torch.from_numpy(slots[:computed]))
        builder.sched_out(alloc, sid, rng.integers(0, 1000, size=total).tolist(), computed)
        seqs.append((sid, total, computed))
        sid += 1
    bi = builder.finish()
    T = bi.tokens.numel()
    if fused_qkv:
        assert Hq == Hkv
        qkv = torch.randn((T, 3, Hq, d), generator=g).to(dtype)
        q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    else:
        q = torch.randn((T, Hq, d), generator=g).to(dtype)
        k = torch.randn((T, Hkv, d), generator=g).to(dtype)
        v = torch.randn((T, Hkv, d), generator=g).to(dtype)
        qkv = None
    # ---- oracle: the CPU build's route (every row varlen; paged_attn_kernel_v = 0)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ref.reshape_and_cache(k, v, kc_ref, vc_ref, bi.slot_mapping)
    lens_q = (bi.seqlens_q[1:] - bi.seqlens_q[:-1]).tolist() + [1] * bi.paged_context_lens.numel()
    lens_k = (bi.seqlens_k[1:] - bi.seqlens_k[:-1]).tolist() + bi.paged_context_lens.tolist()
    gather = bi.gather_mapping.tolist()
    for r in range(bi.paged_context_lens.numel()):
        gather += W.slots_for(bi.paged_block_tables[r].tolist(), int(bi.paged_context_lens[r]), bs)
    gm = torch.tensor(gather, dtype=torch.int32)
    gk = torch.empty((len(gather), Hkv, d), dtype=dtype)
    gv = torch.empty_like(gk)
    ref.gather_cached_kv(gk, gv, kc_ref, vc_ref, gm)
    n_rep = Hq // Hkv
    want = ref.varlen_attn(q.float(), ref.repeat_kv(gk, n_rep).float(), ref.repeat_kv(gv, n_rep).float(),
                           W.offsets(lens_q), W.offsets(lens_k), max(lens_q), max(lens_k), 1.0 / math.sqrt(d), True)
    # ---- product: one C-ABI call
    kd, vd = kc.to(device), vc.to(device)
    if fused_qkv:
        qkv_d = qkv.to(device)
        qd, kd_in, vd_in = qkv_d[:, 0], qkv_d[:, 1], qkv_d[:, 2]
    else:
        qd, kd_in, vd_in = q.to(device), k.to(device), v.to(device)
    y = attn.varlen_attn(qd, kd_in, vd_in, bi.to(device), kd, vd, paged_prefill=paged_prefill)
    return y.cpu().reshape(T, Hq, d), want, (kd.cpu(), vd.cpu(), kc_ref, vc_ref), bi


@pytest.mark.parametrize("fused_qkv", [False, True])
def test_mixed_step_phi2_shape_reduced(device, fused_qkv):
    """32 MHA heads of size 80, fp16: 4 chunks of 64 new tokens after 0/100/200/300 cached ones
    plus 20 decode rows, both with contiguous q/k/v and with the fused 3*H*d token stride."""
    y, want, (kc, vc, kc_ref, vc_ref), bi = mixed_step(31, [0, 100, 200, 300], 64, 20, 30, 500, 32, 32, 80,
                                                       torch.float16, 1024, fused_qkv, device)
    assert bi.seqlen_multi == 4 and bi.q_multi == 256 and bi.paged_context_lens.numel() == 20
    assert not torch.isnan(y.float()).any()
    assert (y.float() - want).abs().max().item() <= TOL[torch.float16]
    # the scatter half of the step is bit-exact (NaN-filled slots compare equal as bits)
    assert torch.equal(kc.view(torch.int16), kc_ref.view(torch.int16))
    assert torch.equal(vc.view(torch.int16), vc_ref.view(torch.int16))


def test_mixed_step_gqa_bf16(device):
    y, want, _, bi = mixed_step(32, [0, 17, 640], 200, 33, 1, 900, 32, 8, 128, torch.bfloat16, 2048, False, device)
    assert (y.float() - want).abs().max().item() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("case", ["phi2", "gqa", "all_prefill"])
def test_paged_prefill_route(device, case):
    """The same steps with the multi-token rows reading the cache through block tables
    (hipattn_varlen_attn_paged) instead of a gathered copy."""
    if case == "phi2":
        args, dtype = (31, [0, 100, 200, 300], 64, 20, 30, 500, 32, 32, 80, torch.float16, 1024, True), torch.float16
    elif case == "gqa":
        args, dtype = (32, [0, 17, 640], 200, 33, 1, 900, 32, 8, 128, torch.bfloat16, 2048, False), torch.bfloat16
    else:
        args, dtype = (33, [0, 0, 0], 150, 0, 1, 2, 8, 8, 64, torch.float16, 256, False), torch.float16
    y, want, (kc, vc, kc_ref, vc_ref), bi = mixed_step(*args, device, paged_prefill=True)
    assert bi.multi_block_tables is not None and bi.multi_context_lens.numel() == bi.seqlen_multi
    assert not torch.isnan(y.float()).any()
    assert (y.float() - want).abs().max().item() <= TOL[dtype]
    assert torch.equal(kc.view(torch.int16), kc_ref.view(torch.int16))


@pytest.mark.parametrize("bs", [8, 32])
@pytest.mark.parametrize("paged_prefill", [False, True])
def test_mixed_step_with_8_and_32_token_blocks(device, bs, paged_prefill):
    """The whole composition -- scatter, gather or block tables, prefill rows, decode rows -- on caches of the
    other two block sizes of the reference's matrix."""
    y, want, (kc, vc, kc_ref, vc_ref), bi = mixed_step(35, [0, 17, 640], 200, 33, 1, 900, 32, 8, 128, torch.bfloat16,
                                                       2048 * 16 // bs, False, device, paged_prefill=paged_prefill, bs=bs)
    assert not torch.isnan(y.float()).any()
    assert (y.float() - want).abs().max().item() <= TOL[torch.bfloat16]
    assert torch.equal(kc.view(torch.int16), kc_ref.view(torch.int16))
    assert torch.equal(vc.view(torch.int16), vc_ref.view(torch.int16))


def test_all_prefill_and_all_decode_steps(device):
    y, want, _, bi = mixed_step(33, [0, 0, 0], 150, 0, 1, 2, 8, 8, 64, torch.float16, 256, False, device)
    assert bi.q_multi == 450 and bi.paged_context_lens.numel() == 0
    assert (y.float() - want).abs().max().item() <= TOL[torch.float16]
    y, want, _, bi = mixed_step(34, [], 1, 40, 1, 300, 8, 8, 64, torch.float16, 1024, False, device)
    assert bi.q_multi == 0 and bi.seqlen_multi == 0
    assert (y.float() - want).abs().max().item() <= TOL[torch.float16]


@pytest.mark.parametrize("layout,paged_prefill", [("contiguous", False), ("fused_qkv", False), ("fused_qkv", True)])
def test_config4_full_size_sampled(device, layout, paged_prefill):
    """The benchmark's mixed step at full size: 4 x 512-token chunks after 0/1k/2k/3k cached
    tokens + 120 decode rows with contexts U[1k, 8k], 32 MHA heads, d 80, fp16 -- with contiguous
    q, k, v and with q, k, v as views of one fused [T, 3, H, d] projection (token stride 3*H*d, what
    Phi's layer passes, phi.rs:131-145), the latter also with the multi-token rows reading the cache
    through block tables.  The check (a float64 softmax over the row's gathered context; every row is
    independent) runs on 72 rows: of every chunk its first and last rows and the rows either side of the
    32-, 64-, 96- and 256-row boundaries that the kernels' row blocks and wavefronts cut at, and 24 decode
    rows, the shortest and the longest context among them."""
    rng = np.random.default_rng(4)
    g = torch.Generator().manual_seed(4)
    Hq = Hkv = 32
    d, bs, dtype = 80, 16, torch.float16
    ctxs = rng.integers(1024, 8193, size=120).tolist()
    priors = [0, 1024, 2048, 3072]
    pool = sum((c + 15) // 16 for c in ctxs) + sum((p + 512 + 15) // 16 for p in priors) + 8
    alloc = paged.BlockAllocator(bs, pool)
    builder = paged.BatchInfoBuilder(bs, 1 << 20, 1)
    gd = torch.Generator(device=device).manual_seed(4)
    kd = torch.randn((pool, Hkv, d // 8, bs, 8), generator=gd, dtype=dtype, device=device)
    vd = torch.randn((pool, Hkv, d, bs), generator=gd, dtype=dtype, device=device)
    sid = 1
    for pr in priors:
        alloc.alloc_seq(sid, pr + 512)
        builder.sched_out(alloc, sid, [1] * (pr + 512), pr)
        sid += 1
    for c in ctxs:
        alloc.alloc_seq(sid, c)
        builder.sched_out(alloc, sid, [1] * c, c - 1)
        sid += 1
    bi = builder.finish()
    T = 4 * 512 + 120
    assert bi.tokens.numel() == T and bi.q_multi == 2048
    q = torch.randn((T, Hq, d), generator=g).to(dtype)
    k = torch.randn((T, Hkv, d), generator=g).to(dtype)
    v = torch.randn((T, Hkv, d), generator=g).to(dtype)
    if layout == "fused_qkv":
        qkv = torch.stack([q, k, v], dim=1).to(device)
        qd, kin, vin = qkv[:, 0], qkv[:, 1], qkv[:, 2]
        assert qd.stride(0) == 3 * Hq * d
    else:
        qd, kin, vin = q.to(device), k.to(device), v.to(device)
    y = attn.varlen_attn(qd, kin, vin, bi.to(device), kd, vd, paged_prefill=paged_prefill).reshape(T, Hq, d)
    assert not torch.isnan(y.float()).any()
    kc, vc = kd.cpu(), vd.cpu()  # after the step: holds the new tokens too
    worst = 0.0
    samples = [(512 * i + r, None) for i in range(4) for r in (0, 1, 31, 32, 63, 64, 95, 96, 255, 256, 300, 511)]
    dec_rows = {int(np.argmin(ctxs)), int(np.argmax(ctxs)), *(int(r) for r in rng.choice(120, size=22, replace=False))}
    samples += [(2048 + r, r) for r in sorted(dec_rows)]
    assert len(samples) >= 64
    for row, paged_row in samples:
        if paged_row is None:
            e = row // 512
            lk = priors[e] + 512
            nvis = priors[e] + (row % 512) + 1
            slots = bi.gather_mapping[int(bi.seqlens_k[e]):int(bi.seqlens_k[e]) + lk][:nvis]
        else:
            nvis = int(bi.paged_context_lens[paged_row])
            slots = torch.tensor(W.slots_for(bi.paged_block_tables[paged_row].tolist(), nvis), dtype=torch.int32)
        kk = torch.empty((nvis, Hkv, d), dtype=dtype)
        vv = torch.empty_like(kk)
        ref.gather_cached_kv(kk, vv, kc, vc, slots.to(torch.int32))
        s = torch.einsum("hd,thd->ht", q[row].double(), kk.double()) / math.sqrt(d)
        w = torch.softmax(s, dim=-1)
        want = torch.einsum("ht,thd->hd", w, vv.double())
        worst = max(worst, (y[row].cpu().double() - want).abs().max().item())
    assert worst <= TOL[dtype], worst
