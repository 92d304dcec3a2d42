"""Varlen prefill that reads K/V from the paged cache through block tables
(hipattn_mha_varlen_fwd_paged) against the oracle's route for the same rows -- gather_cached_kv,
repeat_kv, varlen SDPA (llm/mod.rs:181-238 on the CPU build) -- and against the library's own
gather + flash_attn_varlen.  Same gates as the contiguous prefill."""
import math

import numpy as np
import pytest
import torch

from aici_amd import kernels as K
from aici_amd import workloads as W
from aici_amd._lib import HipAttnError
from oracle import refkernels as ref
from tests.common import TOL, make_cache

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "staged"])
def tile_route(request, tuning):
    """Head sizes from 40 up to 128 (and 32) have their tiles copied from the cache into LDS as block images --
    those that do not fill their MFMA tiles (40, 72, 80, 104, ...) with the rest of each image's place cleared;
    the smaller ones -- and every size when the tuning switch paged_prefill_dma is 0 -- are staged through
    registers, as are head sizes above 128, which the four-wavefront kernel takes.  Every test runs both ways."""
    tuning("paged_prefill_dma", -1 if request.param == "auto" else 0)
    return request.param


def paged_case(seed, seqs, Hq, Hkv, d, dtype, pool, bs=16):
    """seqs: (prior, new) token counts.  Every context's K/V (prior and new) is in the cache (blocks of bs
    tokens); every slot no context covers holds NaN, as an uninitialised cache may."""
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    kc, vc = make_cache(pool, Hkv, d, bs, dtype, fill=float("nan"))
    perm = rng.permutation(pool).tolist()
    lens_k = [a + b for a, b in seqs]
    lens_q = [b for _, b in seqs]
    width = max((l + bs - 1) // bs for l in lens_k)
    tables = np.zeros((len(seqs), width), dtype=np.int32)
    slots_all = []
    for i, lk in enumerate(lens_k):
        n = (lk + bs - 1) // bs
        blocks = [perm.pop() for _ in range(n)]
        tables[i, :n] = blocks
        slots = torch.tensor(W.slots_for(blocks, lk, bs), dtype=torch.int64)
        slots_all.append(slots)
        k = torch.randn((lk, Hkv, d), generator=g).to(dtype)
        v = torch.randn((lk, Hkv, d), generator=g).to(dtype)
        ref.reshape_and_cache(k, v, kc, vc, slots)
    q = torch.randn((sum(lens_q), Hq, d), generator=g).to(dtype)
    return dict(q=q, kc=kc, vc=vc, tables=torch.from_numpy(tables), cu_q=W.offsets(lens_q),
                ctx=torch.tensor(lens_k, dtype=torch.int32), lens_q=lens_q, lens_k=lens_k, slots=slots_all,
                scale=1.0 / math.sqrt(d))


def oracle(c, Hq, Hkv, d):
    gm = torch.cat(c["slots"]).to(torch.int32)
    kc, vc = c["kc"].float().nan_to_num(0.0), c["vc"].float().nan_to_num(0.0)   # the oracle reads covered slots only
    gk = torch.empty((gm.numel(), Hkv, d))
    gv = torch.empty_like(gk)
    ref.gather_cached_kv(gk, gv, kc, vc, gm)
    gk, gv = ref.repeat_kv(gk, Hq // Hkv), ref.repeat_kv(gv, Hq // Hkv)
    return ref.varlen_attn(c["q"].float(), gk, gv, c["cu_q"], W.offsets(c["lens_k"]), max(c["lens_q"]),
                           max(c["lens_k"]), c["scale"], True)


def run_paged(c, device, lse=False):
    return K.flash_attn_varlen_paged(c["q"].to(device), c["kc"].to(device), c["vc"].to(device), c["tables"].to(device),
                                     c["cu_q"].to(device), c["ctx"].to(device), max(c["lens_q"]), max(c["lens_k"]),
                                     c["scale"], True, return_lse=lse)


SEQS = [(0, 5), (0, 64), (100, 33), (1000, 256), (17, 1), (0, 300), (63, 65), (2048, 512), (0, 0), (15, 16)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads", [(32, 8, 128), (32, 32, 80), (8, 2, 64), (4, 4, 32), (6, 1, 96), (8, 2, 112), (4, 4, 120),
                                   (4, 2, 8), (4, 2, 40), (4, 4, 72), (2, 1, 104),
                                   (4, 2, 160), (4, 4, 192), (2, 1, 200), (8, 2, 256)])
def test_matches_oracle(device, dtype, heads):
    Hq, Hkv, d = heads
    c = paged_case(31, SEQS, Hq, Hkv, d, dtype, 420)
    got = run_paged(c, device).cpu()
    want = oracle(c, Hq, Hkv, d)
    assert not torch.isnan(got).any()
    assert (got.float() - want).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("bs", [8, 32])
@pytest.mark.parametrize("dtype,heads", [(torch.bfloat16, (32, 8, 128)), (torch.float16, (32, 32, 80)), (torch.bfloat16, (4, 2, 8)),
                                         (torch.float16, (6, 1, 96)), (torch.bfloat16, (4, 4, 72)), (torch.float16, (4, 2, 160)),
                                         (torch.bfloat16, (8, 2, 256))])
def test_caches_of_8_and_32_token_blocks(device, bs, dtype, heads):
    """The reference's gather route works at any block size of the cache (gather_cached_kv takes slots); so does
    the paged prefill, on the kernel that stages its tiles through registers: the same sequences as above,
    with prior contexts that end inside blocks, against the oracle."""
    Hq, Hkv, d = heads
    c = paged_case(33, SEQS, Hq, Hkv, d, dtype, 420 * 16 // bs + 8, bs=bs)
    got, lse = run_paged(c, device, lse=True)
    want = oracle(c, Hq, Hkv, d)
    assert not torch.isnan(got).any()
    assert (got.cpu().float() - want).abs().max().item() <= TOL[dtype]
    # and the same bits as from a cache of 16-token blocks holding the same keys and values (the kernel sees the
    # same tiles), when that one is staged through registers as well
    c16 = paged_case(33, SEQS, Hq, Hkv, d, dtype, 420, bs=16)
    assert torch.equal(c16["q"], c["q"])
    if d > 128 or K.tuning_get("paged_prefill_dma") == 0:
        got16 = run_paged(c16, device)
        if d > 128:
            assert torch.equal(got16, got)


@pytest.mark.parametrize("slope", [6.0, 0.5, -6.0])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_scores_that_drift_along_the_keys(device, dtype, slope):
    """The scores of every row rise (or fall) steadily with the key's position: by `slope` powers of two per
    64-key tile.  Rising fast, the reference maximum of a row (moved only when outgrown by 2^8) moves every
    tile or two and the accumulators are rescaled each time; rising slowly, every sixteen tiles, with
    probabilities up to 256 in between; falling, never after the first tile."""
    Hq, Hkv, d = 8, 2, 128
    c = paged_case(36, [(1500, 520), (0, 700)], Hq, Hkv, d, dtype, 200)
    g = torch.Generator().manual_seed(37)
    u = torch.nn.functional.normalize(torch.randn(d, generator=g), dim=0)
    # q . k * scale * log2(e) = drift(j) + noise, drift(j) = slope * j / 64
    c["q"] = (0.3 * torch.randn(c["q"].shape, generator=g) + 4.0 * u).to(dtype)
    kc, vc = c["kc"], c["vc"]
    for i, lk in enumerate(c["lens_k"]):
        j = torch.arange(lk, dtype=torch.float32)
        along = slope * j / 64.0 / (4.0 * c["scale"] * math.log2(math.e))
        k = (0.3 * torch.randn((lk, Hkv, d), generator=g) + along[:, None, None] * u).to(dtype)
        v = torch.randn((lk, Hkv, d), generator=g).to(dtype)
        ref.reshape_and_cache(k, v, kc, vc, c["slots"][i])
    got, lse = run_paged(c, device, lse=True)
    want = oracle(c, Hq, Hkv, d)
    assert not torch.isnan(got).any()
    assert (got.cpu().float() - want).abs().max().item() <= TOL[dtype]
    # the log-sum-exp against the rows form on the same K/V
    gm = torch.cat(c["slots"]).to(torch.int32).to(device)
    gk = torch.empty((gm.numel(), Hkv, d), dtype=dtype, device=device)
    gv = torch.empty_like(gk)
    K.gather_cached_kv(gk, gv, kc.to(device), vc.to(device), gm)
    _, lse2 = K.flash_attn_varlen(c["q"].to(device), gk, gv, c["cu_q"].to(device), W.offsets(c["lens_k"]).to(device),
                                  max(c["lens_q"]), max(c["lens_k"]), c["scale"], True, return_lse=True)
    for i, lq in enumerate(c["lens_q"]):
        assert torch.allclose(lse[i, :, :lq], lse2[i, :, :lq], atol=2e-3, rtol=1e-4)


def test_random_ragged_cases(device):
    """Sixteen seeded draws of dtype, head shape, batch, and new and prior lengths around the tile and block
    sizes, through the paged cache against the oracle's route."""
    rng = np.random.default_rng(12)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    for case in range(16):
        dtype = pick([torch.bfloat16, torch.float16])
        d = pick([32, 40, 64, 80, 96, 120, 128, 160, 256])
        Hkv = pick([1, 2, 4])
        Hq = Hkv * pick([1, 2, 4])
        seqs = [(pick([0, 0, 7, 16, 64, 100, 333, 700]), pick([1, 5, 15, 16, 17, 63, 64, 65, 255, 257, 513]))
                for _ in range(int(rng.integers(1, 4)))]
        pool = sum((a + b + 15) // 16 for a, b in seqs) + 3
        c = paged_case(200 + case, seqs, Hq, Hkv, d, dtype, pool)
        got = run_paged(c, device).cpu()
        want = oracle(c, Hq, Hkv, d)
        err = (got.float() - want).abs().max().item()
        assert not torch.isnan(got).any() and err <= TOL[dtype], (case, dtype, d, Hq, Hkv, seqs, err)


def test_agrees_with_gather_then_contiguous_prefill_and_lse(device):
    dtype = torch.bfloat16
    Hq, Hkv, d = 32, 8, 128
    c = paged_case(32, [(700, 300), (0, 1024), (3000, 40)], Hq, Hkv, d, dtype, 400)
    got, lse = run_paged(c, device, lse=True)
    gm = torch.cat(c["slots"]).to(torch.int32).to(device)
    gk = torch.empty((gm.numel(), Hkv, d), dtype=dtype, device=device)
    gv = torch.empty_like(gk)
    K.gather_cached_kv(gk, gv, c["kc"].to(device), c["vc"].to(device), gm)
    cu_k = W.offsets(c["lens_k"]).to(device)
    want, lse2 = K.flash_attn_varlen(c["q"].to(device), gk, gv, c["cu_q"].to(device), cu_k, max(c["lens_q"]),
                                     max(c["lens_k"]), c["scale"], True, return_lse=True)
    assert (got.float() - want.float()).abs().max().item() <= TOL[dtype]
    for i, lq in enumerate(c["lens_q"]):
        assert torch.allclose(lse[i, :, :lq], lse2[i, :, :lq], atol=2e-3, rtol=1e-4)


def test_invariant_under_block_permutation(device):
    dtype = torch.float16
    Hq, Hkv, d = 8, 2, 128
    c = paged_case(33, [(130, 70), (0, 257)], Hq, Hkv, d, dtype, 64)
    got = run_paged(c, device)
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(2))
    kc2, vc2 = torch.empty_like(c["kc"]), torch.empty_like(c["vc"])
    kc2[perm] = c["kc"]
    vc2[perm] = c["vc"]
    nblk = [(l + 15) // 16 for l in c["lens_k"]]
    t2 = c["tables"].clone()
    for i, n in enumerate(nblk):
        t2[i, :n] = perm[c["tables"][i, :n].long()].to(torch.int32)
    c2 = dict(c, kc=kc2, vc=vc2, tables=t2)
    assert torch.equal(run_paged(c2, device), got)


def test_argument_errors(device):
    c = paged_case(34, [(0, 20)], 4, 4, 64, torch.float16, 8)
    with pytest.raises(HipAttnError, match="block-table columns"):
        K.flash_attn_varlen_paged(c["q"].to(device), c["kc"].to(device), c["vc"].to(device), c["tables"].to(device),
                                  c["cu_q"].to(device), c["ctx"].to(device), 20, 16 * c["tables"].size(1) + 1,
                                  c["scale"], True)
    big = paged_case(35, [(0, 4)], 2, 2, 264, torch.float16, 4)
    with pytest.raises(HipAttnError, match="head size"):
        run_paged(big, device)


def test_blocks_beyond_4_gib_of_cache(device):
    """A cache of 4.6 GB per tensor whose used blocks lie past the 4 GiB mark: block offsets need 64 bits in
    the scatter, in both paged prefill forms and in the decode kernel.  Checked against the library's own
    gather + contiguous prefill on the same cache (itself checked against the oracle above)."""
    dtype, Hq, Hkv, d, bs = torch.bfloat16, 16, 8, 128, 16
    nb = 140000                                           # x 32 KiB per block = 4.59 GB each for K and V
    kc = torch.zeros((nb, Hkv, d // 8, bs, 8), dtype=dtype, device=device)
    vc = torch.zeros((nb, Hkv, d, bs), dtype=dtype, device=device)
    g = torch.Generator().manual_seed(35)
    seqs = [(1500, 300), (0, 700), (40, 1)]
    lens_k, lens_q = [a + b for a, b in seqs], [b for _, b in seqs]
    high = (136000 + torch.randperm(4000, generator=g)).tolist()      # byte offsets from 4.45 GB up
    width = max((l + 15) // 16 for l in lens_k)
    tables = torch.zeros((len(seqs), width), dtype=torch.int32)
    slots = []
    for i, lk in enumerate(lens_k):
        n = (lk + 15) // 16
        blocks = [high.pop() for _ in range(n)]
        tables[i, :n] = torch.tensor(blocks, dtype=torch.int32)
        slots += W.slots_for(blocks, lk)
    k = torch.randn((sum(lens_k), Hkv, d), generator=g).to(dtype).to(device)
    v = torch.randn((sum(lens_k), Hkv, d), generator=g).to(dtype).to(device)
    q = torch.randn((sum(lens_q), Hq, d), generator=g).to(dtype).to(device)
    slots_d = torch.tensor(slots, dtype=torch.int64, device=device)
    K.reshape_and_cache(k, v, kc, vc, slots_d)
    gk, gv = torch.empty_like(k), torch.empty_like(v)
    K.gather_cached_kv(gk, gv, kc, vc, slots_d.to(torch.int32))
    assert torch.equal(gk, k) and torch.equal(gv, v)
    cu_q, cu_k = W.offsets(lens_q).to(device), W.offsets(lens_k).to(device)
    ctx = torch.tensor(lens_k, dtype=torch.int32, device=device)
    scale = 1.0 / math.sqrt(d)
    want = K.flash_attn_varlen(q, k, v, cu_q, cu_k, max(lens_q), max(lens_k), scale, True)
    got = K.flash_attn_varlen_paged(q, kc, vc, tables.to(device), cu_q, ctx, max(lens_q), max(lens_k), scale, True)
    assert (got.float() - want.float()).abs().max().item() <= TOL[dtype]
    # decode rows over the same contexts: equal to the last row of a prefill over the whole context
    qd = torch.randn((len(seqs), Hq, d), generator=g).to(dtype).to(device)
    out = torch.empty_like(qd)
    K.paged_attention_v1(out, qd, kc, vc, Hkv, scale, tables.to(device), ctx, 16, max(lens_k))
    one = W.offsets([1] * len(seqs)).to(device)
    want_d = K.flash_attn_varlen(qd, k, v, one, cu_k, 1, max(lens_k), scale, True)
    assert (out.float() - want_d.float()).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("heads", [(32, 8, 128), (32, 32, 80)])
def test_fp32_output_is_the_unrounded_result(device, heads):
    """out in f32: the accumulators divided by the row sums; rounding it gives the bf16 output bit for bit,
    and it is closer to the oracle than the rounded one."""
    Hq, Hkv, d = heads
    c = paged_case(35, SEQS, Hq, Hkv, d, torch.bfloat16, 420)
    args = (c["q"].to(device), c["kc"].to(device), c["vc"].to(device), c["tables"].to(device), c["cu_q"].to(device),
            c["ctx"].to(device), max(c["lens_q"]), max(c["lens_k"]), c["scale"], True)
    got32 = K.flash_attn_varlen_paged(*args, out_dtype=torch.float32)
    got = K.flash_attn_varlen_paged(*args)
    assert got32.dtype == torch.float32 and torch.equal(got, got32.to(torch.bfloat16))
    want = oracle(c, Hq, Hkv, d)
    assert (got32.cpu() - want).abs().max().item() <= (got.cpu().float() - want).abs().max().item() <= TOL[torch.bfloat16]
