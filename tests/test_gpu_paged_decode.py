"""Paged decode attention through the C ABI against the oracle (gather + Lq=1 varlen SDPA,
the way rLLM's CPU build computes single-token rows).  Gates: max-abs error <= 2e-2 (bf16),
<= 5e-3 (fp16) against the fp32 oracle on the same rounded inputs."""
import numpy as np
import pytest
import torch

from aici_amd import kernels as K
from aici_amd import workloads as W
from aici_amd._lib import HipAttnError
from oracle import refkernels as ref
from tests.common import TOL

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "flat", "partitioned"])
def launch_strategy(request, tuning):
    """paged_attention_v1 has two launch strategies (one list of block pairs cut into equal
    ranges per wavefront, or one workgroup per context partition) and picks by problem size;
    every test runs under the library's own choice and with each one forced."""
    tuning("decode_flat", {"auto": -1, "flat": 1, "partitioned": 0}[request.param])
    return request.param


_ORACLE_CACHE = {}


def run_v1(c: W.DecodeInputs, device, alibi=None):
    d = c.to(device)
    out = torch.full_like(d.q, float("nan"))
    K.paged_attention_v1(out, d.q, d.key_cache, d.value_cache, c.num_kv_heads, c.scale, d.block_tables,
                         d.context_lens, 16, c.max_ctx, alibi.to(device) if alibi is not None else None)
    return out.cpu()


def oracle(c: W.DecodeInputs, alibi=None, rows=None):
    q, bt, cl = c.q, c.block_tables, c.context_lens
    if rows is not None:
        q, bt, cl = q[rows], bt[rows], cl[rows]
    return ref.paged_attention(q.float(), c.key_cache.float(), c.value_cache.float(), c.num_kv_heads, c.scale, bt,
                               cl, 16, alibi)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads", [(32, 8, 128), (32, 32, 80), (8, 8, 64), (16, 1, 96), (40, 2, 112), (4, 4, 256)])
def test_matches_oracle_over_head_shapes(device, dtype, heads):
    Hq, Hkv, d = heads
    c = W.decode_inputs(11, 9, 1, 1500, Hq, Hkv, d, dtype, 1024)
    got = run_v1(c, device)
    want = oracle(c)
    assert not torch.isnan(got).any()
    assert (got.float() - want).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_context_edge_lengths_and_stale_cache_contents(device, dtype):
    # Contexts around block and partition boundaries, including 0; every cache slot that no
    # context covers holds NaN, as an uninitialised (torch.empty) cache may.
    lens = [0, 1, 15, 16, 17, 31, 32, 33, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1025]
    S = len(lens)
    c = W.decode_inputs(12, S, 1, 2, 32, 8, 128, dtype, 700)
    ctx = np.array(lens, dtype=np.int32)
    nblk = (ctx + 15) // 16
    perm = np.random.default_rng(3).permutation(700)
    tables = np.zeros((S, int(nblk.max())), dtype=np.int32)
    covered = torch.zeros((700, 16), dtype=torch.bool)
    pos = 0
    for s in range(S):
        tables[s, :nblk[s]] = perm[pos:pos + nblk[s]]
        for t in range(ctx[s]):
            covered[tables[s, t // 16], t % 16] = True
        pos += nblk[s]
    c.block_tables, c.context_lens, c.max_ctx = torch.from_numpy(tables), torch.from_numpy(ctx), int(ctx.max())
    kc, vc = c.key_cache, c.value_cache
    kc.permute(0, 3, 1, 2, 4)[~covered] = float("nan")
    vc.permute(0, 3, 1, 2)[~covered] = float("nan")
    got = run_v1(c, device)
    kc.permute(0, 3, 1, 2, 4)[~covered] = 0.0   # the oracle never reads them; avoid NaN*0 in its gathers
    vc.permute(0, 3, 1, 2)[~covered] = 0.0
    want = oracle(c)
    assert not torch.isnan(got).any()
    assert torch.all(got[0] == 0)  # empty context -> zeros
    assert (got.float() - want).abs().max().item() <= TOL[dtype]


def test_single_partition_path_and_many_partitions_agree_with_oracle(device):
    # S large -> one partition per sequence; S = 1 -> the context is split many ways.
    big = W.decode_inputs(13, 300, 100, 400, 8, 2, 128, torch.float16, 8000)
    assert (run_v1(big, device).float() - oracle(big)).abs().max().item() <= TOL[torch.float16]
    one = W.decode_inputs(14, 1, 4000, 4096, 32, 8, 128, torch.float16, 300)
    assert (run_v1(one, device).float() - oracle(one)).abs().max().item() <= TOL[torch.float16]


def test_more_sequences_than_the_flat_split_tables_hold(device):
    # 1100 sequences: beyond the 1024 the flat split keeps in LDS, so every strategy setting
    # must land on the partitioned launch; many empty and one-token contexts among them.
    c = W.decode_inputs(19, 1100, 0, 40, 8, 2, 64, torch.float16, 3400)
    got = run_v1(c, device)
    assert not torch.isnan(got).any()
    assert (got.float() - oracle(c)).abs().max().item() <= TOL[torch.float16]


def test_query_groups_wider_than_one_mfma_tile(device):
    # 40 query heads on one kv head: three column groups of 16, the last one partial
    c = W.decode_inputs(20, 7, 1, 900, 40, 1, 128, torch.bfloat16, 420)
    assert (run_v1(c, device).float() - oracle(c)).abs().max().item() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_v2_entry_with_caller_workspaces(device, dtype):
    c = W.decode_inputs(15, 6, 200, 1400, 32, 8, 128, dtype, 600)
    d = c.to(device)
    want = oracle(c)
    for part_tokens in (512, 96):
        P = (c.max_ctx + part_tokens - 1) // part_tokens
        S, Hq, hd = c.q.shape
        exp_sums = torch.empty((S, Hq, P), dtype=torch.float32, device=device)
        max_logits = torch.empty_like(exp_sums)
        tmp_out = torch.empty((S, Hq, P, hd), dtype=dtype, device=device)
        out = torch.empty_like(d.q)
        K.paged_attention_v2(out, exp_sums, max_logits, tmp_out, d.q, d.key_cache, d.value_cache, 8, c.scale,
                             d.block_tables, d.context_lens, 16, c.max_ctx)
        assert (out.cpu().float() - want).abs().max().item() <= TOL[dtype]
    # the reference's partials: max_logits are natural-log maxima of the scaled scores
    s0 = 0
    ctx0 = int(c.context_lens[s0])
    slots = torch.tensor(W.slots_for(c.block_tables[s0].tolist(), min(ctx0, 96)), dtype=torch.int32)
    kk = torch.empty((len(slots), 8, 128), dtype=dtype)
    vv = torch.empty_like(kk)
    ref.gather_cached_kv(kk, vv, c.key_cache, c.value_cache, slots)
    logits = (kk[:, 0].float() @ c.q[s0, 0].float()) * c.scale
    assert abs(max_logits[s0, 0, 0].item() - logits.max().item()) < 2e-2


def test_alibi_and_strided_query(device):
    dtype = torch.float16
    c = W.decode_inputs(16, 5, 10, 600, 32, 32, 80, dtype, 300)
    slopes = torch.tensor([2.0 ** (-(i + 1) / 4) for i in range(32)], dtype=torch.float32)
    got = run_v1(c, device, slopes)
    want = oracle(c, slopes)
    assert (got.float() - want).abs().max().item() <= TOL[dtype]
    # q as a chunk of a fused [S, 3, H, d] projection (row stride 3*H*d), as Phi passes it
    d = c.to(device)
    fused = torch.zeros((5, 3, 32, 80), dtype=dtype, device=device)
    fused[:, 0] = d.q
    out = torch.empty_like(d.q)
    K.paged_attention_v1(out, fused[:, 0], d.key_cache, d.value_cache, 32, c.scale, d.block_tables, d.context_lens,
                         16, c.max_ctx)
    assert (out.cpu().float() - oracle(c)).abs().max().item() <= TOL[dtype]


def test_invariant_under_block_permutation_and_equals_prefill_last_row(device):
    dtype = torch.bfloat16
    c = W.decode_inputs(17, 4, 50, 700, 32, 8, 128, dtype, 256)
    got = run_v1(c, device)
    perm = torch.randperm(256, generator=torch.Generator().manual_seed(1))
    kc2, vc2 = torch.empty_like(c.key_cache), torch.empty_like(c.value_cache)
    kc2[perm] = c.key_cache
    vc2[perm] = c.value_cache
    c2 = W.DecodeInputs(c.q, kc2, vc2, perm[c.block_tables.long()].to(torch.int32), c.context_lens, c.max_ctx,
                        c.scale, 8)
    assert torch.equal(run_v1(c2, device), got)  # same arithmetic in the same order
    # the decode row equals the last row of a causal prefill over the same keys
    s = 1
    ctx = int(c.context_lens[s])
    slots = torch.tensor(W.slots_for(c.block_tables[s].tolist(), ctx), dtype=torch.int32)
    kk = torch.empty((ctx, 8, 128), dtype=dtype)
    vv = torch.empty_like(kk)
    ref.gather_cached_kv(kk, vv, c.key_cache, c.value_cache, slots)
    qq = torch.zeros((ctx, 32, 128), dtype=dtype)
    qq[-1] = c.q[s]
    cu = W.offsets([ctx]).to(device)
    pre = K.flash_attn_varlen(qq.to(device), kk.to(device), vv.to(device), cu, cu, ctx, ctx, c.scale, True)
    assert (pre[-1].cpu().float() - got[s].float()).abs().max().item() <= 2e-2


def test_blocks_in_token_order_and_scattered_give_the_same_bits_on_long_contexts(device, tuning):
    """A wavefront visits the block pairs of a batch in an order of its own (bit-reversed positions), which depends
    on the position in the context alone: the same keys give the same bits wherever their blocks lie -- in the pool
    in token order, as an allocator hands them to a fresh prompt, or scattered -- and the values are the oracle's.
    Contexts long enough for full batches of 32 pairs and for ragged ends, flat split and partitioned launch."""
    dtype = torch.bfloat16
    c = W.decode_inputs(23, 12, 1500, 5000, 32, 8, 128, dtype, 3000)
    nb = (c.context_lens.numpy().astype(np.int64) + 15) // 16
    order = np.zeros(tuple(c.block_tables.shape), dtype=np.int64)
    start = 0
    for s_, n in enumerate(nb):
        order[s_, :n] = np.arange(start, start + n)
        start += int(n)
    kc2, vc2 = torch.zeros_like(c.key_cache), torch.zeros_like(c.value_cache)
    for s_, n in enumerate(nb):  # the same keys and values, moved to blocks 0, 1, 2, ... in token order
        kc2[order[s_, :n]] = c.key_cache[c.block_tables[s_, :n].long()]
        vc2[order[s_, :n]] = c.value_cache[c.block_tables[s_, :n].long()]
    c2 = W.DecodeInputs(c.q, kc2, vc2, torch.from_numpy(order.astype(np.int32)), c.context_lens, c.max_ctx, c.scale, 8)
    want = ref.paged_attention_fp64(c.q, c.key_cache, c.value_cache, 8, c.scale, c.block_tables, c.context_lens, 16)
    for flat in (1, 0):
        tuning("decode_flat", flat)
        a, b = run_v1(c, device), run_v1(c2, device)
        assert torch.equal(a, b)
        assert (a.cpu().double() - want).abs().max().item() <= TOL[dtype]


def test_config2_full_size(device):
    """The benchmark's decode configuration at full size: every one of the 64 sequences against the float64
    statement of the oracle, and every third one against the slot-by-slot oracle itself."""
    c = W.config2()
    assert c.q.shape == (64, 32, 128) and c.key_cache.shape == (20000, 8, 16, 16, 8)
    got = run_v1(c, device)
    assert not torch.isnan(got).any()
    if "config2" not in _ORACLE_CACHE:
        rows = list(range(0, 64, 3))
        _ORACLE_CACHE["config2"] = (rows, oracle(c, rows=rows),
                                    ref.paged_attention_fp64(c.q, c.key_cache, c.value_cache, c.num_kv_heads, c.scale,
                                                             c.block_tables, c.context_lens, 16))
    rows, want, want64 = _ORACLE_CACHE["config2"]
    assert (got[rows].float() - want).abs().max().item() <= TOL[torch.bfloat16]
    assert (got.double() - want64).abs().max().item() <= TOL[torch.bfloat16]
    # size-independent property on all 64: attention output is a convex combination of the
    # context's V rows, so each coordinate lies within the range of that kv head's values
    assert got.float().abs().max().item() <= c.value_cache.float().abs().max().item()


@pytest.mark.parametrize("bs", [8, 32])
def test_config2_shape_at_the_other_block_sizes(device, bs):
    """The decode configuration's full shape (64 sequences, contexts U[512, 4096], 32 q / 8 kv heads, d 128, bf16)
    with the cache in 8- and 32-token blocks: all 64 sequences against the float64 statement."""
    key = ("config2", bs)
    if key not in _ORACLE_CACHE:
        c = W.decode_inputs(2, 64, 512, 4096, 32, 8, 128, torch.bfloat16, 20000 * 16 // bs, block_size=bs)
        _ORACLE_CACHE[key] = (c, ref.paged_attention_fp64(c.q, c.key_cache, c.value_cache, c.num_kv_heads, c.scale,
                                                          c.block_tables, c.context_lens, bs))
    c, want64 = _ORACLE_CACHE[key]
    d = c.to(device)
    out = torch.full_like(d.q, float("nan"))
    K.paged_attention_v1(out, d.q, d.key_cache, d.value_cache, c.num_kv_heads, c.scale, d.block_tables, d.context_lens,
                         bs, c.max_ctx)
    got = out.cpu()
    assert not torch.isnan(got).any()
    assert (got.double() - want64).abs().max().item() <= TOL[torch.bfloat16]


def test_argument_errors(device):
    c = W.decode_inputs(18, 2, 5, 40, 8, 2, 128, torch.float16, 16).to(device)
    out = torch.empty_like(c.q)
    args = (c.key_cache, c.value_cache, 2, c.scale, c.block_tables, c.context_lens)
    with pytest.raises(HipAttnError, match="unsupported block size 4"):
        K.paged_attention_v1(out, c.q, *args, 4, c.max_ctx)
    with pytest.raises(HipAttnError, match="key_cache shape does not match"):
        K.paged_attention_v1(out, c.q, *args, 32, c.max_ctx)        # the cache holds 16-token blocks
    with pytest.raises(HipAttnError, match="key_cache shape does not match"):                # f32 wants x = 4
        K.paged_attention_v1(out.float(), c.q.float(), c.key_cache.float(), c.value_cache.float(), 2, c.scale,
                             c.block_tables, c.context_lens, 16, c.max_ctx)
    with pytest.raises(HipAttnError, match="unsupported data type"):
        K.paged_attention_v1(out.to(torch.int32), c.q.to(torch.int32), *args, 16, c.max_ctx)
    with pytest.raises(HipAttnError, match="not divisible"):
        K.paged_attention_v1(out, c.q, c.key_cache, c.value_cache, 3, c.scale, c.block_tables, c.context_lens, 16,
                             c.max_ctx)
    with pytest.raises(HipAttnError, match="block-table columns"):
        K.paged_attention_v1(out, c.q, *args, 16, 16 * c.block_tables.size(1) + 1)
    bad = torch.empty((2, 8, 72), dtype=torch.float16, device=c.q.device)
    with pytest.raises(HipAttnError):
        K.paged_attention_v1(bad, bad, *args, 16, c.max_ctx)


# The rest of the reference's support matrix (attention_kernels.cu:594-700: block sizes 8/16/32,
# float / half / bf16): 8- and 32-token blocks of a 2-byte type run on the MFMA kernels (partitioned launch) at the
# reference's head sizes, float caches and other head sizes on a plain fp32 kernel.
FP32_TOL = 2e-5


@pytest.mark.parametrize("case", [
    (torch.bfloat16, 8, (32, 8, 128)), (torch.float16, 32, (32, 8, 128)), (torch.float16, 8, (32, 32, 80)),
    (torch.bfloat16, 32, (16, 1, 96)), (torch.float32, 16, (32, 8, 128)), (torch.float32, 8, (8, 8, 64)),
    (torch.float32, 32, (4, 4, 256)), (torch.float16, 32, (40, 2, 112)), (torch.float32, 16, (6, 3, 72)),
])
def test_other_block_sizes_and_fp32_match_the_oracle(device, case):
    dtype, bs, (Hq, Hkv, d) = case
    c = W.decode_inputs(31, 9, 1, 1500, Hq, Hkv, d, dtype, 9 * (1500 // bs + 1), block_size=bs)
    dd = c.to(device)
    out = torch.full_like(dd.q, float("nan"))
    K.paged_attention_v1(out, dd.q, dd.key_cache, dd.value_cache, Hkv, c.scale, dd.block_tables, dd.context_lens, bs,
                         c.max_ctx)
    want = ref.paged_attention(c.q.float(), c.key_cache.float(), c.value_cache.float(), Hkv, c.scale, c.block_tables,
                               c.context_lens, bs)
    tol = FP32_TOL if dtype == torch.float32 else TOL[dtype]
    assert not torch.isnan(out).any()
    assert (out.cpu().float() - want).abs().max().item() <= tol
    # the caller-workspace form: 3 partitions over the longest context, and far more than needed
    for P in (3, 40):
        out2 = torch.full_like(dd.q, float("nan"))
        exp_sums = torch.full((9, Hq, P), float("nan"), dtype=torch.float32, device=device)
        max_logits = torch.full_like(exp_sums, float("nan"))
        tmp = torch.full((9, Hq, P, d), float("nan"), dtype=dtype, device=device)
        K.paged_attention_v2(out2, exp_sums, max_logits, tmp, dd.q, dd.key_cache, dd.value_cache, Hkv, c.scale,
                             dd.block_tables, dd.context_lens, bs, c.max_ctx)
        assert (out2.cpu().float() - want).abs().max().item() <= tol


@pytest.mark.parametrize("dtype,bs", [(torch.float32, 16), (torch.bfloat16, 8), (torch.float16, 32)])
def test_other_block_sizes_edges_alibi_and_stale_slots(device, dtype, bs):
    lens = [0, 1, bs - 1, bs, bs + 1, 255, 256, 257, 511, 512, 513, 1023, 1025]
    S = len(lens)
    pool = sum(lens) // bs + 2 * S
    c = W.decode_inputs(32, S, 1, 2, 8, 2, 64, dtype, pool, block_size=bs)
    ctx = np.array(lens, dtype=np.int32)
    nblk = (ctx + bs - 1) // bs
    perm = np.random.default_rng(5).permutation(pool)
    tables = np.zeros((S, int(nblk.max())), dtype=np.int32)
    covered = torch.zeros((pool, bs), dtype=torch.bool)
    pos = 0
    for s in range(S):
        tables[s, :nblk[s]] = perm[pos:pos + nblk[s]]
        for t in range(ctx[s]):
            covered[tables[s, t // bs], t % bs] = True
        pos += nblk[s]
    c.block_tables, c.context_lens, c.max_ctx = torch.from_numpy(tables), torch.from_numpy(ctx), int(ctx.max())
    alibi = torch.linspace(-0.3, 0.2, 8)
    want = ref.paged_attention(c.q.float(), c.key_cache.float(), c.value_cache.float(), 2, c.scale, c.block_tables,
                               c.context_lens, bs, alibi)
    c.key_cache.permute(0, 3, 1, 2, 4)[~covered] = float("nan")
    c.value_cache.permute(0, 3, 1, 2)[~covered] = float("nan")
    dd = c.to(device)
    out = torch.full_like(dd.q, float("nan"))
    K.paged_attention_v1(out, dd.q, dd.key_cache, dd.value_cache, 2, c.scale, dd.block_tables, dd.context_lens, bs,
                         c.max_ctx, alibi.to(device))
    assert not torch.isnan(out).any()
    assert torch.all(out[0] == 0)   # no context: a zero row, as the oracle gives
    # one token of context: its value, exactly -- the normaliser is 1 / sum as in rLLM's CPU reference kernels
    # (refkernels.rs:59-148), not the CUDA kernel's 1 / (sum + 1e-6) (attention_kernels.cu:262), which would give
    # v / (1 + 1e-6) and shows in float32
    one = c.value_cache[int(tables[1, 0]), :, :, 0].repeat_interleave(4, dim=0)   # [Hq, d]: 8 q heads on 2 kv heads
    assert torch.equal(out[1].cpu(), one.to(dtype))
    tol = 5e-5 if dtype == torch.float32 else TOL[dtype]
    assert (out.cpu().float() - want).abs().max().item() <= tol


@pytest.mark.parametrize("dtype,heads", [(torch.bfloat16, (32, 8, 128)), (torch.float16, (40, 1, 64)),
                                         (torch.bfloat16, (8, 8, 80)), (torch.float16, (6, 2, 256))])
@pytest.mark.parametrize("part_blocks", [0, 2, 64, "flat"])
def test_block_sizes_8_and_32_give_the_bits_of_block_size_16(device, tuning, dtype, heads, part_blocks):
    """The MFMA kernels walk a context in runs of 16 tokens whatever the cache's block size is, so the same keys
    and values scattered into caches of 8-, 16- and 32-token blocks (each with its own shuffled table, the
    unused slots holding NaN) must give the same bits when the contexts are cut in the same places -- partitions
    of the library's own choice, the shortest (2 runs) and the longest (64 runs: with 8-token blocks a partition
    then spans 128 table columns), and the flat split.  One of them is held against the float64 statement."""
    Hq, Hkv, d = heads
    if part_blocks == "flat":          # one list of block pairs cut into equal ranges: the same cut at every block size
        tuning("decode_flat", 1)
    else:
        tuning("decode_flat", 0)
        tuning("decode_part_blocks", part_blocks)
    lens = [1, 7, 17, 500, 1111, 2049, 4100]
    S, T = len(lens), sum(lens)
    g = torch.Generator().manual_seed(77)
    q = torch.randn((S, Hq, d), generator=g).to(dtype)
    k = torch.randn((T, Hkv, d), generator=g).to(dtype)
    v = torch.randn((T, Hkv, d), generator=g).to(dtype)
    ctx = torch.tensor(lens, dtype=torch.int32)
    outs = {}
    for bs in (16, 8, 32):
        nblk = [(l + bs - 1) // bs for l in lens]
        pool = sum(nblk) + 7
        perm = np.random.default_rng(bs).permutation(pool)
        tables = np.zeros((S, max(nblk)), dtype=np.int32)
        slots, pos = [], 0
        for i, n in enumerate(nblk):
            tables[i, :n] = perm[pos:pos + n]
            slots += W.slots_for(perm[pos:pos + n].tolist(), lens[i], bs)
            pos += n
        kshape, vshape = W.cache_shapes(pool, Hkv, d, bs, dtype)
        kc = torch.full(kshape, float("nan"), dtype=dtype, device=device)
        vc = torch.full(vshape, float("nan"), dtype=dtype, device=device)
        K.reshape_and_cache(k.to(device), v.to(device), kc, vc, torch.tensor(slots, dtype=torch.int64, device=device))
        out = torch.full((S, Hq, d), float("nan"), dtype=dtype, device=device)
        K.paged_attention_v1(out, q.to(device), kc, vc, Hkv, d ** -0.5, torch.from_numpy(tables).to(device),
                             ctx.to(device), bs, max(lens))
        outs[bs] = out.cpu()
        assert not torch.isnan(outs[bs]).any()
        if bs == 8:
            want = ref.paged_attention_fp64(q, torch.nan_to_num(kc.cpu()), torch.nan_to_num(vc.cpu()), Hkv, d ** -0.5,
                                            torch.from_numpy(tables), ctx, bs)
            assert (outs[bs].double() - want).abs().max().item() <= TOL[dtype]
    assert torch.equal(outs[8], outs[16]) and torch.equal(outs[32], outs[16])


# ---- scratch memory: caller-provided workspaces, streams, context lengths beyond the stated maximum ----

WS_CASES = [
    ("flat", (40, 900, 2048, 32, 8, 128, torch.bfloat16, 4000)),
    ("partitioned", (9, 1, 1500, 32, 8, 128, torch.float16, 1024)),
    ("flat_wide_groups", (24, 1000, 3000, 40, 1, 128, torch.bfloat16, 4800)),
]


@pytest.mark.parametrize("name,shape", WS_CASES, ids=[n for n, _ in WS_CASES])
def test_caller_workspace_entry_matches_v1(device, name, shape):
    """hipattn_paged_attention_v1_ws on a workspace of exactly the reported size, filled with
    garbage (nothing in it has to survive or be prepared between calls): bit-identical to v1, twice in a
    row on the same workspace, and no byte outside the reported size is touched."""
    S, lo, hi, Hq, Hkv, d, dtype, pool = shape
    c = W.decode_inputs(41, S, lo, hi, Hq, Hkv, d, dtype, pool)
    dd = c.to(device)
    want = torch.full_like(dd.q, float("nan"))
    K.paged_attention_v1(want, dd.q, dd.key_cache, dd.value_cache, Hkv, c.scale, dd.block_tables, dd.context_lens,
                         16, c.max_ctx)
    n = K.paged_attention_workspace_size(S, Hq, Hkv, d, 16, c.max_ctx, dtype)
    assert n >= 0 and n % 4 == 0
    guard = 4096
    ws = torch.full((n + guard,), 0xA5, dtype=torch.uint8, device=device)
    for _ in range(2):
        out = torch.full_like(dd.q, float("nan"))
        K.paged_attention_v1_ws(out, dd.q, dd.key_cache, dd.value_cache, Hkv, c.scale, dd.block_tables,
                                dd.context_lens, 16, c.max_ctx, ws[:n] if n else None)
        assert torch.equal(out, want)
    assert torch.all(ws[n:] == 0xA5)
    if n:
        with pytest.raises(HipAttnError, match="too small"):
            K.paged_attention_v1_ws(out, dd.q, dd.key_cache, dd.value_cache, Hkv, c.scale, dd.block_tables,
                                    dd.context_lens, 16, c.max_ctx, ws[:n - 256])
        with pytest.raises(HipAttnError, match="workspace is NULL"):
            K.paged_attention_v1_ws(out, dd.q, dd.key_cache, dd.value_cache, Hkv, c.scale, dd.block_tables,
                                    dd.context_lens, 16, c.max_ctx, None)
    assert (want.cpu().float() - oracle(c)).abs().max().item() <= TOL[dtype]


def test_two_streams_share_nothing(device):
    """v1 keeps its scratch memory per stream: two streams running steps of different sizes at the
    same time both get the results they get when run alone."""
    a = W.decode_inputs(42, 48, 1000, 4096, 32, 8, 128, torch.bfloat16, 9000)
    b = W.decode_inputs(43, 7, 200, 1400, 32, 8, 128, torch.bfloat16, 700)
    da, db = a.to(device), b.to(device)

    def call(d, c, out):
        K.paged_attention_v1(out, d.q, d.key_cache, d.value_cache, 8, c.scale, d.block_tables, d.context_lens, 16,
                             c.max_ctx)

    alone_a, alone_b = torch.empty_like(da.q), torch.empty_like(db.q)
    call(da, a, alone_a)
    call(db, b, alone_b)
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a = [torch.full_like(da.q, float("nan")) for _ in range(6)]
    outs_b = [torch.full_like(db.q, float("nan")) for _ in range(6)]
    for i in range(6):  # interleaved enqueues: the two streams' kernels overlap on the device
        with torch.cuda.stream(sa):
            call(da, a, outs_a[i])
        with torch.cuda.stream(sb):
            call(db, b, outs_b[i])
    torch.cuda.synchronize()
    for o in outs_a:
        assert torch.equal(o, alone_a)
    for o in outs_b:
        assert torch.equal(o, alone_b)
    assert (alone_a.cpu().float()[::6] - oracle(a, rows=list(range(0, 48, 6)))).abs().max().item() <= TOL[torch.bfloat16]
    assert (alone_b.cpu().float() - oracle(b)).abs().max().item() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype,bs", [(torch.bfloat16, 16), (torch.float32, 16), (torch.float16, 8)])
def test_context_lengths_above_the_stated_maximum_are_cut_there(device, dtype, bs):
    """A context_lens entry above max_context_len: every kernel attends to the first max_context_len
    tokens, as if the entry had been that."""
    c = W.decode_inputs(44, 6, 300, 1200, 8, 2, 128, dtype, 6 * (1200 // bs + 1), block_size=bs)
    cut = 640
    dd = c.to(device)
    out = torch.full_like(dd.q, float("nan"))
    K.paged_attention_v1(out, dd.q, dd.key_cache, dd.value_cache, 2, c.scale, dd.block_tables, dd.context_lens, bs,
                         cut)
    want = ref.paged_attention(c.q.float(), c.key_cache.float(), c.value_cache.float(), 2, c.scale, c.block_tables,
                               torch.clamp(c.context_lens, max=cut), bs)
    tol = FP32_TOL if dtype == torch.float32 else TOL[dtype]
    assert not torch.isnan(out).any()
    assert (out.cpu().float() - want).abs().max().item() <= tol


def test_config5_decode_shape(device):
    """The decode attention of the full-model configuration at its own shape: 128 sequences with contexts
    U[1024, 16384] (seed 5), 32 q / 8 kv heads, d 128, bf16 -- 1.1 M context tokens, 4.6 GB of K/V in a
    70k-block pool.  The cache is filled on the GPU (seeded); every sequence is checked against the float64
    statement of the oracle on its own blocks brought to the CPU, 18 of them -- the shortest and the longest
    among them -- against the slot-by-slot oracle as well, and all by the range property (an attention
    output is a convex combination of its context's V rows)."""
    rng = np.random.default_rng(5)
    S = 128
    ctx = rng.integers(1024, 16384 + 1, size=S)
    pool = int(((ctx + 15) // 16).sum()) + 64
    c = W.decode_inputs(5, S, 1024, 16384, 32, 8, 128, torch.bfloat16, pool, device=device)
    assert np.array_equal(c.context_lens.cpu().numpy(), ctx.astype(np.int32))   # the same draw as the benchmark's
    out = torch.full_like(c.q, float("nan"))
    K.paged_attention_v1(out, c.q, c.key_cache, c.value_cache, 8, c.scale, c.block_tables, c.context_lens, 16,
                         c.max_ctx)
    assert not torch.isnan(out).any()
    assert out.float().abs().max().item() <= c.value_cache.float().abs().max().item()
    rows = sorted({int(np.argmin(ctx)), int(np.argmax(ctx)), *range(0, S, 8)})
    assert len(rows) >= 16
    if "config5" not in _ORACLE_CACHE:
        want = []
        for s in rows:
            n = (int(ctx[s]) + 15) // 16
            blocks = c.block_tables[s, :n].long()
            kc, vc = c.key_cache[blocks].cpu(), c.value_cache[blocks].cpu()   # this sequence's blocks, renumbered 0..n-1
            want.append(ref.paged_attention(c.q[s:s + 1].cpu().float(), kc.float(), vc.float(), 8, c.scale,
                                            torch.arange(n, dtype=torch.int32)[None], c.context_lens[s:s + 1].cpu(), 16)[0])
        want64 = []
        for s in range(S):
            n = (int(ctx[s]) + 15) // 16
            blocks = c.block_tables[s, :n].long()
            want64.append(ref.paged_attention_fp64(c.q[s:s + 1].cpu(), c.key_cache[blocks].cpu(), c.value_cache[blocks].cpu(),
                                                   8, c.scale, torch.arange(n, dtype=torch.int32)[None],
                                                   c.context_lens[s:s + 1].cpu(), 16)[0])
        _ORACLE_CACHE["config5"] = (torch.stack(want), torch.stack(want64))
    want, want64 = _ORACLE_CACHE["config5"]
    err = (out[rows].cpu().float() - want).abs().max().item()
    assert err <= TOL[torch.bfloat16], err
    err64 = (out.cpu().double() - want64).abs().max().item()
    assert err64 <= TOL[torch.bfloat16], err64
