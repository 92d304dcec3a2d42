"""reshape_and_cache / gather_cached_kv / copy_blocks / swap_blocks through the C ABI against
the oracle: bit-exact."""
import pytest
import torch

from aici_amd import kernels as K
from aici_amd import workloads as W
from aici_amd._lib import HipAttnError
from oracle import refkernels as ref
from tests.common import make_cache

pytestmark = pytest.mark.gpu


def bits(t: torch.Tensor) -> torch.Tensor:
    return t.cpu().contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("slot_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("strided", [False, True])
def test_reshape_and_cache_and_gather_bit_exact(device, dtype, slot_dtype, strided):
    g = torch.Generator().manual_seed(1)
    T, H, d, bs, nb = 150, 5, 80, 16, 24
    if strided:  # k and v as chunks of a fused [T, 3, H, d] projection, as rLLM's Phi layer passes them
        qkv = torch.randn((T, 3, H, d), generator=g).to(dtype)
        key, value = qkv[:, 1], qkv[:, 2]
    else:
        key = torch.randn((T, H, d), generator=g).to(dtype)
        value = torch.randn((T, H, d), generator=g).to(dtype)
    kc, vc = make_cache(nb, H, d, bs, dtype, fill=-3.0)
    slots = torch.randperm(nb * bs, generator=g)[:T].to(slot_dtype)
    slots[7] = -1
    slots[T - 1] = -5
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ref.reshape_and_cache(key, value, kc_ref, vc_ref, slots)
    kd, vd = kc.to(device), vc.to(device)
    if strided:
        qkv_d = qkv.to(device)
        key_d, value_d = qkv_d[:, 1], qkv_d[:, 2]
    else:
        key_d, value_d = key.to(device), value.to(device)
    if slot_dtype == torch.int64:
        K.reshape_and_cache(key_d, value_d, kd, vd, slots.to(device))
    else:  # int32 straight through the ABI (the Python mirror widens; the ABI accepts both)
        from aici_amd.kernels import _desc, _stream, call
        call("hipattn_reshape_and_cache", _desc(key_d), _desc(value_d), _desc(kd), _desc(vd),
             _desc(slots.to(device)), _stream(key_d))
    assert torch.equal(bits(kd), bits(kc_ref)) and torch.equal(bits(vd), bits(vc_ref))
    valid = slots >= 0
    n = int(valid.sum())
    ko = torch.zeros((n, H, d), dtype=dtype, device=device)
    vo = torch.zeros_like(ko)
    gslots = slots[valid].to(torch.int32 if slot_dtype == torch.int32 else torch.int64)
    K.gather_cached_kv(ko, vo, kd, vd, gslots.to(device))
    assert torch.equal(bits(ko), bits(key[valid])) and torch.equal(bits(vo), bits(value[valid]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("strided", [False, True])
@pytest.mark.parametrize("d,first", [(96, 512), (128, 512),      # the register-tile kernel (under 16384 tokens)
                                     (128, 16000), (64, 16000),   # the LDS-tile kernel
                                     (96, 16000), (80, 16000)])   # ... with a partial last chunk group per head
def test_long_inputs_runs_of_tokens_mixed_with_everything_else(device, dtype, strided, d, first):
    """More than 1024 tokens: the kernels move aligned runs of 8 tokens as tiles and fall back per
    token elsewhere.  The slot list mixes prompts that fill permuted blocks in order (lengths not
    multiples of 8, so runs straddle sequences), a prompt that starts in the middle of a block,
    padding slots inside a run, decode-like random slots, a slot past the cache and a ragged tail."""
    g = torch.Generator().manual_seed(7)
    H, bs, nb = 4, 16, 1200
    perm = torch.randperm(nb, generator=g).tolist()
    slots = []

    def prompt(n, start_off=0):
        need = (start_off + n + bs - 1) // bs
        blocks = [perm.pop() for _ in range(need)]
        slots.extend(blocks[(start_off + t) // bs] * bs + (start_off + t) % bs for t in range(n))

    prompt(first)
    prompt(203)
    prompt(77, start_off=5)
    prompt(256)
    free = [b * bs + o for b in perm[:20] for o in range(bs)]
    pick = torch.randperm(len(free), generator=g)[:150].tolist()
    slots.extend(free[i] for i in pick)              # decode-like: unrelated slots
    del perm[:20]
    prompt(131)
    slots[40] = -1                                   # padding inside a run
    slots[520] = nb * bs + 3                         # outside the cache: dropped
    T = len(slots)
    assert T >= 1024 and T % 8 != 0
    slots_t = torch.tensor(slots, dtype=torch.int64)
    if strided:
        qkv = torch.randn((T, 3, H, d), generator=g).to(dtype)
        key, value = qkv[:, 1], qkv[:, 2]
    else:
        key = torch.randn((T, H, d), generator=g).to(dtype)
        value = torch.randn((T, H, d), generator=g).to(dtype)
    kc, vc = make_cache(nb, H, d, bs, dtype, fill=-3.0)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ok = (slots_t >= 0) & (slots_t < nb * bs)
    ref.reshape_and_cache(key[ok], value[ok], kc_ref, vc_ref, slots_t[ok])
    kd, vd = kc.to(device), vc.to(device)
    src = qkv.to(device) if strided else None
    key_d, value_d = (src[:, 1], src[:, 2]) if strided else (key.to(device), value.to(device))
    K.reshape_and_cache(key_d, value_d, kd, vd, slots_t.to(device))
    assert torch.equal(bits(kd), bits(kc_ref)) and torch.equal(bits(vd), bits(vc_ref))
    # gather through the same list (invalid slots leave their output rows untouched)
    ko = torch.full((T, H, d), 9.0, dtype=dtype, device=device)
    vo = torch.full_like(ko, 9.0)
    K.gather_cached_kv(ko, vo, kd, vd, slots_t.to(torch.int32).to(device))
    want_k, want_v = key.clone(), value.clone()
    want_k[~ok], want_v[~ok] = 9.0, 9.0
    assert torch.equal(bits(ko), bits(want_k)) and torch.equal(bits(vo), bits(want_v))


def test_config1_scatter_bit_exact(device):
    p, extra = W.config1()
    nb = extra["pool_blocks"]
    kc, vc = make_cache(nb, 32, 128, 16, torch.float16, fill=0.5)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    ref.reshape_and_cache(p.k, p.v, kc_ref, vc_ref, extra["slot_mapping"])
    kd, vd = kc.to(device), vc.to(device)
    K.reshape_and_cache(p.k.to(device), p.v.to(device), kd, vd, extra["slot_mapping"].to(device))
    assert torch.equal(bits(kd), bits(kc_ref)) and torch.equal(bits(vd), bits(vc_ref))
    # 80 of the 128 blocks are used; the others still hold the fill value
    used = torch.unique(extra["slot_mapping"] // 16)
    assert used.numel() == 80
    mask = torch.ones(nb, dtype=torch.bool)
    mask[used.long()] = False
    assert torch.all(kd.cpu()[mask] == 0.5) and torch.all(vd.cpu()[mask] == 0.5)


def test_empty_and_out_of_range(device):
    kc, vc = make_cache(4, 2, 64, 16, torch.bfloat16, fill=1.0)
    kd, vd = kc.to(device), vc.to(device)
    e = torch.zeros((0, 2, 64), dtype=torch.bfloat16, device=device)
    K.reshape_and_cache(e, e, kd, vd, torch.zeros((0,), dtype=torch.int64, device=device))
    K.gather_cached_kv(e, e, kd, vd, torch.zeros((0,), dtype=torch.int32, device=device))
    # a slot beyond the cache is dropped instead of written out of bounds
    one = torch.ones((1, 2, 64), dtype=torch.bfloat16, device=device) * 9
    K.reshape_and_cache(one, one, kd, vd, torch.tensor([4 * 16 + 3], dtype=torch.int64, device=device))
    torch.cuda.synchronize()
    assert torch.all(kd.cpu() == 1.0) and torch.all(vd.cpu() == 1.0)


def test_argument_errors(device):
    kc, vc = make_cache(4, 2, 64, 16, torch.float16)
    kd, vd = kc.to(device), vc.to(device)
    k = torch.zeros((3, 2, 64), dtype=torch.float16, device=device)
    s = torch.zeros((3,), dtype=torch.int64, device=device)
    with pytest.raises(HipAttnError, match="dtype must match"):
        K.reshape_and_cache(k.to(torch.bfloat16), k.to(torch.bfloat16), kd, vd, s)
    with pytest.raises(HipAttnError, match="heads of size"):
        K.reshape_and_cache(k[:, :1], k[:, :1], kd, vd, s)
    with pytest.raises(HipAttnError, match="slot_mapping has"):
        K.reshape_and_cache(k, k, kd, vd, s[:2])
    with pytest.raises(HipAttnError, match="GPU tensor"):
        K.reshape_and_cache(k.cpu(), k, kd, vd, s)


def test_copy_blocks_and_swap_blocks(device):
    g = torch.Generator().manual_seed(5)
    layers = 3
    caches = [make_cache(10, 2, 64, 16, torch.bfloat16, gen=g) for _ in range(layers)]
    kcs = [c[0].clone() for c in caches]
    vcs = [c[1].clone() for c in caches]
    mapping = {1: [4, 5], 2: [0], 9: [8]}
    kd = [k.to(device) for k in kcs]
    vd = [v.to(device) for v in vcs]
    K.copy_blocks(kd, vd, mapping)
    ref.copy_blocks(kcs, vcs, mapping)
    for l in range(layers):
        assert torch.equal(bits(kd[l]), bits(kcs[l])) and torch.equal(bits(vd[l]), bits(vcs[l]))
    K.copy_blocks(kd, vd, {})  # no pairs: no launch
    # swap out blocks 3,4 to a pinned host cache at 0,1 and back in at 6,7
    host = torch.zeros((4,) + tuple(kd[0].shape[1:]), dtype=torch.bfloat16).pin_memory()
    K.swap_blocks(kd[0], host, {3: 0, 4: 1})
    torch.cuda.synchronize()
    assert torch.equal(bits(host[0]), bits(kcs[0][3])) and torch.equal(bits(host[1]), bits(kcs[0][4]))
    K.swap_blocks(host, kd[0], {0: 6, 1: 7})
    torch.cuda.synchronize()
    assert torch.equal(bits(kd[0][6]), bits(kcs[0][3])) and torch.equal(bits(kd[0][7]), bits(kcs[0][4]))
    with pytest.raises(HipAttnError, match="out of range"):
        K.swap_blocks(kd[0], host, {3: 99})


def test_cache_engine_swap_round_trip_and_copy(device):
    """cache_engine.rs:40-175 end to end: swap blocks out to the host caches and back in on the side
    stream, the per-layer events ordering the compute stream behind them; copy-on-write copies; sizes."""
    from aici_amd import paged

    layers, Hkv, d, BS, dt = 3, 2, 64, 16, torch.bfloat16
    eng = paged.CacheEngine(layers, Hkv, d, BS, dt, num_gpu_blocks=12, num_cpu_blocks=4, device=device)
    assert eng.gpu_cache[0][0].shape == (12, Hkv, d // 8, BS, 8) and eng.gpu_cache[0][1].shape == (12, Hkv, d, BS)
    assert eng.cpu_cache[1][0].shape == (4, Hkv, d // 8, BS, 8) and eng.cpu_cache[1][0].is_pinned()
    assert paged.CacheEngine.get_cache_block_size(BS, Hkv, d, layers, dt) == 2 * BS * Hkv * d * 2 * layers
    g = torch.Generator().manual_seed(9)
    want = []
    for k, v in eng.gpu_cache:
        kc = torch.randn(k.shape, generator=g).to(dt)
        vc = torch.randn(v.shape, generator=g).to(dt)
        k.copy_(kc)
        v.copy_(vc)
        want.append((kc, vc))
    torch.cuda.synchronize()
    get = eng.get_cache_iface()          # no swap issued yet: plain access
    assert get(1)[0] is eng.gpu_cache[1][0]
    eng.swap_out({3: 0, 7: 2})
    eng.swap_in({0: 10, 2: 11})
    get = eng.get_cache_iface()          # waits for each layer's swap on the current stream
    for l in range(layers):
        k, v = get(l)
        kk, vv = k.clone(), v.clone()    # ordered behind the layer's event on the current stream
        torch.cuda.synchronize()
        assert torch.equal(bits(kk[10]), bits(want[l][0][3])) and torch.equal(bits(kk[11]), bits(want[l][0][7]))
        assert torch.equal(bits(vv[10]), bits(want[l][1][3])) and torch.equal(bits(vv[11]), bits(want[l][1][7]))
        assert torch.equal(bits(eng.cpu_cache[l][0][0]), bits(want[l][0][3]))
        assert torch.equal(bits(kk[:10]), bits(want[l][0][:10]))
    eng.new_round()
    assert eng.used_events is False
    eng.copy({3: [0, 1], 7: [2]})
    torch.cuda.synchronize()
    for l in range(layers):
        k, v = eng.gpu_cache[l]
        assert torch.equal(bits(k[0]), bits(want[l][0][3])) and torch.equal(bits(k[1]), bits(want[l][0][3]))
        assert torch.equal(bits(v[2]), bits(want[l][1][7]))


def test_swapped_out_sequence_decodes_the_same_after_swap_in(device):
    """BlockSpaceManager + CacheEngine together (scheduler.rs preemption by swapping): a sequence's
    blocks go to the host caches, its device blocks are reused by another sequence, it comes back into
    different blocks, and paged attention over it gives the same bits as before."""
    from aici_amd import paged

    Hq, Hkv, d, BS, dt = 8, 2, 64, 16, torch.float16
    g = torch.Generator().manual_seed(77)
    mgr = paged.BlockSpaceManager(BS, 12, 8, watermark=0.0)
    eng = paged.CacheEngine(1, Hkv, d, BS, dt, num_gpu_blocks=12, num_cpu_blocks=8, device=device)
    kc, vc = eng.gpu_cache[0]
    kc.zero_()
    vc.zero_()
    ctx = 5 * BS + 3
    mgr.allocate(1, ctx)
    k = torch.randn((ctx, Hkv, d), generator=g).to(dt).to(device)
    v = torch.randn((ctx, Hkv, d), generator=g).to(dt).to(device)
    slots = torch.from_numpy(mgr.gpu_allocator.get_block_idxes(1, ctx)).to(device)
    K.reshape_and_cache(k, v, kc, vc, slots)
    q = torch.randn((1, Hq, d), generator=g).to(dt).to(device)

    def decode():
        blocks = mgr.gpu_allocator.get_block_idxes(1, ctx)[::BS] // BS
        tables = torch.tensor([blocks.tolist()], dtype=torch.int32, device=device)
        out = torch.empty_like(q)
        K.paged_attention_v1(out, q, kc, vc, Hkv, d ** -0.5, tables, torch.tensor([ctx], dtype=torch.int32, device=device),
                             BS, ctx)
        return out.cpu(), blocks.tolist()

    before, blocks_before = decode()
    assert mgr.can_swap_out([1])
    eng.swap_out(mgr.swap_out([1]))
    torch.cuda.synchronize()
    mgr.allocate(2, 4 * BS)                                  # takes some of the blocks sequence 1 had
    taken = mgr.gpu_allocator.get_block_idxes(2, 4 * BS)
    K.reshape_and_cache(torch.ones((4 * BS, Hkv, d), dtype=dt, device=device), torch.ones((4 * BS, Hkv, d), dtype=dt, device=device),
                        kc, vc, torch.from_numpy(taken).to(device))
    assert set((taken[::BS] // BS).tolist()) & set(blocks_before)
    assert mgr.can_swap_in([1])
    eng.new_round()
    eng.swap_in(mgr.swap_in([1]))
    kc2, vc2 = eng.get_cache_iface()(0)                      # orders the current stream behind the swap
    assert kc2 is kc
    after, blocks_after = decode()
    assert blocks_after != blocks_before
    assert torch.equal(bits(after), bits(before))


@pytest.mark.parametrize("case", [
    (torch.bfloat16, 32, 8, 128, 128, True, torch.int64),    # Llama: the fused kernel
    (torch.float16, 32, 32, 80, 32, True, torch.int32),      # Phi-2: rot_dim < d, pass-through chunks
    (torch.float16, 8, 2, 64, 64, False, torch.int64),       # GPT-J pairing: the two calls behind the entry point
    (torch.float32, 4, 4, 64, 64, True, torch.int64),        # fp32: likewise
    (torch.bfloat16, 4, 1, 96, 48, True, torch.int64),       # rot_dim not a multiple of 16: likewise
])
def test_rotary_and_cache_equals_the_two_calls(device, case):
    """hipattn_rotary_embedding_and_cache against the oracle's rotary_embedding + reshape_and_cache, bit for
    bit, on strided q/k/v (chunks of one fused QKV row), with padding slots, a slot past the cache and
    positions outside the table."""
    dtype, Hq, Hkv, d, rot, neox, slot_dtype = case
    g = torch.Generator().manual_seed(41)
    T, bs, nb, max_pos = 150, 16, 24, 500
    qkv = torch.randn((T, (Hq + 2 * Hkv) * d), generator=g).to(dtype)
    q, k, v = qkv[:, :Hq * d], qkv[:, Hq * d:(Hq + Hkv) * d], qkv[:, (Hq + Hkv) * d:].view(T, Hkv, d)
    pos = torch.randint(0, max_pos, (T,), generator=g)
    pos[7], pos[8] = max_pos + 3, -1                       # outside the table: rows left as they are
    slots = torch.randperm(nb * bs, generator=g)[:T].to(torch.int64)
    slots[11], slots[12] = -1, nb * bs + 5                 # not cached
    table = ref.rotary_table(rot, 10000.0, max_pos, dtype)
    kc, vc = make_cache(nb, Hkv, d, bs, dtype, fill=-2.0)
    # oracle: rotate (valid positions only), then scatter (valid slots only)
    q_ref, k_ref = q.clone(), k.clone()
    okp = (pos >= 0) & (pos < max_pos)
    qr, kr = q_ref[okp].clone(), k_ref[okp].clone()
    ref.rotary_embedding(pos[okp], qr, kr, d, table, neox)
    q_ref[okp], k_ref[okp] = qr, kr
    kc_ref, vc_ref = kc.clone(), vc.clone()
    oks = (slots >= 0) & (slots < nb * bs)
    ref.reshape_and_cache(k_ref.view(T, Hkv, d)[oks], v[oks], kc_ref, vc_ref, slots[oks])
    qkv_d = qkv.to(device)
    qd, kd = qkv_d[:, :Hq * d], qkv_d[:, Hq * d:(Hq + Hkv) * d]
    vd = qkv_d[:, (Hq + Hkv) * d:].view(T, Hkv, d)
    kcd, vcd = kc.to(device), vc.to(device)
    K.rotary_embedding_and_cache(pos.to(device), qd, kd, vd, d, table.to(device), neox, kcd, vcd,
                                 slots.to(slot_dtype).to(device))
    assert torch.equal(bits(qd), bits(q_ref)) and torch.equal(bits(kd), bits(k_ref))
    assert torch.equal(bits(kcd), bits(kc_ref)) and torch.equal(bits(vcd), bits(vc_ref))
    assert torch.equal(bits(vd), bits(v))
