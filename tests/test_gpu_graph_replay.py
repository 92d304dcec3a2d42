"""The attention path under HIP graph capture: a step's calls (rotary + cache scatter, varlen prefill from
rows and from the paged cache, paged decode in both launch strategies, bias + arg-max) are captured once and
replayed with new inputs written into the same buffers; every replay must equal the eager result on the same
inputs, bit for bit.  Between replays the process does eager work and synchronises, as a serving loop would."""
import math

import pytest
import torch

from aici_amd import kernels as K
from aici_amd import workloads as W
from oracle import refkernels as ref

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("decode_launch", ["flat", "partitioned"])
def test_captured_step_replays_like_eager(device, tuning, decode_launch):
    tuning("decode_flat", 1 if decode_launch == "flat" else 0)
    dtype, Hq, Hkv, d, bs = torch.bfloat16, 32, 8, 128, 16
    g = torch.Generator().manual_seed(51)
    # prefill rows: 3 sequences with some prior context; decode rows: 40 sequences and 3
    seqs = [(300, 200), (0, 513), (1000, 64)]
    lens_k, lens_q = [a + b for a, b in seqs], [b for _, b in seqs]
    nb = sum((l + 15) // 16 for l in lens_k) + 8
    perm = torch.randperm(nb, generator=g).tolist()
    tables = torch.zeros((len(seqs), max((l + 15) // 16 for l in lens_k)), dtype=torch.int32)
    slots_new, slots_all, pos = [], [], 0
    for i, (prior, new) in enumerate(seqs):
        n = (prior + new + 15) // 16
        blocks = perm[pos:pos + n]
        pos += n
        tables[i, :n] = torch.tensor(blocks, dtype=torch.int32)
        s = W.slots_for(blocks, prior + new)
        slots_all += s
        slots_new += s[prior:]
    Tq, Tk = sum(lens_q), sum(lens_k)
    kc = torch.randn((nb, Hkv, d // 8, bs, 8), generator=g).to(dtype).to(device)
    vc = torch.randn((nb, Hkv, d, bs), generator=g).to(dtype).to(device)
    table = ref.rotary_table(d, 10000.0, 4096, dtype).to(device)
    positions = torch.cat([torch.arange(a, a + b) for a, b in seqs]).to(device)
    qkv = torch.empty((Tq, (Hq + 2 * Hkv) * d), dtype=dtype, device=device)
    q2, k2 = qkv[:, :Hq * d], qkv[:, Hq * d:(Hq + Hkv) * d]
    v3 = qkv[:, (Hq + Hkv) * d:].view(Tq, Hkv, d)
    slots_new_d = torch.tensor(slots_new, dtype=torch.int64, device=device)
    gather_d = torch.tensor(slots_all, dtype=torch.int32, device=device)
    gk = torch.empty((Tk, Hkv, d), dtype=dtype, device=device)
    gv = torch.empty_like(gk)
    cu_q, cu_k = W.offsets(lens_q).to(device), W.offsets(lens_k).to(device)
    ctx = torch.tensor(lens_k, dtype=torch.int32, device=device)
    tables_d = tables.to(device)
    scale = 1.0 / math.sqrt(d)
    dec = {S: W.decode_inputs(52 + S, S, 900, 2600, Hq, Hkv, d, dtype, S * 170, device=device) for S in (40, 3)}
    dec_out = {S: torch.empty_like(c.q) for S, c in dec.items()}
    V = 5000
    logits = torch.empty((Tq, V), dtype=dtype, device=device)
    masks = torch.randint(0, 256, (Tq, 4 * ((V + 31) // 32)), generator=g, dtype=torch.uint8).to(device)
    masks[:, 0] |= 1

    def step():
        K.rotary_embedding_and_cache(positions, q2, k2, v3, d, table, True, kc, vc, slots_new_d)
        K.gather_cached_kv(gk, gv, kc, vc, gather_d)
        q3 = q2.view(Tq, Hq, d)
        out_rows = K.flash_attn_varlen(q3, gk, gv, cu_q, cu_k, max(lens_q), max(lens_k), scale, True)
        out_paged = K.flash_attn_varlen_paged(q3, kc, vc, tables_d, cu_q, ctx, max(lens_q), max(lens_k), scale, True)
        for S, c in dec.items():
            K.paged_attention_v1(dec_out[S], c.q, c.key_cache, c.value_cache, Hkv, c.scale, c.block_tables,
                                 c.context_lens, 16, c.max_ctx)
        toks = K.bias_argmax(logits, mask=masks)
        return [out_rows, out_paged, toks]

    def fill(seed):
        gg = torch.Generator(device=device).manual_seed(seed)
        qkv.normal_(generator=gg)
        logits.normal_(generator=gg)
        for c in dec.values():
            c.q.normal_(generator=gg)

    def snapshot(outs):
        return [t.clone() for t in (qkv, kc, vc, *outs, *dec_out.values())]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fill(1)
        step()      # grows the library's scratch buffers of this stream and sets kernel attributes outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    # captured on the stream that was warmed up: the library keeps its scratch buffers per stream and
    # cannot grow one during a capture
    with torch.cuda.graph(graph, stream=side):
        graph_outs = step()
    kc0, vc0 = kc.clone(), vc.clone()
    for seed in (2, 3, 4):
        kc.copy_(kc0)
        vc.copy_(vc0)
        fill(seed)
        qkv_in = qkv.clone()
        graph.replay()
        torch.cuda.synchronize()
        got = snapshot(graph_outs)
        # eager on the same inputs (rotary works in place: restore them first), with unrelated work before it
        junk = torch.randn((512, 512), device=device) @ torch.randn((512, 512), device=device)
        kc.copy_(kc0)
        vc.copy_(vc0)
        qkv.copy_(qkv_in)
        eager_outs = step()
        torch.cuda.synchronize()
        want = snapshot(eager_outs)
        assert junk.isfinite().all()
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
