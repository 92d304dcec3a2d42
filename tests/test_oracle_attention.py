"""Pins the attention oracle (oracle/refkernels.py) without importing the reference:
the reference's own known-answer vector, an independent fp64 restatement, closed forms
and structural invariants chosen so that a dropped scale, a wrong mask alignment, a
transposed operand or a wrong GQA head mapping fails at least one of them."""
import math

import numpy as np
import pytest
import torch

from oracle import refkernels as ref
from tests.common import cu, kat_inputs, load_kat, make_cache, round4, slots_for


def test_kat_flash_numerics_model_reproduces_all_48_values():
    kat = load_kat()
    q, k, v = kat_inputs()
    cs = torch.tensor(kat["inputs"]["cu_seqlens"], dtype=torch.int32)
    y = ref.flash_numerics_model(q, k, v, cs, cs, kat["inputs"]["softmax_scale"], kat["inputs"]["causal"])
    got = round4(y.transpose(0, 1))
    want = torch.tensor(kat["expected_rounded_4"], dtype=torch.float32)
    assert got.shape == (3, 2, 8)
    assert torch.equal(got, want), (got - want).abs().max()


def test_kat_pins_layout_scale_and_noncausal_path_of_the_fp32_oracle():
    # The fp32 oracle, rounded to bf16, agrees with the printed table to within one bf16 ulp
    # everywhere (40 of 48 exactly; the other 8 are one row where the GPU's bf16-rounded
    # probabilities tip the result by one ulp): pins [total, heads, d] layout, cu_seqlens, scale.
    kat = load_kat()
    q, k, v = kat_inputs()
    cs = torch.tensor(kat["inputs"]["cu_seqlens"], dtype=torch.int32)
    y = ref.varlen_attn(q.float(), k.float(), v.float(), cs, cs, 32, 32, 0.5, causal=False)
    got = round4(y.to(torch.bfloat16).transpose(0, 1))
    want = torch.tensor(kat["expected_rounded_4"], dtype=torch.float32)
    assert (got == want).sum().item() >= 40
    assert (got - want).abs().max().item() <= 2 ** -8 + 1e-6  # one bf16 ulp below 1.0
    # and a plausible mistake is caught: dropping the scale moves values by far more
    y_bad = ref.varlen_attn(q.float(), k.float(), v.float(), cs, cs, 32, 32, 1.0, causal=False)
    assert (round4(y_bad.to(torch.bfloat16).transpose(0, 1)) != want).sum().item() > 10


@pytest.mark.parametrize("seed", range(6))
def test_sdpa_oracle_equals_independent_fp64_statement(seed):
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    b = int(rng.integers(1, 4))
    lq = rng.integers(1, 20, size=b)
    lk = lq + rng.integers(0, 24, size=b)  # Lk >= Lq: every row sees at least one key
    H, d = int(rng.choice([1, 2, 4])), int(rng.choice([8, 16, 40]))
    q = torch.randn((int(lq.sum()), H, d), generator=g)
    k = torch.randn((int(lk.sum()), H, d), generator=g)
    v = torch.randn((int(lk.sum()), H, d), generator=g)
    scale = 1.0 / math.sqrt(d)
    a = ref.varlen_attn(q, k, v, cu(lq), cu(lk), int(lq.max()), int(lk.max()), scale, True)
    b64 = ref.varlen_attn_fp64(q, k, v, cu(lq), cu(lk), scale, True)
    assert (a.double() - b64).abs().max().item() < 1e-5


def test_brute_force_triple_loop_tiny():
    # Scalar loops, no tensor algebra shared with the oracle.
    g = torch.Generator().manual_seed(11)
    lq, lk, H, d = 3, 5, 2, 4
    q, k, v = (torch.randn((n, H, d), generator=g) for n in (lq, lk, lk))
    scale = 0.37
    want = torch.zeros(lq, H, d, dtype=torch.float64)
    for i in range(lq):
        for h in range(H):
            ws = []
            for j in range(lk):
                if j <= i + (lk - lq):
                    ws.append(math.exp(scale * sum(float(q[i, h, e]) * float(k[j, h, e]) for e in range(d))))
                else:
                    ws.append(0.0)
            z = sum(ws)
            for e in range(d):
                want[i, h, e] = sum(w * float(v[j, h, e]) for j, w in enumerate(ws)) / z
    got = ref.varlen_attn(q, k, v, cu([lq]), cu([lk]), lq, lk, scale, True)
    assert (got.double() - want).abs().max().item() < 1e-6


def test_closed_forms():
    g = torch.Generator().manual_seed(3)
    H, d, L = 2, 8, 7
    q, k, v = (torch.randn((L, H, d), generator=g) for _ in range(3))
    # Lq = Lk = 1: O = V
    o = ref.varlen_attn(q[:1], k[:1], v[:1], cu([1]), cu([1]), 1, 1, 0.3, True)
    assert torch.allclose(o, v[:1], atol=1e-6)
    # causal Lq = Lk: row 0 sees only key 0
    o = ref.varlen_attn(q, k, v, cu([L]), cu([L]), L, L, 0.3, True)
    assert torch.allclose(o[0], v[0], atol=1e-6)
    # all keys equal -> uniform weights -> prefix mean of V
    k_same = k[:1].expand(L, H, d).contiguous()
    o = ref.varlen_attn(q, k_same, v, cu([L]), cu([L]), L, L, 0.3, True)
    want = torch.cumsum(v, 0) / torch.arange(1, L + 1).reshape(L, 1, 1)
    assert torch.allclose(o, want, atol=1e-5)
    # constant V -> constant output
    v_c = torch.full((L, H, d), 2.5)
    o = ref.varlen_attn(q, k, v_c, cu([L]), cu([L]), L, L, 0.3, True)
    assert torch.allclose(o, v_c, atol=1e-5)


def test_bottom_right_alignment_is_chunk_consistent():
    # A chunk of the last Lq queries against the full keys equals the last Lq rows of the
    # full causal result; a top-left aligned mask would fail this.
    g = torch.Generator().manual_seed(5)
    H, d, L, Lq = 2, 16, 23, 6
    q, k, v = (torch.randn((L, H, d), generator=g) for _ in range(3))
    full = ref.varlen_attn(q, k, v, cu([L]), cu([L]), L, L, 0.25, True)
    chunk = ref.varlen_attn(q[L - Lq:], k, v, cu([Lq]), cu([L]), Lq, L, 0.25, True)
    assert torch.allclose(chunk, full[L - Lq:], atol=1e-6)
    # both reference statements of the rule agree (refkernels.rs:102-108 vs softmax.h:159-160)
    bias = ref.causal_bias(Lq, L)
    rows = torch.arange(Lq).reshape(Lq, 1)
    cols = torch.arange(L).reshape(1, L)
    assert torch.equal(bias == 0, cols <= rows + (L - Lq))


def test_sequences_are_independent_and_ragged():
    g = torch.Generator().manual_seed(7)
    lens = [5, 1, 9]
    H, d = 3, 8
    T = sum(lens)
    q, k, v = (torch.randn((T, H, d), generator=g) for _ in range(3))
    allo = ref.varlen_attn(q, k, v, cu(lens), cu(lens), 9, 9, 0.3, True)
    off = 0
    for l in lens:
        one = ref.varlen_attn(q[off:off + l], k[off:off + l], v[off:off + l], cu([l]), cu([l]), l, l, 0.3, True)
        assert torch.allclose(allo[off:off + l], one, atol=1e-6)
        off += l
    # empty batch
    e = ref.varlen_attn(q[:0], k[:0], v[:0], cu([]), cu([]), 0, 0, 0.3, True)
    assert e.shape == (0, H, d)
    # empty sequences inside a batch, and rows without keys, in the fp64 statement
    lens2 = [4, 0, 3]
    a = ref.varlen_attn(q[:7], k[:7], v[:7], cu(lens2), cu(lens2), 4, 4, 0.3, True)
    b = ref.varlen_attn_fp64(q[:7], k[:7], v[:7], cu(lens2), cu(lens2), 0.3, True)
    assert (a.double() - b).abs().max().item() < 1e-5
    z = ref.varlen_attn_fp64(q[:5], k[:0], v[:0], cu([5]), cu([0]), 0.3, True)
    assert torch.all(z == 0)


def test_gqa_head_mapping_of_fp64_statement_matches_repeat_kv():
    g = torch.Generator().manual_seed(9)
    L, Hq, Hkv, d = 6, 8, 2, 8
    q = torch.randn((L, Hq, d), generator=g)
    k = torch.randn((L, Hkv, d), generator=g)
    v = torch.randn((L, Hkv, d), generator=g)
    a = ref.varlen_attn(q, ref.repeat_kv(k, 4), ref.repeat_kv(v, 4), cu([L]), cu([L]), L, L, 0.3, True)
    b = ref.varlen_attn_fp64(q, k, v, cu([L]), cu([L]), 0.3, True)
    assert (a.double() - b).abs().max().item() < 1e-5
    # repeat_interleave, not tile: head 1 uses kv head 0, head 4 uses kv head 1
    r = ref.repeat_kv(k, 4)
    assert torch.equal(r[:, 1], k[:, 0]) and torch.equal(r[:, 4], k[:, 1])


def _paged_setup(seed, S=3, Hq=4, Hkv=2, d=16, bs=16, pool=32):
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    ctx = rng.integers(1, 70, size=S)
    kc, vc = make_cache(pool, Hkv, d, bs, torch.float32, gen=g)
    perm = torch.randperm(pool, generator=g).tolist()
    tables, pos = [], 0
    width = int(max((c + bs - 1) // bs for c in ctx))
    for c in ctx:
        n = (int(c) + bs - 1) // bs
        tables.append(perm[pos:pos + n] + [0] * (width - n))
        pos += n
    q = torch.randn((S, Hq, d), generator=g)
    return q, kc, vc, torch.tensor(tables, dtype=torch.int32), torch.tensor(ctx, dtype=torch.int32)


def test_paged_attention_equals_dense_softmax_over_gathered_context():
    q, kc, vc, tables, ctx = _paged_setup(1)
    S, Hq, d = q.shape
    Hkv, bs = kc.shape[1], kc.shape[3]
    out = ref.paged_attention(q, kc, vc, Hkv, 0.25, tables, ctx, bs)
    for s in range(S):
        c = int(ctx[s])
        slots = slots_for(tables[s].tolist(), c, bs)
        for h in range(Hq):
            kv = h // (Hq // Hkv)
            K = torch.stack([kc[sl // bs, kv, :, sl % bs, :].reshape(-1) for sl in slots]).double()
            V = torch.stack([vc[sl // bs, kv, :, sl % bs] for sl in slots]).double()
            p = torch.softmax(K @ q[s, h].double() * 0.25, dim=0)
            assert (out[s, h].double() - p @ V).abs().max().item() < 1e-5


def test_paged_attention_fp64_statement_agrees_with_the_slot_by_slot_one():
    """The float64 whole-block statement used for full-size steps against the slot-by-slot oracle (itself
    pinned above by a per-head dense softmax), over ragged contexts including 0, 1 and block edges."""
    for seed in (1, 2, 3):
        q, kc, vc, tables, ctx = _paged_setup(seed)
        Hkv, bs = kc.shape[1], kc.shape[3]
        a = ref.paged_attention(q, kc, vc, Hkv, 0.25, tables, ctx, bs)
        b = ref.paged_attention_fp64(q, kc, vc, Hkv, 0.25, tables, ctx, bs)
        assert b.dtype == torch.float64 and (a.double() - b).abs().max().item() < 1e-5
    # a context of one token is that token's value, exactly
    q, kc, vc, tables, ctx = _paged_setup(4)
    ctx[:] = 1
    Hkv, bs = kc.shape[1], kc.shape[3]
    b = ref.paged_attention_fp64(q, kc, vc, Hkv, 0.25, tables, ctx, bs)
    for s in range(q.shape[0]):
        for h in range(q.shape[1]):
            assert torch.equal(b[s, h], vc[int(tables[s, 0]), h // (q.shape[1] // Hkv), :, 0].double())


def test_paged_attention_invariant_under_block_permutation_and_equals_prefill_last_row():
    q, kc, vc, tables, ctx = _paged_setup(2)
    Hkv, bs = kc.shape[1], kc.shape[3]
    out = ref.paged_attention(q, kc, vc, Hkv, 0.25, tables, ctx, bs)
    # move every physical block somewhere else
    pool = kc.shape[0]
    perm = torch.randperm(pool, generator=torch.Generator().manual_seed(99))
    kc2, vc2 = torch.empty_like(kc), torch.empty_like(vc)
    kc2[perm] = kc
    vc2[perm] = vc
    tables2 = perm[tables.long()].to(torch.int32)
    out2 = ref.paged_attention(q, kc2, vc2, Hkv, 0.25, tables2, ctx, bs)
    assert torch.equal(out, out2)
    # last row of a causal prefill over the same keys
    s = 0
    c = int(ctx[s])
    slots = torch.tensor(slots_for(tables[s].tolist(), c, bs), dtype=torch.int32)
    kk = torch.empty((c, Hkv, q.shape[2]))
    vv = torch.empty_like(kk)
    ref.gather_cached_kv(kk, vv, kc, vc, slots)
    n_rep = q.shape[1] // Hkv
    qq = torch.randn((c, q.shape[1], q.shape[2]), generator=torch.Generator().manual_seed(4))
    qq[-1] = q[s]
    full = ref.varlen_attn(qq, ref.repeat_kv(kk, n_rep), ref.repeat_kv(vv, n_rep), cu([c]), cu([c]), c, c, 0.25, True)
    assert torch.allclose(full[-1], out[s], atol=1e-6)


def test_sliding_window_special_cases_and_triple_loop():
    """The window of mha_varlen_fwd_C (softmax.h:155-166) in the fp64 statement: open = unmasked,
    (-1, 0) = causal, causal overrides the right bound, (0, 0) = exactly one key per row, a window
    wider than the sequence = no window, and a scalar triple loop over a chunk with prior context."""
    g = torch.Generator().manual_seed(31)
    lq, lk, H, d = 5, 9, 2, 4
    q = torch.randn((lq, H, d), generator=g)
    k, v = (torch.randn((lk, H, d), generator=g) for _ in range(2))
    a = dict(seqlens_q=cu([lq]), seqlens_k=cu([lk]), softmax_scale=0.41)
    f = lambda causal, window: ref.varlen_attn_fp64(q, k, v, causal=causal, window=window, **a)
    assert torch.equal(f(False, (-1, -1)), ref.varlen_attn_fp64(q, k, v, causal=False, **a))
    assert torch.equal(f(False, (-1, 0)), f(True, (-1, -1)))
    assert torch.equal(f(True, (-1, 3)), f(True, (-1, -1)))
    assert torch.equal(f(False, (100, 100)), f(False, (-1, -1)))
    assert torch.equal(f(True, (100, -1)), f(True, (-1, -1)))
    one = f(False, (0, 0))  # row i sees only key i + (lk - lq)
    assert torch.allclose(one, v[lk - lq:].double(), atol=1e-12)
    for causal, (wl, wr) in [(False, (2, 1)), (True, (3, -1)), (False, (-1, 2)), (False, (1, -1)), (False, (0, 3))]:
        want = torch.zeros(lq, H, d, dtype=torch.float64)
        for i in range(lq):
            for h in range(H):
                ws = []
                for j in range(lk):
                    hi_ok = True if (wr < 0 and not causal) else j <= i + (lk - lq) + (0 if causal else wr)
                    lo_ok = True if wl < 0 else j >= i + (lk - lq) - wl
                    ws.append(math.exp(0.41 * sum(float(q[i, h, e]) * float(k[j, h, e]) for e in range(d)))
                              if hi_ok and lo_ok else 0.0)
                z = sum(ws)
                for e in range(d):
                    want[i, h, e] = sum(w * float(v[j, h, e]) for j, w in enumerate(ws)) / z if z > 0 else 0.0
        assert (f(causal, (wl, wr)) - want).abs().max().item() < 1e-12, (causal, wl, wr)
    # more queries than keys: rows whose window lies before key 0 give zeros
    q2 = torch.randn((6, H, d), generator=g)
    o = ref.varlen_attn_fp64(q2, k[:2], v[:2], cu([6]), cu([2]), 0.41, causal=False, window=(1, 0))
    assert torch.all(o[:3] == 0) and not torch.all(o[4] == 0)
