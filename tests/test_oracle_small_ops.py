"""Pins the data-movement, rotary, norm, activation and AICI-bias oracles with closed
forms, round trips and hand-computed cases."""
import math

import numpy as np
import pytest
import torch

from oracle import aici
from oracle import refkernels as ref
from tests.common import make_cache


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_reshape_and_cache_closed_form_and_round_trip(dtype):
    g = torch.Generator().manual_seed(0)
    T, H, d, bs, nb = 37, 3, 16, 16, 8
    key = torch.randn((T, H, d), generator=g).to(dtype)
    value = torch.randn((T, H, d), generator=g).to(dtype)
    sentinel = 7.0
    kc, vc = make_cache(nb, H, d, bs, dtype, fill=sentinel)
    x = kc.shape[4]
    slots = torch.randperm(nb * bs, generator=g)[:T].to(torch.int32)
    slots[5] = -1  # padding token: skipped
    ref.reshape_and_cache(key, value, kc, vc, slots)
    # closed-form index formulas of cache_kernels.cu:201-211
    for t in [0, 1, 17, 36]:
        s = int(slots[t])
        b, o = s // bs, s % bs
        for h in range(H):
            for j in range(d):
                assert kc[b, h, j // x, o, j % x] == key[t, h, j]
                assert vc[b, h, j, o] == value[t, h, j]
    # untouched slots keep the sentinel; exactly (T-1)*H*d elements changed in each cache
    assert (kc != sentinel).sum().item() <= (T - 1) * H * d
    used = torch.zeros(nb * bs, dtype=torch.bool)
    used[slots[slots >= 0].long()] = True
    kview = kc.permute(0, 3, 1, 2, 4).reshape(nb * bs, H, d)  # [slot, H, d]
    vview = vc.permute(0, 3, 1, 2).reshape(nb * bs, H, d)
    assert torch.all(kview[~used] == sentinel) and torch.all(vview[~used] == sentinel)
    # gather(reshape(x)) == x, bit-exact
    valid = slots >= 0
    k2 = torch.zeros((int(valid.sum()), H, d), dtype=dtype)
    v2 = torch.zeros_like(k2)
    ref.gather_cached_kv(k2, v2, kc, vc, slots[valid])
    assert torch.equal(k2, key[valid]) and torch.equal(v2, value[valid])


def test_copy_blocks():
    g = torch.Generator().manual_seed(1)
    kcs, vcs = zip(*[make_cache(6, 2, 16, 16, torch.float16, gen=g) for _ in range(3)])
    kcs, vcs = [k.clone() for k in kcs], [v.clone() for v in vcs]
    k0, v0 = [k.clone() for k in kcs], [v.clone() for v in vcs]
    ref.copy_blocks(kcs, vcs, {1: [4, 5], 2: [0]})
    for l in range(3):
        assert torch.equal(kcs[l][4], k0[l][1]) and torch.equal(kcs[l][5], k0[l][1]) and torch.equal(kcs[l][0], k0[l][2])
        assert torch.equal(vcs[l][4], v0[l][1]) and torch.equal(vcs[l][0], v0[l][2])
        assert torch.equal(kcs[l][3], k0[l][3])


def test_rotary_table_and_closed_form_neox():
    rot, theta, L = 8, 10000.0, 50
    tab = ref.rotary_table(rot, theta, L, torch.float32)
    assert tab.shape == (L, rot)
    for pos in [0, 1, 17, 49]:
        for i in range(rot // 2):
            ang = pos * (1.0 / theta ** (2 * i / rot))
            assert abs(float(tab[pos, i]) - math.cos(ang)) < 1e-4
            assert abs(float(tab[pos, rot // 2 + i]) - math.sin(ang)) < 1e-4
    g = torch.Generator().manual_seed(2)
    T, Hq, Hkv, d = 5, 3, 1, 12  # rot < d: tail passes through
    q = torch.randn((T, Hq * d), generator=g)
    k = torch.randn((T, Hkv * d), generator=g)
    pos = torch.tensor([0, 3, 7, 49, 1], dtype=torch.int64)
    q0, k0 = q.clone(), k.clone()
    ref.rotary_embedding(pos, q, k, d, tab, True)
    qv, q0v = q.view(T, Hq, d), q0.view(T, Hq, d)
    for t in range(T):
        for h in range(Hq):
            for i in range(rot // 2):
                c, s = float(tab[pos[t], i]), float(tab[pos[t], rot // 2 + i])
                x, y = float(q0v[t, h, i]), float(q0v[t, h, i + rot // 2])
                assert abs(float(qv[t, h, i]) - (x * c - y * s)) < 1e-6
                assert abs(float(qv[t, h, i + rot // 2]) - (y * c + x * s)) < 1e-6
    assert torch.equal(qv[:, :, rot:], q0v[:, :, rot:])           # pass-through tail
    assert torch.equal(q[0], q0[0]) and torch.equal(k[0], k0[0])   # position 0 = identity
    # rotation preserves the norm of the rotated part
    assert torch.allclose(qv[:, :, :rot].norm(dim=-1), q0v[:, :, :rot].norm(dim=-1), atol=1e-5)


def test_rotary_gptj_pairs():
    rot, L = 4, 10
    tab = ref.rotary_table(rot, 100.0, L, torch.float32)
    q = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    k = q.clone()
    ref.rotary_embedding(torch.tensor([3]), q, k, 4, tab, False)
    c0, c1, s0, s1 = (float(tab[3, i]) for i in range(4))
    want = [1 * c0 - 2 * s0, 2 * c0 + 1 * s0, 3 * c1 - 4 * s1, 4 * c1 + 3 * s1]
    assert torch.allclose(q[0], torch.tensor(want), atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_closed_form_and_rounding_order(dtype):
    g = torch.Generator().manual_seed(3)
    x = torch.randn((4, 64), generator=g).to(dtype)
    w = torch.randn((64,), generator=g).to(dtype)
    eps = 1e-5
    got = ref.rms_norm(x, w, eps)
    xd = x.double()
    inv = 1.0 / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps)
    normed = (xd * inv).to(dtype)          # rounded BEFORE the weight multiply
    want = (normed.double() * w.double()).to(dtype)
    assert got.dtype == dtype
    tol = 0 if dtype == torch.float32 else 0
    assert (got.double() - want.double()).abs().max().item() <= (1e-6 if dtype == torch.float32 else 2 ** -7 * 8)
    if dtype == torch.bfloat16:
        assert (got == want).float().mean().item() > 0.98
    # fused variant: residual = x + r, input = norm(residual) * w
    r = torch.randn((4, 64), generator=g).to(dtype)
    xi, ri = x.clone(), r.clone()
    ref.fused_add_rms_norm(xi, ri, w, eps)
    assert torch.equal(ri, (x.float() + r.float()).to(dtype))
    assert (xi.float() - ref.rms_norm(ri, w, eps).float()).abs().max().item() <= 2 ** -6 * 8


def test_activations_closed_form_fp32():
    x = torch.linspace(-4, 4, 33)
    a = ref.silu_and_mul(torch.cat([x, 2 * x]).reshape(1, -1))
    assert torch.allclose(a[0], x * torch.sigmoid(x) * 2 * x, atol=1e-6)
    want = 0.5 * x * (1 + torch.tanh(0.79788456 * (x + 0.044715 * x ** 3)))
    assert torch.allclose(ref.gelu_new(x), want, atol=1e-6)
    assert torch.allclose(ref.gelu_fast(x), want, atol=1e-6)


def test_aici_mask_bit_order_and_bias():
    V = 70
    allowed = np.zeros(V, dtype=bool)
    allowed[[0, 9, 31, 32, 69]] = True
    packed = aici.pack_allowed(allowed)
    assert packed.shape[0] == aici.mask_bytes_for(V) == 12
    # token 9 = byte 1 bit 1; token 31 = byte 3 bit 7; token 69 = byte 8 bit 5
    assert packed[0] == 1 and packed[1] == 2 and packed[3] == 0x80 and packed[4] == 1 and packed[8] == 0x20
    row = aici.apply_to_slice(packed, aici.bias_row_len(V))
    assert row.shape[0] == (V + 1000) & ~63
    assert np.array_equal(np.nonzero(row == 0.0)[0], np.array([0, 9, 31, 32, 69]))
    assert np.all(np.isneginf(row[row != 0.0]))
    assert np.array_equal(row, aici.apply_to_slice_fast(packed, aici.bias_row_len(V)))
    logits = torch.arange(V, dtype=torch.float32).reshape(1, V)  # increasing: unbiased argmax = V-1
    tok = aici.biased_argmax(logits, torch.from_numpy(row).reshape(1, -1))
    assert tok.item() == 69
    logits[0, 9] = 1000.0
    assert aici.biased_argmax(logits, torch.from_numpy(row).reshape(1, -1)).item() == 9


# ---- sampling (tmodel.rs:172-194, 236-268): pinned by what the procedure reduces to in special cases -------

def test_nucleus_weights_hand_case_and_brute_force():
    # sorted: 0.4 (id 2), 0.3 (id 0), 0.2 (id 3), 0.1 (id 1).  top_p 0.65: 0.4 kept (before: 0), 0.3 kept
    # (before: 0.4 < 0.65), 0.2 dropped (before: 0.7 >= 0.65)
    prs = np.array([0.3, 0.1, 0.4, 0.2], dtype=np.float32)
    assert aici.nucleus_weights(prs, 0.65).tolist() == [np.float32(0.3), 0.0, np.float32(0.4), 0.0]
    # a token is kept exactly when the mass before it is below top_p: 0.7 itself keeps the third
    assert np.count_nonzero(aici.nucleus_weights(prs, 0.7000001)) == 3
    # equal values: the stable sort takes the lower ids first
    tie = np.array([0.25, 0.25, 0.25, 0.25], dtype=np.float32)
    assert aici.nucleus_weights(tie, 0.5).tolist() == [0.25, 0.25, 0.0, 0.0]
    assert aici.nucleus_weights(tie, 0.51).tolist() == [0.25, 0.25, 0.25, 0.0]
    # brute force on random small distributions: the kept set is the shortest prefix of the sorted order
    # whose mass reaches top_p
    rng = np.random.default_rng(0)
    for _ in range(200):
        n = int(rng.integers(2, 12))
        p = rng.random(n).astype(np.float32)
        p /= p.sum()
        top_p = float(rng.uniform(0.05, 0.95))
        kept = aici.nucleus_weights(p, top_p)
        order = sorted(range(n), key=lambda i: (-p[i], i))
        want, mass = np.zeros(n, dtype=np.float32), np.float32(0.0)
        for i in order:
            if mass >= np.float32(top_p):
                break
            want[i] = p[i]
            mass = np.float32(mass + p[i])
        assert np.array_equal(kept, want)


def test_weighted_index_is_the_inverse_cdf():
    w = np.array([0.0, 2.0, 0.0, 1.0, 1.0], dtype=np.float32)   # cumulative 0 2 2 3 4
    assert [aici.weighted_index(w, u) for u in (0.0, 0.49, 0.5, 0.74, 0.75, 0.999)] == [1, 1, 3, 3, 4, 4]
    # a zero weight is never drawn, whatever u
    assert all(aici.weighted_index(w, u) in (1, 3, 4) for u in np.linspace(0, 0.9999, 1000))
    # frequencies over an even grid of u follow the weights
    p = np.array([0.1, 0.2, 0.3, 0.4], dtype=np.float32)
    draws = np.array([aici.weighted_index(p, u) for u in (np.arange(10000) + 0.5) / 10000])
    assert np.allclose(np.bincount(draws, minlength=4) / 10000, p, atol=2e-4)


def test_sample_reduces_to_known_procedures():
    g = torch.Generator().manual_seed(3)
    V = 500
    logits = torch.randn((V,), generator=g) * 3
    bias = torch.zeros((aici.bias_row_len(V),))
    bias[::3] = float("-inf")
    allowed = torch.isfinite(bias[:V])
    greedy = int((logits + bias[:V]).argmax())
    # temperature below SAMPLING_EPS is the arg-max; a sharp temperature or a tiny nucleus gives it too
    assert aici.sample(logits, bias, 0.0, 0.9, 0.37) == greedy
    assert all(aici.sample(logits, bias, 1e-3, 1.0, u) == greedy for u in (0.0, 0.5, 0.999))
    assert all(aici.sample(logits, bias, 1.0, 1e-6, u) == greedy for u in (0.0, 0.5, 0.999))
    # top_p = 1 (or 0): plain sampling -- over an even grid of u the frequencies are the softmax, and no
    # disallowed token is ever drawn
    p = torch.softmax((logits + bias[:V]) / 0.8, 0).numpy()
    n = 20000
    draws = np.array([aici.sample(logits, bias, 0.8, 1.0, u) for u in (np.arange(n) + 0.5) / n])
    assert allowed[draws].all()
    assert np.abs(np.bincount(draws, minlength=V) / n - p).max() < 1.5 / n + 1e-6
    # with a nucleus the draws stay inside the kept set and follow its renormalised weights
    kept = aici.nucleus_weights(p, 0.6)
    draws = np.array([aici.sample(logits, bias, 0.8, 0.6, u) for u in (np.arange(n) + 0.5) / n])
    assert (kept[draws] > 0).all() and 0.6 <= kept.sum() < 0.6 + p.max()
    assert np.abs(np.bincount(draws, minlength=V) / n - kept / kept.sum()).max() < 1.5 / n + 1e-6


def test_linear_against_a_triple_loop_and_closed_forms():
    g = torch.Generator().manual_seed(11)
    M, N, Kd = 5, 7, 6
    # small integers: every product and sum is exact in any float type, so the comparison is exact
    x = torch.randint(-4, 5, (M, Kd), generator=g).float()
    w = torch.randint(-4, 5, (N, Kd), generator=g).float()
    b = torch.randint(-4, 5, (N,), generator=g).float()
    want = torch.zeros((M, N), dtype=torch.float64)
    for i in range(M):
        for j in range(N):
            acc = 0.0
            for k in range(Kd):
                acc += float(x[i, k]) * float(w[j, k])  # weight is [out, in]: row j makes output j
            want[i, j] = acc + float(b[j])
    assert torch.equal(ref.linear(x, w, b), want)
    assert torch.equal(ref.linear(x, w), want - b.double())
    # identity weight returns x; a one-hot row picks a column of x; a transposed operand would fail both
    xr = torch.randn((4, 6), generator=g)
    assert torch.equal(ref.linear(xr, torch.eye(6)), xr.double())
    pick = torch.zeros((2, 6))
    pick[0, 4] = 1.0
    pick[1, 1] = -2.0
    assert torch.equal(ref.linear(xr, pick), torch.stack([xr[:, 4], -2.0 * xr[:, 1]], dim=1).double())
    # linear in x
    x2 = torch.randint(-4, 5, (M, Kd), generator=g).float()
    assert torch.equal(ref.linear(x + x2, w), ref.linear(x, w) + ref.linear(x2, w))
    # the residual is added to the value as the data type holds it
    xb, wb = torch.randn((3, 8), generator=g).bfloat16(), torch.randn((4, 8), generator=g).bfloat16()
    r = torch.randn((3, 4), generator=g).bfloat16()
    y = ref.linear(xb, wb)
    assert torch.equal(ref.linear(xb, wb, residual=r), y.to(torch.bfloat16).double() + r.double())
