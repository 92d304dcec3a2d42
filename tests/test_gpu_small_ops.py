"""rotary_embedding, rms_norm, activations, bias_argmax and the runtime plumbing through the
C ABI against the oracle."""
import numpy as np
import pytest
import torch

from aici_amd import attn, kernels as K
from aici_amd import workloads as W
from aici_amd._lib import HipAttnError
from oracle import aici
from oracle import refkernels as ref

pytestmark = pytest.mark.gpu


def ulp_diff16(a: torch.Tensor, b: torch.Tensor) -> int:
    """Largest distance in representable values between two fp16/bf16 tensors."""
    def key(t):
        i = t.cpu().contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return int((key(a) - key(b)).abs().max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(32, 8, 128, 128), (32, 32, 80, 32), (4, 1, 64, 64)])  # Hq, Hkv, d, rot
@pytest.mark.parametrize("neox", [True, False])
def test_rotary_matches_oracle(device, dtype, shape, neox):
    Hq, Hkv, d, rot = shape
    g = torch.Generator().manual_seed(3)
    T, max_pos = 37, 512
    table = ref.rotary_table(rot, 10000.0, max_pos, dtype)
    assert torch.equal(table, attn.RotaryEmbedding.build_table(rot, 10000.0, max_pos, dtype))
    q = torch.randn((T, Hq * d), generator=g).to(dtype)
    k = torch.randn((T, Hkv * d), generator=g).to(dtype)
    pos = torch.randint(0, max_pos, (T,), generator=g, dtype=torch.int64)
    pos[0] = 0
    qd, kd = q.clone().to(device), k.clone().to(device)
    K.rotary_embedding(pos.to(device), qd, kd, d, table.to(device), neox)
    ref.rotary_embedding(pos, q, k, d, table, neox)
    if dtype == torch.float32:
        # the reference's own self-check tolerance for this op is 1e-5 (llm/mod.rs:104-105)
        assert (qd.cpu() - q).abs().max().item() <= 1e-6 and (kd.cpu() - k).abs().max().item() <= 1e-6
    else:  # same rounding points as the oracle's per-op arithmetic: bit-exact
        assert torch.equal(qd.cpu().view(torch.int16), q.view(torch.int16))
        assert torch.equal(kd.cpu().view(torch.int16), k.view(torch.int16))


def test_rotary_strided_rows_and_int32_positions(device):
    g = torch.Generator().manual_seed(4)
    T, H, d = 9, 4, 64
    table = ref.rotary_table(d, 10000.0, 64, torch.float16)
    big = torch.randn((T, 3 * H * d), generator=g).to(torch.float16)
    q, k = big[:, :H * d], big[:, H * d:2 * H * d]  # row stride 3*H*d
    pos = torch.arange(T, dtype=torch.int32)
    bd = big.clone().to(device)
    K.rotary_embedding(pos.to(device), bd[:, :H * d], bd[:, H * d:2 * H * d], d, table.to(device), True)
    qc, kc = q.clone().contiguous(), k.clone().contiguous()
    ref.rotary_embedding(pos, qc, kc, d, table, True)
    out = bd.cpu()
    assert torch.equal(out[:, :H * d], qc) and torch.equal(out[:, H * d:2 * H * d], kc)
    assert torch.equal(out[:, 2 * H * d:], big[:, 2 * H * d:])  # the v third is untouched


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("hidden", [4096, 2560, 100])
def test_rms_norm_and_fused(device, dtype, hidden):
    g = torch.Generator().manual_seed(5)
    x = (torch.randn((17, hidden), generator=g) * 3).to(dtype)
    w = (1 + 0.1 * torch.randn((hidden,), generator=g)).to(dtype)
    out = torch.empty_like(x).to(device)
    K.rms_norm(out, x.to(device), w.to(device), 1e-5)
    want = ref.rms_norm(x, w, 1e-5)
    if dtype == torch.float32:
        assert (out.cpu() - want).abs().max().item() <= 2e-6 * want.abs().max().item()
    else:
        # The fp32 reduction order differs, which can move the first rounding by one value; the
        # multiply by a weight above 1 can stretch that to two values of the result.
        assert ulp_diff16(out, want) <= 2
        assert (out.cpu() == want).float().mean().item() > 0.995
    r = torch.randn((17, hidden), generator=g).to(dtype)
    xi, ri = x.clone(), r.clone()
    ref.fused_add_rms_norm(xi, ri, w, 1e-5)
    xd, rd = x.clone().to(device), r.clone().to(device)
    K.fused_add_rms_norm(xd, rd, w.to(device), 1e-5)
    assert torch.equal(rd.cpu(), ri)  # the residual sum is exact
    if dtype == torch.float32:
        assert (xd.cpu() - xi).abs().max().item() <= 2e-6 * xi.abs().max().item()
    else:
        assert ulp_diff16(xd, xi) <= 2
        assert (xd.cpu() == xi).float().mean().item() > 0.995
    m = attn.RmsNorm(w.to(device), 1e-5)
    assert torch.equal(m.forward(x.to(device)), out)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_activations(device, dtype):
    g = torch.Generator().manual_seed(6)
    x = (torch.randn((5, 2 * 300), generator=g) * 2).to(dtype)
    tol = dict(atol=1e-6, rtol=1e-6) if dtype == torch.float32 else None
    out = torch.empty((5, 300), dtype=dtype, device=device)
    K.silu_and_mul(out, x.to(device))
    want = ref.silu_and_mul(x)
    # expf / tanhf on the GPU and on the CPU may differ in the last place before rounding
    if tol:
        assert torch.allclose(out.cpu(), want, **tol)
    else:
        assert ulp_diff16(out, want) <= 1
    # a width the 16-byte kernel takes (multiple of 8), Llama-3-8B's FFN size
    xw = (torch.randn((3, 2 * 14336), generator=g) * 2).to(dtype)
    outw = torch.empty((3, 14336), dtype=dtype, device=device)
    K.silu_and_mul(outw, xw.to(device))
    if tol:
        assert torch.allclose(outw.cpu(), ref.silu_and_mul(xw), **tol)
    else:
        assert ulp_diff16(outw, ref.silu_and_mul(xw)) <= 1
    for fn, rf in ((K.gelu_new, ref.gelu_new), (K.gelu_fast, ref.gelu_fast)):
        o = torch.empty_like(x).to(device)
        fn(o, x.to(device))
        w = rf(x)
        if tol:
            assert torch.allclose(o.cpu(), w, atol=1e-6, rtol=1e-5)
        else:
            assert ulp_diff16(o, w) <= 2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_bias_argmax_bias_rows_and_packed_mask(device, dtype):
    S, V = 9, 128256
    g = torch.Generator().manual_seed(7)
    logits = torch.randn((S, V), generator=g).to(dtype)
    allowed = W.allow_mask(5, S, V, 0.05)
    allowed[3, :] = False            # nothing allowed: argmax of all -inf is token 0
    allowed[4, :] = False
    allowed[4, V - 1] = True         # only the last token
    packed = np.stack([aici.pack_allowed(a) for a in allowed])
    rows = np.stack([aici.apply_to_slice_fast(p, aici.bias_row_len(V)) for p in packed])
    bias = torch.from_numpy(rows)
    want = aici.biased_argmax(logits, bias)
    assert want[3].item() == 0 and want[4].item() == V - 1
    ld = logits.to(device)
    got_bias, best = K.bias_argmax(ld, bias=bias.to(device), return_logits=True)
    got_mask = K.bias_argmax(ld, mask=torch.from_numpy(packed).to(device))
    assert torch.equal(got_bias.cpu().long(), want) and torch.equal(got_mask.cpu().long(), want)
    picked = logits.float()[torch.arange(S), want]
    picked[3] = float("-inf")
    assert torch.equal(best.cpu(), picked)
    # row indirection: every sequence uses bias row 2
    sel = torch.full((S,), 2, dtype=torch.int32)
    got = K.bias_argmax(ld, bias=bias.to(device), bias_rows=sel.to(device))
    assert torch.equal(got.cpu().long(), aici.biased_argmax(logits, bias[2:3].expand(S, -1)))
    # ties resolve to the lowest token id
    flat = torch.zeros((2, 1000), dtype=dtype, device=device)
    assert K.bias_argmax(flat, bias=torch.zeros((2, 1024), device=device)).tolist() == [0, 0]
    # ... also across the slices a long row is cut into: equal maxima at ids 70000 and 16, fp16
    wide = torch.full((3, 131072), -1.0, dtype=torch.float16, device=device)
    wide[0, 70000] = 2.0
    wide[0, 16] = 2.0
    wide[1, 131071] = 5.0
    allow_all = torch.full((3, 131072 // 8), 255, dtype=torch.uint8, device=device)
    assert K.bias_argmax(wide, mask=allow_all).tolist() == [16, 131071, 0]
    allow_all[0, 2] = 0              # forbid ids 16..23: the later maximum wins
    assert K.bias_argmax(wide, mask=allow_all).tolist() == [70000, 131071, 0]
    with pytest.raises(HipAttnError, match="exactly one"):
        K.bias_argmax(ld)


def test_bias_argmax_wide_rows_call_after_call(device):
    """Long 16-bit rows are cut into slices whose winners meet in a per-row key and counter in a buffer the
    library keeps per stream and clears in front of every launch: call after call with changing row counts,
    vocabularies and slice counts, negative and infinite winners, and the winning value itself."""
    g = torch.Generator().manual_seed(11)
    for S, V in ((128, 65536), (5, 65536), (64, 131072), (1, 65536), (200, 16384), (3, 131072)):
        logits = (torch.randn((S, V), generator=g) - 6.0).to(torch.bfloat16)      # every value negative
        logits[0, 4242] = float("-inf")
        allowed = torch.rand((S, V), generator=g) < 0.03
        if S > 2:
            allowed[2, :] = False
            allowed[2, 77] = True                                                  # one token, wherever its value lies
        packed = torch.from_numpy(np.stack([aici.pack_allowed(a) for a in allowed.numpy()]))
        masked = torch.where(allowed, logits.float(), torch.tensor(float("-inf")))
        want = masked.argmax(dim=1)
        for _ in range(3):
            tok, best = K.bias_argmax(logits.to(device), mask=packed.to(device), return_logits=True)
            assert torch.equal(tok.cpu().long(), want)
            assert torch.equal(best.cpu(), masked[torch.arange(S), want])
    V = 65536
    pos_inf = torch.zeros((2, V), dtype=torch.float16, device=device)
    pos_inf[1, 40000] = float("inf")
    tok, best = K.bias_argmax(pos_inf, mask=torch.full((2, V // 8), 255, dtype=torch.uint8, device=device),
                              return_logits=True)
    assert tok.tolist() == [0, 40000] and best.tolist() == [0.0, float("inf")]


def _sample_check(logits, bias, temperature, top_p, u, got):
    """Row by row against the oracle.  The oracle's token is expected; where the two differ the draw must sit
    on an edge: u * total within 1e-5 (relative) of the cumulative weight that separates the two tokens, or
    the nucleus cut within f32 rounding of admitting one more token.  Returns the number of rows that differ."""
    differ = 0
    V = logits.shape[1]
    for s in range(logits.shape[0]):
        want = aici.sample(logits[s], bias[s], float(temperature[s]), float(top_p[s]), float(u[s]))
        t = int(got[s])
        if t == want:
            continue
        differ += 1
        assert temperature[s] >= aici.SAMPLING_EPS, (s, t, want)      # the arg-max is exact
        prs = torch.softmax((logits[s].float() + bias[s][:V]).double() / float(temperature[s]), 0).numpy()
        w = prs.copy()
        if 0.0 < top_p[s] < 1.0:
            order = sorted(range(V), key=lambda i: (-prs[i], i))
            mass, kept = 0.0, np.zeros(V, dtype=bool)
            for i in order:
                if mass >= float(top_p[s]) * (1 + 1e-5):
                    break
                kept[i] = True
                mass += prs[i]
            w = np.where(kept, prs, 0.0)
        assert w[t] > 0, (s, t, want)
        cum = np.cumsum(w)
        c = float(u[s])
        lo, hi = (cum[t - 1] if t else 0.0) / cum[-1], cum[t] / cum[-1]
        assert lo - 1e-4 <= c <= hi + 1e-4, (s, t, want, lo, c, hi)
    return differ


@pytest.mark.parametrize("dtype,V,mode", [(torch.bfloat16, 128256, "mask"), (torch.float16, 50000, "bias"),
                                          (torch.float32, 1000, "bias"), (torch.bfloat16, 4097, "mask")])
def test_bias_sample_matches_the_oracle(device, dtype, V, mode):
    """Temperature + top-p sampling under the AICI bias against the restatement of tmodel.rs:172-194,
    236-268, row by row with the caller's uniform numbers: greedy rows, plain sampling (top_p 0 and 1),
    nuclei from tiny to almost everything, sharp and flat temperatures."""
    S = 40
    g = torch.Generator().manual_seed(11)
    rng = np.random.default_rng(11)
    logits = (torch.randn((S, V), generator=g) * 2.5).to(dtype)
    allowed = W.allow_mask(6, S, V, 0.05 if V > 5000 else 0.5)
    allowed[:, 17] = True
    packed = np.stack([aici.pack_allowed(a) for a in allowed])
    bias = torch.from_numpy(np.stack([aici.apply_to_slice_fast(p, aici.bias_row_len(V)) for p in packed]))
    temperature = torch.tensor(rng.choice([0.0, 1e-6, 0.05, 0.5, 0.8, 1.0, 1.7, 10.0], size=S), dtype=torch.float32)
    top_p = torch.tensor(rng.choice([0.0, 1.0, 1e-4, 0.1, 0.5, 0.9, 0.95, 0.999], size=S), dtype=torch.float32)
    u = torch.tensor(rng.random(S), dtype=torch.float32)
    u[0], u[1] = 0.0, 0.99999994
    kw = dict(mask=torch.from_numpy(packed).to(device)) if mode == "mask" else dict(bias=bias.to(device))
    got = K.bias_sample(logits.to(device), temperature.to(device), top_p.to(device), u.to(device), **kw).cpu()
    assert allowed[np.arange(S), got.numpy()].all()           # never a disallowed token
    differ = _sample_check(logits, bias, temperature, top_p, u, got)
    assert differ <= 2, differ
    # the launch is a function of its inputs: same tokens again
    again = K.bias_sample(logits.to(device), temperature.to(device), top_p.to(device), u.to(device), **kw).cpu()
    assert torch.equal(got, again)


def test_bias_sample_equal_values_and_distribution(device):
    """Coarse logits (many equal probabilities, the usual case with 16-bit logits): one row drawn with 4096
    evenly spaced uniform numbers.  The nucleus cut must split a run of equal values by ascending id, and the
    draws must reproduce the kept weights as frequencies."""
    V, n = 3000, 4096
    g = torch.Generator().manual_seed(12)
    row = (torch.randn((V,), generator=g) * 1.5).mul(2).round().div(2).to(torch.bfloat16)   # steps of 0.5
    logits = row[None].expand(n, V).contiguous()
    bias = torch.zeros((1, aici.bias_row_len(V)))
    bias[0, 5::7] = float("-inf")
    rows = torch.zeros((n,), dtype=torch.int32)
    u = ((torch.arange(n) + 0.5) / n).float()
    for top_p in (0.3, 0.62, 0.9, 1.0):
        temperature = torch.full((n,), 0.7)
        got = K.bias_sample(logits.to(device), temperature.to(device), torch.full((n,), top_p).to(device),
                            u.to(device), bias=bias.to(device), bias_rows=rows.to(device)).cpu().numpy()
        prs = torch.softmax((row.float() + bias[0, :V]) / 0.7, 0).numpy()
        w = aici.nucleus_weights(prs, top_p) if top_p < 1.0 else prs
        kept = w > 0
        # the kept set: everything above the cut, and of the values equal to the cut the lowest ids
        cut = prs[kept].min()
        assert np.array_equal(kept, (prs > cut) | ((prs == cut) & (np.cumsum(prs == cut) <= (kept & (prs == cut)).sum())))
        assert kept[got].all()
        freq = np.bincount(got, minlength=V) / n
        assert np.abs(freq - w / w.sum()).max() <= 1.01 / n + 1e-6
        # draw by draw: the oracle's token, except where u sits on an edge between two tokens -- the
        # cumulative weights are f32 sums formed in different orders on the two sides (3000 terms: 1e-5)
        want = np.array([aici.weighted_index(w, float(x)) for x in u])
        off = np.nonzero(got != want)[0]
        assert len(off) <= n // 100, len(off)
        cum = np.cumsum(w.astype(np.float64)) / w.astype(np.float64).sum()
        for i in off:
            t = int(got[i])
            assert (cum[t - 1] if t else 0.0) - 1e-4 <= float(u[i]) <= cum[t] + 1e-4, (top_p, i, t, int(want[i]))


def test_bias_sample_corner_rows(device):
    """Rows outside what the reference defines still give a defined, allowed token: an infinite logit (its first
    holder), uniform numbers outside [0, 1) (the first / the last token with weight), an infinite temperature
    (uniform over the allowed tokens only), nothing allowed (token 0)."""
    V = 4096
    g = torch.Generator().manual_seed(5)
    logits = torch.randn((6, V), generator=g).to(torch.bfloat16)
    allowed = torch.rand((6, V), generator=g) < 0.1
    allowed[:, 0] = False
    logits[0, 777] = float("inf")
    logits[0, 900] = float("inf")
    allowed[0, 777] = allowed[0, 900] = True
    allowed[5, :] = False
    packed = torch.from_numpy(np.stack([aici.pack_allowed(a) for a in allowed.numpy()]))
    f = lambda *v: torch.tensor(v, dtype=torch.float32, device=device)
    temperature = f(1.0, 1.0, 1.0, float("inf"), 1e30, 1.0)
    top_p = f(0.9, 1.0, 1.0, 1.0, 0.5, 0.9)
    u = f(0.3, -0.5, 7.0, 0.5, 0.999, 0.5)
    got = K.bias_sample(logits.to(device), temperature, top_p, u, mask=packed.to(device)).tolist()
    ids = [torch.nonzero(a).flatten().tolist() for a in allowed]
    assert got[0] == 777
    assert got[1] == ids[1][0] and got[2] == ids[2][-1]
    assert got[3] == ids[3][len(ids[3]) // 2]              # equal weights: the middle one at u = 0.5
    assert got[4] in ids[4]
    assert got[5] == 0


def test_aici_sample_with_a_seeded_generator(device):
    """llama.aici_sample draws its uniform numbers from a seeded generator when none are given: the same seed
    gives the same tokens, those the oracle picks for the same numbers, and only allowed ones."""
    from aici_amd import llama
    S, V = 16, 32000
    g = torch.Generator().manual_seed(21)
    logits = (torch.randn((S, V), generator=g) * 3).to(torch.bfloat16)
    allowed = torch.rand((S, V), generator=g) < 0.02
    packed = torch.from_numpy(np.stack([aici.pack_allowed(a) for a in allowed.numpy()]))
    temperature = torch.full((S,), 0.7, device=device)
    top_p = torch.full((S,), 0.95, device=device)
    draw = lambda seed: llama.aici_sample(logits.to(device), packed.to(device), temperature, top_p,
                                          generator=torch.Generator().manual_seed(seed)).cpu()
    a, b, c = draw(5), draw(5), draw(6)
    assert torch.equal(a, b) and not torch.equal(a, c)
    assert all(allowed[s, int(a[s])] for s in range(S))
    u = torch.rand((S,), generator=torch.Generator().manual_seed(5), dtype=torch.float32)
    bias = torch.where(allowed, 0.0, float("-inf"))
    differ = _sample_check(logits, bias, temperature.cpu(), top_p.cpu(), u, a)
    assert differ <= 1


def test_bias_sample_argument_errors(device):
    lg = torch.zeros((2, 64), dtype=torch.float16, device=device)
    f = lambda *v: torch.tensor(v, dtype=torch.float32, device=device)
    m = torch.full((2, 8), 255, dtype=torch.uint8, device=device)
    assert K.bias_sample(lg, f(1.0, 0.0), f(1.0, 1.0), f(0.5, 0.5), mask=m).tolist() == [32, 0]
    with pytest.raises(HipAttnError, match="exactly one"):
        K.bias_sample(lg, f(1.0, 1.0), f(1.0, 1.0), f(0.5, 0.5))
    with pytest.raises(HipAttnError, match=r"top_p must be f32 \[S\]"):
        K.bias_sample(lg, f(1.0, 1.0), f(1.0), f(0.5, 0.5), mask=m)
    none = torch.zeros((2, 8), dtype=torch.uint8, device=device)
    assert K.bias_sample(lg, f(1.0, 1.0), f(0.9, 1.0), f(0.5, 0.5), mask=none).tolist() == [0, 0]   # nothing allowed
    # a bias row index outside the rows given reads the nearest row, never beyond
    far = torch.tensor([5, -3], dtype=torch.int32, device=device)
    assert K.bias_sample(lg, f(0.0, 0.0), f(1.0, 1.0), f(0.5, 0.5), mask=m, bias_rows=far).tolist() == [0, 0]
    assert K.bias_argmax(lg, mask=m, bias_rows=far).tolist() == [0, 0]


def test_streams_events_and_memory_figures(device):
    props = K.cuda_get_device_properties(0)
    assert props.multi_processor_count == 256 and props.total_memory > 200 * 2 ** 30
    K.cuda_reset_peak_memory_stats(0)
    st = K.cuda_get_stats_allocated_bytes(0)
    assert st.current > 0 and st.peak >= st.current
    assert "GiB" in str(st)
    s = K.CudaStream()  # pool stream
    assert s.device_index() == 0 and s.raw != 0 and s.id() == s.raw
    c = s.clone()
    assert c.raw == s.raw
    e0, e1 = K.CudaEvent(timing=True), K.CudaEvent(timing=True)
    x = torch.ones((1 << 20,), dtype=torch.float16, device=device)
    out = torch.empty_like(x)
    torch.cuda.synchronize()  # the pool stream does not order itself after torch's stream
    import ctypes
    from aici_amd.kernels import _desc, call
    e0.record(s)
    call("hipattn_gelu_new", _desc(out), _desc(x), ctypes.c_void_p(s.raw))  # explicit stream argument
    e1.record(s)
    e1.synchronize()
    assert e0.query() and e1.query() and s.query()
    assert e0.elapsed_time(e1) >= 0.0
    s.synchronize()
    assert torch.allclose(out[:4].float().cpu(), ref.gelu_new(torch.ones(4, dtype=torch.float16)).float())
    # NULL stream argument = the thread's current stream
    s.set_current()
    call("hipattn_gelu_new", _desc(out), _desc(x), None)
    K.CudaStream.current().synchronize()
    K.CudaStream.default().set_current()
    ev = K.CudaEvent()
    ev.record(K.CudaStream.default())
    ev.wait(s)
    s.synchronize()


def test_memory_yardsticks_of_the_benchmark(device):
    """The benchmark's memory-system yardsticks (a library of their own, libmembench.so): copy and fill do
    what they say, the reads launch and leave their source alone, bad arguments are refused."""
    from aici_amd import membench
    g = torch.Generator().manual_seed(5)
    src = torch.randint(0, 255, (8 * 4096 + 16,), generator=g, dtype=torch.uint8).to(device)
    dst = torch.zeros_like(src)
    membench.probe("copy", dst, src)
    assert torch.equal(dst.cpu(), src.cpu())
    membench.probe("fill", dst, None)
    want = torch.tensor([1, 2, 3, 4], dtype=torch.int32).repeat(dst.numel() // 16)
    assert torch.equal(dst.cpu().view(torch.int32), want)
    before = src.cpu().clone()
    membench.probe("read", None, src)
    chunks = torch.tensor([7, 0, 3, 3, 5], dtype=torch.int32, device=device)
    membench.probe("read_chunks", None, src[: 8 * 4096], chunks)
    membench.probe("read_chunks", None, src[: 8 * 4096], torch.tensor([1, 0], dtype=torch.int32, device=device), 16384)
    torch.cuda.synchronize()
    assert torch.equal(src.cpu(), before)
    with pytest.raises(RuntimeError, match="bad arguments"):
        membench.probe("read", None, src[:100])
    with pytest.raises(RuntimeError, match="bad arguments"):
        membench.probe("read_chunks", None, src[: 4096 + 16], chunks)


def test_matrix_pipe_yardstick_of_the_benchmark(device):
    """The benchmark's bare stream of MFMAs launches, counts its flops as 16 x iters MFMAs of 32 x 32 x 16 per
    wavefront, leaves its operands alone and refuses operands of another kind."""
    from aici_amd import membench
    ops = torch.randn(membench.MFMA_STREAM_OPERAND_ELEMS, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16).to(device)
    before = ops.cpu().clone()
    flop = membench.mfma_stream(ops, 4, 10)
    torch.cuda.synchronize()
    assert flop == 4 * 8 * 10 * 16 * 2 * 32 * 32 * 16
    assert torch.equal(ops.cpu().view(torch.int16), before.view(torch.int16))
    with pytest.raises(ValueError):
        membench.mfma_stream(ops.float(), 4, 10)
    with pytest.raises(ValueError):
        membench.mfma_stream(ops[:100], 4, 10)
