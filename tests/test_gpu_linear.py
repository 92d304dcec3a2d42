"""hipattn_linear (x . weight^T + bias + residual for the rows of a generation step) through the C ABI against
the oracle's fp64 product, on the projection shapes of the configured models and on awkward ones."""
import pytest
import torch

from aici_amd import kernels as K
from aici_amd._lib import HipAttnError
from oracle import refkernels as ref

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def library_choice():
    yield
    for name in ("linear_tiles", "linear_waves", "linear_splits"):
        K.tuning_set(name, 0)


def operands(M, N, Kd, dtype, seed, ldx=None, ldw=None):
    g = torch.Generator().manual_seed(seed)
    xw = torch.randn((M, ldx or Kd), generator=g).to(dtype)
    ww = (torch.randn((N, ldw or Kd), generator=g) * 0.05).to(dtype)
    return xw[:, :Kd], ww[:, :Kd], g


def check(y: torch.Tensor, x, w, bias=None, residual=None):
    """Distance to the fp64 product at most half a unit in the last place of the data type (2^-9 of the value for
    bf16 with its 8 significant bits, 2^-12 for fp16) at each of the two roundings, plus what fp32 accumulation in
    any order can lose: 2^-22 of sum |x||w|."""
    want = ref.linear(x, w, bias)
    eps = 2.0 ** -8 if x.dtype == torch.bfloat16 else 2.0 ** -11
    slack = (x.double().abs() @ w.double().abs().t()) * 2.0 ** -22
    bound = eps * want.abs() + slack
    if residual is not None:
        # the first rounding moves the value by at most eps * |want|; then the sum is rounded once more
        total = want + residual.double()
        bound = bound + eps * total.abs() + eps * bound
        want = total
    err = (y.cpu().double() - want).abs()
    worst = (err - bound).max().item()
    assert worst <= 0.0, f"off by {err.max().item():.3e}, {worst:.3e} past the bound"


SHAPES = [
    # (M, N, K): the projections of Llama-3-8B, Phi-2 (hidden 2560, FFN 10240) and small / ragged ones
    (128, 4096, 4096), (128, 6144, 4096), (128, 4096, 14336), (128, 28672, 4096),
    (120, 2560, 2560), (124, 7680, 2560), (100, 2560, 10240),
    (1, 64, 256), (7, 48, 512), (16, 16, 256), (17, 272, 768), (128, 4112, 1024),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", SHAPES)
def test_matches_the_fp64_product(device, dtype, shape):
    M, N, Kd = shape
    x, w, _ = operands(M, N, Kd, dtype, seed=M + N + Kd)
    y = K.linear(x.to(device), w.to(device))
    assert y.shape == (M, N) and y.dtype == dtype
    check(y, x, w)


@pytest.mark.parametrize("tiles", [1, 2])
@pytest.mark.parametrize("waves", [4, 8])
@pytest.mark.parametrize("splits", [1, 2, 3, 8, 32])
def test_every_launch_shape(device, tiles, waves, splits):
    K.tuning_set("linear_tiles", tiles)
    K.tuning_set("linear_waves", waves)
    K.tuning_set("linear_splits", splits)
    for (M, N, Kd) in [(128, 4096, 4096), (37, 208, 1792), (128, 1040, 256)]:
        x, w, g = operands(M, N, Kd, torch.bfloat16, seed=tiles * 100 + waves * 10 + splits)
        bias = torch.randn((N,), generator=g).bfloat16()
        res = torch.randn((M, N), generator=g).bfloat16()
        y = K.linear(x.to(device), w.to(device), bias=bias.to(device), residual=res.to(device))
        check(y, x, w, bias, res)


def test_identity_and_one_hot_weights_are_exact(device):
    g = torch.Generator().manual_seed(5)
    x = torch.randn((128, 512), generator=g).bfloat16()
    for splits in (1, 2):
        K.tuning_set("linear_splits", splits)
        y = K.linear(x.to(device), torch.eye(512).bfloat16().to(device))
        assert torch.equal(y.cpu(), x)
        pick = torch.zeros((16, 512))
        cols = torch.randperm(512, generator=g)[:16]
        pick[torch.arange(16), cols] = 1.0
        y = K.linear(x.to(device), pick.bfloat16().to(device))
        assert torch.equal(y.cpu(), x[:, cols])


def test_residual_is_a_second_rounding_and_bias_is_not(device):
    x, w, g = operands(128, 4096, 4096, torch.bfloat16, seed=9)
    res = torch.randn((128, 4096), generator=g).bfloat16()
    bias = torch.randn((4096,), generator=g).bfloat16()
    xd, wd = x.to(device), w.to(device)
    plain = K.linear(xd, wd)
    with_res = K.linear(xd, wd, residual=res.to(device))
    # exactly the separate addition of llama.rs:166: T(T(x . W^T) + residual)
    assert torch.equal(with_res.cpu(), (plain.cpu().float() + res.float()).bfloat16())
    # the bias goes in before the only rounding: closer to the fp64 value than a rounded product plus bias
    check(K.linear(xd, wd, bias=bias.to(device)), x, w, bias)
    both = K.linear(xd, wd, bias=bias.to(device), residual=res.to(device))
    with_bias = K.linear(xd, wd, bias=bias.to(device))
    assert torch.equal(both.cpu(), (with_bias.cpu().float() + res.float()).bfloat16())


def test_row_strides_of_every_operand(device):
    M, N, Kd = 96, 1024, 768
    x, w, g = operands(M, N, Kd, torch.float16, seed=21, ldx=3 * Kd, ldw=Kd + 64)
    assert x.stride(0) == 3 * Kd and w.stride(0) == Kd + 64
    wide_res = torch.randn((M, 2 * N), generator=g).half()
    res = wide_res[:, N:]
    xd = torch.randn((M, 3 * Kd), generator=g).half().to(device)
    xd[:, :Kd] = x.to(device)
    wd = torch.zeros((N, Kd + 64), dtype=torch.float16, device=device)
    wd[:, :Kd] = w.to(device)
    out_wide = torch.full((M, N + 8), 7.0, dtype=torch.float16, device=device)
    K.linear(xd[:, :Kd], wd[:, :Kd], residual=wide_res.to(device)[:, N:], out=out_wide[:, :N])
    check(out_wide[:, :N], x, w, residual=res)
    assert torch.all(out_wide[:, N:] == 7.0)  # nothing written past a row's end


def test_same_bits_on_every_run_and_rows_do_not_mix(device):
    x, w, _ = operands(128, 4096, 14336, torch.bfloat16, seed=33)
    xd, wd = x.to(device), w.to(device)
    first = K.linear(xd, wd)
    for _ in range(3):
        assert torch.equal(K.linear(xd, wd), first)
    # a row's result does not depend on how many other rows come along
    for m in (1, 5, 64):
        assert torch.equal(K.linear(xd[:m].contiguous(), wd), first[:m])


def test_workspace_from_the_caller(device):
    x, w, _ = operands(128, 4096, 4096, torch.bfloat16, seed=41)
    xd, wd = x.to(device), w.to(device)
    need = K.linear_workspace_size(xd, wd)
    assert need > 0
    ws = torch.empty((need,), dtype=torch.uint8, device=device)
    assert torch.equal(K.linear(xd, wd, workspace=ws), K.linear(xd, wd))
    with pytest.raises(HipAttnError, match="workspace has"):
        K.linear(xd, wd, workspace=ws[: need - 256])
    K.tuning_set("linear_splits", 1)
    assert K.linear_workspace_size(xd, wd) == 0


@pytest.mark.parametrize("splits", [0, 1, 3, 8])
def test_linear_rms_norm_gives_the_bits_of_the_two_calls(device, splits):
    K.tuning_set("linear_splits", splits)
    for (M, N, Kd, dtype, with_bias) in [(128, 4096, 4096, torch.bfloat16, False), (128, 4096, 14336, torch.bfloat16, False),
                                         (37, 2560, 2560, torch.float16, True), (5, 64, 256, torch.bfloat16, True),
                                         (128, 8192, 512, torch.bfloat16, False)]:
        x, w, g = operands(M, N, Kd, dtype, seed=N + Kd + splits)
        res = torch.randn((M, N), generator=g).to(dtype).to(device)
        bias = torch.randn((N,), generator=g).to(dtype).to(device) if with_bias else None
        nw = (1.0 + 0.1 * torch.randn((N,), generator=g)).to(dtype).to(device)
        xd, wd = x.to(device), w.to(device)
        out, normed = K.linear_rms_norm(xd, wd, nw, 1e-5, bias=bias, residual=res)
        want = K.linear(xd, wd, bias=bias, residual=res)
        assert torch.equal(out, want)
        want_n = torch.empty_like(want)
        K.rms_norm(want_n, want, nw, 1e-5)
        assert torch.equal(normed, want_n)
        # and the norm is the oracle's, from the rounded rows
        o = ref.rms_norm(out.cpu(), nw.cpu(), 1e-5)
        assert (normed.cpu().float() - o.float()).abs().max().item() <= (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) * max(1.0, o.float().abs().max().item())
    # without a residual, from the caller's workspace, and what is refused
    x, w, g = operands(64, 1024, 768, torch.bfloat16, seed=77)
    nw = torch.ones((1024,), dtype=torch.bfloat16, device=device)
    xd, wd = x.to(device), w.to(device)
    ws = torch.empty((K.linear_rms_norm_workspace_size(xd, wd),), dtype=torch.uint8, device=device)
    assert ws.numel() > 0
    out, normed = K.linear_rms_norm(xd, wd, nw, 1e-6, workspace=ws)
    assert torch.equal(out, K.linear(xd, wd))
    with pytest.raises(HipAttnError, match="at most 8192"):
        K.linear_rms_norm(torch.zeros((8, 256), dtype=torch.bfloat16, device=device),
                          torch.zeros((8208, 256), dtype=torch.bfloat16, device=device),
                          torch.ones((8208,), dtype=torch.bfloat16, device=device), 1e-5)
    with pytest.raises(HipAttnError, match="norm_weight must be"):
        K.linear_rms_norm(xd, wd, nw[:512], 1e-5)


def test_refusals(device):
    def t(*shape, dtype=torch.bfloat16):
        return torch.zeros(shape, dtype=dtype, device=device)
    with pytest.raises(HipAttnError, match="at most 128"):
        K.linear(t(129, 256), t(64, 256))
    with pytest.raises(HipAttnError, match="multiple of 256"):
        K.linear(t(8, 320), t(64, 320))
    with pytest.raises(HipAttnError, match="multiple of 16"):
        K.linear(t(8, 256), t(40, 256))
    with pytest.raises(HipAttnError, match="weight is f16"):
        K.linear(t(8, 256), t(64, 256, dtype=torch.float16))
    with pytest.raises(HipAttnError, match="f16 or bf16"):
        K.linear(t(8, 256, dtype=torch.float32), t(64, 256, dtype=torch.float32))
    with pytest.raises(HipAttnError, match="columns"):
        K.linear(t(8, 256), t(64, 512))
    with pytest.raises(HipAttnError, match="out is"):
        K.linear(t(8, 256), t(64, 256), out=t(8, 32))
    with pytest.raises(HipAttnError, match="residual must be"):
        K.linear(t(8, 256), t(64, 256), residual=t(8, 32))
    with pytest.raises(HipAttnError, match="bias must be"):
        K.linear(t(8, 256), t(64, 256), bias=t(32))
    assert not K.linear_takes(t(129, 256), t(64, 256)) and not K.linear_takes(t(8, 320), t(64, 320))
    assert K.linear_takes(t(8, 256), t(64, 256))
    assert K.linear(t(0, 256), t(64, 256)).shape == (0, 64)
