"""hipattn_paged_attention_v1_static, the decode entry point that allocates nothing (its split-K scratch
memory is an array built into the library), against hipattn_paged_attention_v1: same bits, on two calls
in a row of which the second is smaller, for both launch strategies; shapes beyond the array are refused."""
import pytest
import torch

from aici_amd import kernels as K
from aici_amd import workloads as W
from aici_amd._lib import HipAttnError

pytestmark = pytest.mark.gpu


def both(c, device):
    d = c.to(device)
    args = (d.q, d.key_cache, d.value_cache, c.num_kv_heads, c.scale, d.block_tables, d.context_lens, 16, c.max_ctx)
    want = torch.full_like(d.q, float("nan"))
    K.paged_attention_v1(want, *args)
    got = torch.full_like(d.q, float("nan"))
    K.paged_attention_v1_static(got, *args)
    torch.cuda.synchronize()
    return got, want


@pytest.mark.parametrize("strategy", ["flat", "partitioned"])
def test_static_scratch_entry_matches_v1_twice_in_a_row(device, tuning, strategy):
    tuning("decode_flat", 1 if strategy == "flat" else 0)
    K.init()
    big = W.decode_inputs(61, 48, 700, 4096, 32, 8, 128, torch.bfloat16, 9000)
    small = W.decode_inputs(62, 5, 30, 900, 32, 8, 128, torch.bfloat16, 400)
    for c in (big, small, big):
        got, want = both(c, device)
        assert not torch.isnan(want).any()
        assert torch.equal(got, want)
    assert K.paged_attention_workspace_size(48, 32, 8, 128, 16, big.max_ctx, torch.bfloat16) <= 16 << 20


def test_static_scratch_entry_refuses_what_does_not_fit(device, tuning):
    tuning("decode_flat", 0)
    # 600 sequences x 32 heads x 2 partitions of partial results: more than the 16 MiB array
    c = W.decode_inputs(63, 600, 1000, 1100, 32, 8, 128, torch.float16, 600 * 70)
    need = K.paged_attention_workspace_size(600, 32, 8, 128, 16, c.max_ctx, torch.float16)
    assert need > 16 << 20
    d = c.to(device)
    out = torch.empty_like(d.q)
    with pytest.raises(HipAttnError, match="more than the 16777216 bytes of the built-in array"):
        K.paged_attention_v1_static(out, d.q, d.key_cache, d.value_cache, 8, c.scale, d.block_tables, d.context_lens,
                                    16, c.max_ctx)


@pytest.mark.filterwarnings("ignore:The CUDA Graph is empty")   # the refused capture records nothing, as it should
def test_capture_on_a_cold_stream(device, tuning):
    """What the entry point is for: on a stream the library has never seen, under graph capture, v1 has no
    scratch buffer and may not allocate one -- it must say so -- while the static-array form and the
    caller-workspace form record and replay, and give v1's bits."""
    tuning("decode_flat", 1)
    K.init()
    c = W.decode_inputs(64, 24, 600, 3000, 32, 8, 128, torch.bfloat16, 24 * 200)
    d = c.to(device)
    args = (d.q, d.key_cache, d.value_cache, c.num_kv_heads, c.scale, d.block_tables, d.context_lens, 16, c.max_ctx)
    want = torch.empty_like(d.q)
    K.paged_attention_v1(want, *args)                    # eager, on the default stream: kernels loaded, attributes set
    warm = torch.empty_like(d.q)
    K.paged_attention_v1_static(warm, *args)
    ws = torch.empty(K.paged_attention_workspace_size(24, 32, 8, 128, 16, c.max_ctx, torch.bfloat16), dtype=torch.uint8,
                     device=device)
    torch.cuda.synchronize()
    before = K.cuda_get_stats_allocated_bytes(0).allocated

    refused = torch.cuda.Stream()
    graph0 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph0, stream=refused):
        with pytest.raises(HipAttnError, match="cannot happen while the stream is being captured"):
            K.paged_attention_v1(torch.empty_like(d.q), *args)

    cold = torch.cuda.Stream()
    got_static = torch.full_like(d.q, float("nan"))
    got_ws = torch.full_like(d.q, float("nan"))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=cold):
        K.paged_attention_v1_static(got_static, *args)
        K.paged_attention_v1_ws(got_ws, *args, ws)
    for _ in range(3):
        got_static.fill_(float("nan"))
        got_ws.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got_static, want) and torch.equal(got_ws, want)
    # nothing was allocated by the library on the way (its own counter of device allocations)
    assert K.cuda_get_stats_allocated_bytes(0).allocated == before
