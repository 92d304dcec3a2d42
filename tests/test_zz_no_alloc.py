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
