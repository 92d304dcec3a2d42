"""The CPU restatement of the Llama-shaped step (oracle/llama.py) against closed forms:
special weights reduce the step to expressions that can be written down directly, so a
wrong residual, a missing norm, a wrong row selection or a wrong kv-head mapping shows."""
import types

import torch

from oracle import hostkv, llama as ollama
from oracle import refkernels as ref


def small_cfg(layers=2):
    return types.SimpleNamespace(hidden_size=64, intermediate_size=96, vocab_size=50, num_hidden_layers=layers,
                                 num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, rope_theta=10000.0,
                                 max_position_embeddings=128)


def rand_weights(cfg, seed, std=0.2):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    d = H // cfg.num_attention_heads
    qd, kvd = d * cfg.num_attention_heads, d * cfg.num_key_value_heads
    r = lambda *s: torch.randn(*s, generator=g) * std
    ws = {"model.embed_tokens": r(V, H), "model.norm": 1 + r(H), "lm_head": r(V, H)}
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        ws.update({p + "input_layernorm": 1 + r(H), p + "self_attn.q_proj": r(qd, H), p + "self_attn.k_proj": r(kvd, H),
                   p + "self_attn.v_proj": r(kvd, H), p + "self_attn.o_proj": r(H, qd),
                   p + "post_attention_layernorm": 1 + r(H), p + "mlp.gate_proj": r(I, H), p + "mlp.up_proj": r(I, H),
                   p + "mlp.down_proj": r(H, I)})
    return ws


def plain_rms(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def build(cfg, seqs, pool=16):
    """seqs: list of token lists, all new (nothing computed)."""
    alloc = hostkv.BlockAllocator(16, pool)
    entries = []
    for i, toks in enumerate(seqs):
        alloc.alloc_seq(i + 1, len(toks))
        entries.append(hostkv.sched_entry(alloc, i + 1, toks, 0))
    bi = hostkv.build_batch(entries, 16, 128, 0)
    d = cfg.hidden_size // cfg.num_attention_heads
    caches = [(torch.zeros(pool, cfg.num_key_value_heads, d // 4, 16, 4), torch.zeros(pool, cfg.num_key_value_heads, d, 16))
              for _ in range(cfg.num_hidden_layers)]
    return bi, caches


def test_zero_output_projections_leave_the_embedding_stream():
    cfg = small_cfg()
    ws = rand_weights(cfg, 1)
    for i in range(cfg.num_hidden_layers):
        ws[f"model.layers.{i}.self_attn.o_proj"].zero_()
        ws[f"model.layers.{i}.mlp.down_proj"].zero_()
    seqs = [[3, 7, 9], [11], [2, 2, 2, 2, 5]]
    bi, caches = build(cfg, seqs)
    cos_sin = ref.rotary_table(16, cfg.rope_theta, 128, torch.float32)
    got = ollama.forward(cfg, ws, bi, caches, cos_sin)
    last = torch.tensor([s[-1] for s in seqs])
    want = plain_rms(ws["model.embed_tokens"][last], ws["model.norm"], cfg.rms_norm_eps) @ ws["lm_head"].t()
    assert got.shape == (3, cfg.vocab_size)
    assert torch.allclose(got, want, atol=1e-5)
    # the new tokens' K and V still reached every layer's cache: slot 0 of block 0 is token 0 of sequence 1
    assert all(kc.abs().sum() > 0 and vc.abs().sum() > 0 for kc, vc in caches)


def test_one_token_sequences_attend_to_themselves():
    # With a single token per sequence the softmax has one term, so the attention output is
    # that token's v, each kv head serving its group of query heads; with the MLP switched
    # off the block is x + o_proj(repeat(v)).  Rotary cannot matter (it never touches v).
    cfg = small_cfg(layers=1)
    ws = rand_weights(cfg, 2)
    ws["model.layers.0.mlp.down_proj"].zero_()
    seqs = [[4], [8], [15]]
    bi, caches = build(cfg, seqs)
    cos_sin = ref.rotary_table(16, cfg.rope_theta, 128, torch.float32)
    got = ollama.forward(cfg, ws, bi, caches, cos_sin)
    x = ws["model.embed_tokens"][torch.tensor([4, 8, 15])]
    h = plain_rms(x, ws["model.layers.0.input_layernorm"], cfg.rms_norm_eps)
    v = (h @ ws["model.layers.0.self_attn.v_proj"].t()).reshape(3, 2, 16)
    y = torch.stack([v[:, 0], v[:, 0], v[:, 1], v[:, 1]], dim=1).reshape(3, 64)   # 4 query heads on 2 kv heads
    x1 = y @ ws["model.layers.0.self_attn.o_proj"].t() + x
    want = plain_rms(x1, ws["model.norm"], cfg.rms_norm_eps) @ ws["lm_head"].t()
    assert torch.allclose(got, want, atol=1e-5)


def test_prefill_then_decode_equals_one_longer_prefill():
    # Causality across steps: logits of the last token do not depend on whether the earlier
    # tokens' K/V were computed in this step or read back from the cache.
    cfg = small_cfg()
    ws = rand_weights(cfg, 3)
    cos_sin = ref.rotary_table(16, cfg.rope_theta, 128, torch.float32)
    toks = [5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20, 21, 22]  # crosses a block boundary
    bi, caches = build(cfg, [toks])
    full = ollama.forward(cfg, ws, bi, caches, cos_sin)
    alloc = hostkv.BlockAllocator(16, 16)
    alloc.alloc_seq(1, len(toks) - 1)
    bi1 = hostkv.build_batch([hostkv.sched_entry(alloc, 1, toks[:-1], 0)], 16, 128, 0)
    d = 16
    caches2 = [(torch.zeros(16, 2, d // 4, 16, 4), torch.zeros(16, 2, d, 16)) for _ in range(2)]
    ollama.forward(cfg, ws, bi1, caches2, cos_sin)
    alloc.append_slots(1, len(toks) - 1, len(toks))
    bi2 = hostkv.build_batch([hostkv.sched_entry(alloc, 1, toks, len(toks) - 1)], 16, 128, 0)
    step = ollama.forward(cfg, ws, bi2, caches2, cos_sin)
    assert torch.allclose(step, full, atol=1e-5)
