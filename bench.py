"""Benchmark of the rLLM attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline (`value`): paged decode attention over the benchmark's decode configuration
(64 sequences, contexts U[512,4096], 32 q / 8 kv heads, d 128, bf16, block size 16, tables from
a shuffled 20k-block pool) as algorithmic HBM GB/s, with inputs resident in HBM.  One step = one
`paged_attention_v1` call over the batch (both of its kernels).  The block of `--steps` steps is
repeated until at least 100 ms have been timed; `value` is the median block, the spread is reported.
The same line carries the other configurations: `prefill` (8 x 4096 GQA causal varlen prefill,
TFLOP/s against the bf16 MFMA peak, with its own CPU baseline), `mixed_step` (the Phi-2-shaped
continuous-batching step), `llama_step` (the full Llama-3-8B-shaped decode step with the AICI mask),
`decode_c5_shape` (that step's decode attention alone, one layer, against the HBM roofline),
`memory_system` (what plain read / copy / fill kernels reach on this device) and `cpu_baseline`
(the oracle, i.e. rLLM's CPU reference route restated in torch-CPU, timed on a bounded sample of
the decode workload on this box's host cores).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16
# Figures bench.py cannot measure itself (hardware counters, single kernels of a multi-kernel step):
# taken from the rocprofv3 summaries under profiles/, which name the commands that made them.
PROFILED = {
    "decode_traffic_bytes": 642.7e6,      # FETCH_SIZE + WRITE_SIZE per decode step, scaled by a 1 GiB copy
    "decode_traffic_source": "profiles/decode_c2_prefill_c3_hbm_traffic.md",
    "decode_main_kernel_us": 101.9,       # paged_decode_flat_kernel, average duration in the kernel trace
    "decode_reduce_kernel_us": 4.7,       # paged_decode_flat_reduce_kernel
    "decode_kernels_source": "profiles/decode_c2_prefill_c3_kernel_trace.md",
    "prefill_traffic_bytes": 671.4e6,     # FETCH_SIZE + WRITE_SIZE per prefill launch, same scaling
    "prefill_traffic_source": "profiles/decode_c2_prefill_c3_hbm_traffic.md",
}
MIN_TIMED_MS = 100.0


def timed_blocks(fn, steps: int, min_total_ms: float = MIN_TIMED_MS, max_blocks: int = 400) -> list:
    """Wall time per step (ms) of blocks of exactly `steps` calls, each block bracketed by a device
    synchronisation on both sides; blocks are repeated until `min_total_ms` of timed work has run."""
    import torch

    per_step, total = [], 0.0
    while (total < min_total_ms or len(per_step) < 3) and len(per_step) < max_blocks:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        per_step.append(dt / steps)
        total += dt
    return per_step


def spread(xs: list) -> dict:
    import statistics

    return {"blocks": len(xs), "median": round(statistics.median(xs), 5), "min": round(min(xs), 5),
            "max": round(max(xs), 5)}


class PowerSampler:
    """Reads the card's power (W) from the amdgpu hwmon files every 20 ms on a thread of its own, where the box
    shows them; `mean(t0, t1)` is None where it does not."""

    def __init__(self):
        import glob

        dirs = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.file = next((os.path.join(d, "power1_input") for d in dirs if os.path.exists(os.path.join(d, "power1_input"))), None)
        self.cap_w = None
        if self.file:
            try:
                self.cap_w = int(open(os.path.join(os.path.dirname(self.file), "power1_cap")).read()) / 1e6
            except (OSError, ValueError):
                pass
        self.samples, self._stop, self._thread = [], False, None

    def _run(self):
        while not self._stop:
            try:
                self.samples.append((time.perf_counter(), int(open(self.file).read()) / 1e6))
            except (OSError, ValueError):
                return
            time.sleep(0.02)

    def __enter__(self):
        if self.file:
            import threading

            self._thread = threading.Thread(target=self._run, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self._thread:
            self._thread.join()

    def mean(self, t0: float, t1: float):
        xs = [w for (t, w) in self.samples if t0 <= t <= t1]
        return round(sum(xs) / len(xs), 0) if xs else None


def sustained(fn, seconds: float, est_ms: float, power: "PowerSampler") -> dict:
    """`fn` back to back for about `seconds`: time per call over the whole run and the card's mean power over its
    last two thirds.  Short timed runs start on a card that has been resting; this is what the same kernel does
    once the card's power management has settled."""
    import torch

    n = max(50, int(seconds * 1e3 / est_ms))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return {"launches": n, "ms_per_step": round((t1 - t0) * 1e3 / n, 4), "mean_power_w": power.mean(t0 + (t1 - t0) / 3, t1),
            "power_cap_w": power.cap_w}


def matrix_pipe_leg(dev, power: "PowerSampler") -> dict:
    """What the matrix pipes of this card give a kernel that does nothing but issue v_mfma_f32_32x32x16_bf16 (two
    wavefronts per SIMD on every compute unit, operands in registers), beside the published 2.5 PFLOP/s: after a
    short warm-up as the prefill leg is timed, and sustained; with operands of ones and with N(0,1) operands like
    the prefill leg's -- what the card's power management lets the pipes do depends on the values."""
    import torch
    from aici_amd import membench

    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    iters = 2000  # 32000 MFMAs per wavefront and launch
    out = {"kernel": "mfma_stream_kernel (csrc/bench/membench.hip), one workgroup of eight wavefronts per compute unit",
           "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s"}
    g = torch.Generator().manual_seed(23)
    for name in ("ones", "normal"):
        ops = (torch.ones(membench.MFMA_STREAM_OPERAND_ELEMS) if name == "ones"
               else torch.randn(membench.MFMA_STREAM_OPERAND_ELEMS, generator=g)).to(torch.bfloat16).to(dev)
        flop = [0.0]

        def fn():
            flop[0] = membench.mfma_stream(ops, cus, iters)

        time.sleep(0.5)  # from a rested card, like the legs before it
        for _ in range(25):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(50):
            fn()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / 50
        sus = sustained(fn, 1.5, ms, power)
        out[f"operands_{name}"] = {
            "after_25_launches": {"value": round(flop[0] / (ms * 1e-3) / 1e12, 1), "frac": round(flop[0] / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)},
            "sustained": {**sus, "value": round(flop[0] / (sus["ms_per_step"] * 1e-3) / 1e12, 1),
                          "frac": round(flop[0] / (sus["ms_per_step"] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}}
    return out


def host_cores() -> dict:
    """Cores this process may run on and cores the box reports (a container's share can be smaller); the CPU
    baselines run on every core the process may use, up to the thread count the box sets for such pools
    (OMP_NUM_THREADS), and say how many that was."""
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    cap = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    threads = min(usable, cap) if cap > 0 else usable
    return {"usable": usable, "reported": os.cpu_count() or 1, "omp_num_threads": cap or None, "threads_used": max(1, threads)}


def cpu_baseline_prefill(p_cpu, seq: int, threads: int) -> dict:
    """The oracle's varlen attention (repeat_kv -> per-sequence fp32 SDPA with an additive causal bias, the
    route of rLLM's CPU build) on one of the prefill configuration's sequences."""
    import torch

    from oracle import refkernels as ref

    torch.set_num_threads(threads)
    L = p_cpu.lens_q[seq]
    a, b = int(p_cpu.cu_q[seq]), int(p_cpu.cu_q[seq + 1])
    q, k, v = p_cpu.q[a:b].float(), p_cpu.k[a:b].float(), p_cpu.v[a:b].float()
    n_rep = q.shape[1] // k.shape[1]
    cu = torch.tensor([0, L], dtype=torch.int32)
    reps, dt = 0, 0.0
    t0 = time.perf_counter()
    while dt < 10.0:  # a bounded sample: about 10 s of CPU work
        ref.varlen_attn(q, ref.repeat_kv(k, n_rep), ref.repeat_kv(v, n_rep), cu, cu, L, L, p_cpu.scale, True)
        reps += 1
        dt = time.perf_counter() - t0
    dt /= reps
    flops = 4.0 * q.shape[2] * q.shape[1] * (L * (L + 1) // 2)
    return {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"sequence {seq} of {len(p_cpu.lens_q)} ({L} tokens; every sequence costs the same), {reps} "
                      f"passes of {dt:.2f} s; flops counted as for the GPU (unmasked pairs only, although the CPU "
                      "route computes the full L x L products)"}



def event_times_ms(fn, steps: int, stream) -> list:
    """Per-launch durations from HIP events recorded on the stream the kernels run on."""
    import torch

    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        a.record(stream)
        fn()
        b.record(stream)
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


def event_blocks_ms(fn, steps: int, stream, min_total_ms: float = MIN_TIMED_MS, max_blocks: int = 400) -> list:
    """Duration per step (ms) of blocks of `steps` back-to-back calls, each block between two HIP events
    recorded on the stream the kernels run on (an event between every two calls would hold the next launch
    back by about 3 us); blocks are repeated until `min_total_ms` have been timed."""
    import torch

    per_step, total = [], 0.0
    while (total < min_total_ms or len(per_step) < 3) and len(per_step) < max_blocks:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for _ in range(steps):
            fn()
        b.record(stream)
        torch.cuda.synchronize()
        dt = a.elapsed_time(b)
        per_step.append(dt / steps)
        total += dt
    return per_step


def cpu_baseline_decode(c_cpu, rows, threads: int) -> dict:
    """The oracle (gather_cached_kv -> repeat_kv -> Lq=1 varlen SDPA in fp32, the route rLLM's CPU
    build takes) on a sample of the sequences."""
    import torch

    from oracle import refkernels as ref

    torch.set_num_threads(threads)
    q = c_cpu.q[rows].float()
    kc, vc = c_cpu.key_cache.float(), c_cpu.value_cache.float()
    bt, cl = c_cpu.block_tables[rows], c_cpu.context_lens[rows]
    reps, dt = 0, 0.0
    t0 = time.perf_counter()
    while dt < 12.0:  # a bounded sample: about 12 s of CPU work
        ref.paged_attention(q, kc, vc, c_cpu.num_kv_heads, c_cpu.scale, bt, cl, 16)
        reps += 1
        dt = time.perf_counter() - t0
    dt /= reps
    elt = c_cpu.q.element_size()
    tokens = int(cl.sum())
    nbytes = tokens * 2 * c_cpu.num_kv_heads * c_cpu.q.shape[2] * elt + 2 * len(rows) * q.shape[1] * q.shape[2] * elt
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{len(rows)} of {c_cpu.q.shape[0]} sequences ({tokens} context tokens), {reps} passes of {dt:.2f} s; "
                      "bytes counted as for the GPU (bf16 K/V once per kv head)"}


def memory_system_leg(dev, stream, steps: int) -> dict:
    """What this device's memory system delivers to the simplest possible kernels (16 bytes per lane,
    grid-stride), beside the published 8 TB/s: a 1 GiB read, a 1 GiB copy, a 1 GiB fill, and the read of
    a 1.3 GB buffer in shuffled 4 KiB chunks -- the granule and footprint of the decode leg's K/V blocks."""
    import torch
    from aici_amd import membench

    n = 1 << 30
    src = torch.empty((n,), dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    big = torch.empty((20000 * 16 * 4096,), dtype=torch.uint8, device=dev).fill_(1)  # 20k blocks x 8 heads x (K, V)
    g = torch.Generator().manual_seed(17)
    order = torch.randperm(big.numel() // 4096, generator=g)[:154_000].to(torch.int32).to(dev)  # ~631 MB of distinct chunks
    out = {}

    def run(name, fn, nbytes):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        ts = event_times_ms(fn, steps, stream)
        ms = sum(ts) / len(ts)
        out[name] = {"GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1), "us": round(ms * 1e3, 1), "bytes": nbytes}

    run("read_1GiB", lambda: membench.probe("read", None, src), n)
    run("copy_1GiB_read_plus_write", lambda: membench.probe("copy", dst, src), 2 * n)
    run("fill_1GiB", lambda: membench.probe("fill", dst, None), n)
    run("read_4KiB_chunks_shuffled", lambda: membench.probe("read_chunks", None, big, order), order.numel() * 4096)
    # the same with the non-temporal hint on every load and store (what the decode kernels' cache loads carry)
    run("read_1GiB_nontemporal", lambda: membench.probe("read", None, src, nontemporal=True), n)
    run("copy_1GiB_read_plus_write_nontemporal", lambda: membench.probe("copy", dst, src, nontemporal=True), 2 * n)
    run("fill_1GiB_nontemporal", lambda: membench.probe("fill", dst, None, nontemporal=True), n)
    run("read_4KiB_chunks_shuffled_nontemporal",
        lambda: membench.probe("read_chunks", None, big, order, nontemporal=True), order.numel() * 4096)
    # the same amount in larger granules: what reading several kv heads of a block as one piece could give
    for kib in (16, 32):
        cb = kib * 1024
        order_k = torch.randperm(big.numel() // cb, generator=g)[:154_000 * 4096 // cb].to(torch.int32).to(dev)
        run(f"read_{kib}KiB_chunks_shuffled", lambda: membench.probe("read_chunks", None, big, order_k, cb),
            order_k.numel() * cb)
    return out


def streaming_leg(dev, stream, steps: int) -> dict:
    """The HBM-bound helpers of the path at the sizes of the prefill (config 3: 32768 tokens) and of the
    full decode step (config 5: 128 x 128256 logits): algorithmic bytes / average launch time (HIP events)."""
    import numpy as np
    import torch

    from aici_amd import kernels as K
    from aici_amd import paged
    from aici_amd import workloads as W
    from aici_amd.attn import RotaryEmbedding

    bf = torch.bfloat16
    res = {}

    def run(name, fn, nbytes):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        ms = event_times_ms(fn, steps, stream)
        ms = sum(ms) / len(ms)
        res[name] = {"us": round(ms * 1e3, 2), "bytes": int(nbytes), "gbs": round(nbytes / ms / 1e6, 1),
                     "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}

    T, H, d, nb = 32768, 8, 128, 2304
    k = torch.randn(T, H, d, device=dev, dtype=bf)
    v = torch.randn(T, H, d, device=dev, dtype=bf)
    kc, vc = paged.alloc_gpu_cache_layer(nb, H, d, 16, bf, dev)
    blocks = torch.randperm(nb, device=dev)[:T // 16]
    slots = (blocks.repeat_interleave(16) * 16 + torch.arange(T, device=dev) % 16).to(torch.int64)
    run("reshape_and_cache 32768 tok x 8 kv heads x 128", lambda: K.reshape_and_cache(k, v, kc, vc, slots),
        2 * 2 * T * H * d * 2 + 8 * T)
    s32 = slots.to(torch.int32)
    ko, vo = torch.empty_like(k), torch.empty_like(v)
    run("gather_cached_kv 32768 tok x 8 kv heads x 128", lambda: K.gather_cached_kv(ko, vo, kc, vc, s32),
        2 * 2 * T * H * d * 2 + 4 * T)
    q2 = torch.randn(T, 32 * 128, device=dev, dtype=bf)
    k2 = torch.randn(T, 8 * 128, device=dev, dtype=bf)
    pos = torch.arange(T, device=dev, dtype=torch.int64) % 4096
    cs = RotaryEmbedding.build_table(128, 500000.0, 4096, bf).to(dev)
    run("rotary_embedding 32768 tok, 32+8 heads x 128", lambda: K.rotary_embedding(pos, q2, k2, 128, cs, True),
        2 * T * (32 + 8) * 128 * 2)
    x = torch.randn(T, 4096, device=dev, dtype=bf)
    w = torch.randn(4096, device=dev, dtype=bf)
    o = torch.empty_like(x)
    run("rms_norm 32768 x 4096", lambda: K.rms_norm(o, x, w, 1e-5), 2 * T * 4096 * 2)
    r = torch.randn(T, 4096, device=dev, dtype=bf)
    run("fused_add_rms_norm 32768 x 4096", lambda: K.fused_add_rms_norm(x, r, w, 1e-5), 4 * T * 4096 * 2)
    gu = torch.randn(T, 2 * 14336, device=dev, dtype=bf)
    act = torch.empty(T, 14336, device=dev, dtype=bf)
    run("silu_and_mul 32768 x 14336", lambda: K.silu_and_mul(act, gu), 3 * T * 14336 * 2)
    del k, v, kc, vc, ko, vo, q2, k2, x, o, r, gu, act
    S, V = 128, 128256
    lg = torch.randn(S, V, device=dev, dtype=bf)
    allowed = W.allow_mask(5, S, V)
    mask = torch.from_numpy(np.packbits(np.pad(allowed, ((0, 0), (0, (-V) % 32))), axis=1, bitorder="little")).to(dev)
    run("bias_argmax 128 x 128256, packed allow-bits", lambda: K.bias_argmax(lg, mask=mask), S * V * 2 + mask.numel())
    temp = torch.full((S,), 0.8, device=dev)
    u = torch.rand((S,), device=dev)
    for tp in (1.0, 0.9):
        top_p = torch.full((S,), tp, device=dev)
        run(f"bias_sample 128 x 128256, packed allow-bits, temperature 0.8, top_p {tp} (algorithmic bytes: one pass)",
            lambda: K.bias_sample(lg, temp, top_p, u, mask=mask), S * V * 2 + mask.numel())
    row = (V + 1000) & ~63
    bias = torch.full((S, row), float("-inf"), dtype=torch.float32, device=dev)
    bias[:, :V][torch.from_numpy(allowed).to(dev)] = 0.0
    run("bias_argmax 128 x 128256, f32 bias rows", lambda: K.bias_argmax(lg, bias=bias), S * V * 2 + S * V * 4)
    return res


def mixed_step_leg(dev, stream, steps: int) -> dict:
    """One layer's attention for a mixed continuous-batching step in the Phi-2 shape (32 MHA heads, d 80,
    fp16): four 512-token chunks with 0/1k/2k/3k tokens already cached plus 120 single-token rows with
    contexts U[1k,8k] (seed 4) -- `llm::varlen_attn` as one C-ABI call, by the reference's route (scatter,
    gather, varlen prefill, paged decode) and with the multi-token rows reading the cache through block tables."""
    import math

    import numpy as np
    import torch

    from aici_amd import attn, paged

    rng = np.random.default_rng(4)
    H, d, dt = 32, 80, torch.float16
    priors, chunk = [0, 1024, 2048, 3072], 512
    dec = rng.integers(1024, 8193, size=120).tolist()
    pool = sum((p + chunk + 15) // 16 for p in priors) + sum((c + 15) // 16 for c in dec) + 8
    alloc = paged.BlockAllocator(16, pool)
    b = paged.BatchInfoBuilder(16, 1 << 20, 1)
    sid = 1
    for p in priors:
        alloc.alloc_seq(sid, p + chunk)
        b.sched_out(alloc, sid, rng.integers(0, 1000, size=p + chunk).astype(np.int32), p)
        sid += 1
    for c in dec:
        alloc.alloc_seq(sid, c)
        b.sched_out(alloc, sid, rng.integers(0, 1000, size=c).astype(np.int32), c - 1)
        sid += 1
    bi = b.finish().to(dev)
    T = bi.tokens.numel()
    g = torch.Generator(device=dev).manual_seed(4)
    kc, vc = paged.alloc_gpu_cache_layer(pool, H, d, 16, dt, dev)
    kc.normal_(generator=g)
    vc.normal_(generator=g)
    q, k, v = (torch.randn((T, H, d), generator=g, device=dev, dtype=dt) for _ in range(3))
    flops = 4 * d * H * sum(chunk * p + chunk * (chunk + 1) // 2 for p in priors)
    kv_bytes = int(sum(dec)) * 2 * H * d * 2
    out = {"config": {"workload": "mixed step: 4 x 512 new tokens after 0/1k/2k/3k cached + 120 decode rows ctx "
                                  "U[1k,8k] (seed 4), 32 MHA heads, d 80, fp16", "tokens": T,
                      "prefill_flops": flops, "decode_kv_bytes": kv_bytes}}
    for name, paged_prefill in (("reference_route", False), ("paged_prefill_route", True)):
        fn = lambda: attn.varlen_attn(q, k, v, bi, kc, vc, 1.0 / math.sqrt(d), paged_prefill=paged_prefill)
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        ms = event_times_ms(fn, steps, stream)
        out[name] = {"us_per_step": round(sum(ms) / len(ms) * 1e3, 1)}
    # The two attention kernels of the step on their own (the same calls the composition makes, on the cache the
    # step above has filled), each against its roofline: the chunks against the fp16 MFMA peak, the decode rows
    # against the HBM peak.
    from aici_amd import kernels as K
    scale = 1.0 / math.sqrt(d)
    qm = q[:bi.q_multi]
    chunks = lambda: K.flash_attn_varlen_paged(qm, kc, vc, bi.multi_block_tables, bi.seqlens_q, bi.multi_context_lens,
                                               bi.max_seqlen_q, bi.max_seqlen_k, scale, True)
    qd, o_d = q[bi.q_multi:], torch.empty_like(q[bi.q_multi:])
    # the decode rows cycle through three copies of the cache, so that no launch finds in the 256 MB Infinity Cache
    # what the launch before it left there (a single 6 GB cache re-read at once would: up to 4 % of its bytes)
    row_caches = [(kc, vc), (kc.clone(), vc.clone()), (kc.clone(), vc.clone())]
    turn = [0]

    def rows():
        kcr, vcr = row_caches[turn[0] % 3]
        turn[0] += 1
        K.paged_attention_v1(o_d, qd, kcr, vcr, H, scale, bi.paged_block_tables, bi.paged_context_lens, 16,
                             bi.paged_max_context_len)
    dec_bytes = kv_bytes + 2 * len(dec) * H * d * 2 + 4 * sum((c + 15) // 16 for c in dec) + 4 * len(dec)
    for fn in (chunks, rows):
        for _ in range(10):
            fn()
    torch.cuda.synchronize()
    ms_c = event_blocks_ms(chunks, max(steps, 10), stream)
    ms_r = event_blocks_ms(rows, max(steps, 10), stream)
    import statistics
    mc, mr = statistics.median(ms_c), statistics.median(ms_r)
    out["prefill_chunks"] = {"us": round(mc * 1e3, 1), "roofline": {
        "bound": "mfma", "achieved": round(flops / (mc * 1e-3) / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(flops / (mc * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
        "kernel": "hipattn_mha_varlen_fwd_paged (block images), 4 x 512 rows, d 80 in the 96-wide instance"}}
    out["decode_rows"] = {"us": round(mr * 1e3, 1), "algorithmic_bytes": dec_bytes, "roofline": {
        "bound": "hbm", "achieved": round(dec_bytes / (mr * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(dec_bytes / (mr * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
        "kernel": "paged_attention_v1, whole call (main + merge kernel), 120 rows, MHA d 80; three copies of the "
                  "cache in turns"}}
    del row_caches
    return out


def decode_c5_shape_leg(dev, stream, steps: int) -> dict:
    """The decode attention of the full-model configuration at its own shape, one layer: 128 sequences with
    contexts U[1024, 16384] (seed 5), 32 q / 8 kv heads, d 128, bf16, block tables over a shuffled pool -- the
    whole `paged_attention_v1` call (main + merge kernel) as algorithmic HBM GB/s."""
    import statistics

    import numpy as np
    import torch

    from aici_amd import kernels as K
    from aici_amd import workloads as W

    rng = np.random.default_rng(5)
    S = 128
    ctx = rng.integers(1024, 16384 + 1, size=S)
    pool = int(((ctx + 15) // 16).sum()) + 64
    c = W.decode_inputs(5, S, 1024, 16384, 32, 8, 128, torch.bfloat16, pool, device=dev)
    out = torch.empty_like(c.q)
    # three copies of the 4.5 GB cache in turns, as a step's 32 layers each read their own: a single cache read
    # again at once finds up to 256 MB of itself (5.7 %) still in the Infinity Cache
    caches = [(c.key_cache, c.value_cache)] + [(c.key_cache.clone(), c.value_cache.clone()) for _ in range(2)]
    turn = [0]

    def fn():
        kc, vc = caches[turn[0] % 3]
        turn[0] += 1
        K.paged_attention_v1(out, c.q, kc, vc, 8, c.scale, c.block_tables, c.context_lens, 16, c.max_ctx)

    for _ in range(6):
        fn()
    torch.cuda.synchronize()
    ms = statistics.median(event_blocks_ms(fn, max(steps, 10), stream))
    nbytes = c.algorithmic_bytes()
    return {"us_per_step": round(ms * 1e3, 1), "algorithmic_bytes": nbytes,
            "roofline": {"bound": "hbm", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                         "kernel": "paged_attention_v1, whole call (main + merge kernel); three copies of the cache in turns"},
            "config": {"workload": "paged decode attention, 128 seqs, ctx U[1024,16384] (seed 5), 32q/8kv heads, d128, "
                                   "bf16, block 16, one layer", "context_tokens": int(ctx.sum())}}


def llama_step_leg(dev, stream, steps: int, layers: int, share_cache: bool) -> dict:
    """One full engine step of a Llama-3-8B-shaped model (random weights): 128 sequences decoding
    one token each over contexts U[1024,16384] (seed 5), every layer with its own paged KV cache,
    then the AICI step (5 % of the vocabulary allowed per sequence, packed bit masks) and greedy
    arg-max.  q/k/v, gate/up and lm_head are library GEMMs; o_proj and down_proj (few rows of the weight: a
    library GEMM leaves most of the device idle) and everything else run through the C ABI.
    `ms_per_step_library_gemms_only` is the same step with those two projections as library GEMMs as well."""
    import numpy as np
    import torch

    from aici_amd import llama, paged
    from aici_amd import workloads as W

    cfg = llama.LlamaConfig.llama3_8b()
    cfg.num_hidden_layers = layers
    rng = np.random.default_rng(5)
    S = 128
    ctx = rng.integers(1024, 16384 + 1, size=S)
    pool = int(((ctx + 15) // 16).sum()) + 64
    alloc = paged.BlockAllocator(16, pool)
    builder = paged.BatchInfoBuilder(16, cfg.max_position_embeddings, 1)
    for sid, n in enumerate(ctx.tolist(), start=1):
        alloc.alloc_seq(sid, n)
        builder.sched_out(alloc, sid, rng.integers(0, cfg.vocab_size, size=n).astype(np.int32), n - 1)
    bi = builder.finish().to(dev)
    model = llama.Llama(cfg, llama.random_weights(cfg, 5, device=dev), dev)
    g = torch.Generator(device=dev).manual_seed(5)
    caches = []
    for i in range(layers):
        if share_cache and i > 0:
            caches.append(caches[0])
            continue
        kc, vc = paged.alloc_gpu_cache_layer(pool, cfg.num_key_value_heads, cfg.head_dim, 16, cfg.dtype, dev)
        kc.normal_(generator=g)
        vc.normal_(generator=g)
        caches.append((kc, vc))
    allowed = W.allow_mask(5, S, cfg.vocab_size)
    masks = torch.from_numpy(np.packbits(np.pad(allowed, ((0, 0), (0, (-cfg.vocab_size) % 32))), axis=1,
                                         bitorder="little")).to(dev)

    def step(fused=True):
        return llama.aici_greedy(model.forward(bi, caches, fused=fused), masks)

    for _ in range(2):
        toks = step()
    torch.cuda.synchronize()
    ok = bool(torch.from_numpy(allowed)[torch.arange(S), toks.cpu().long()].all())
    # the reference's call sequence (q, k, v copied out of the projection, rotary and cache scatter apart)
    same = bool(torch.equal(toks, step(False)))
    ms_ref = event_times_ms(lambda: step(False), steps, stream)
    ms_ref = sum(ms_ref) / len(ms_ref)
    model.skinny_linear = False
    # different summation orders, random weights: near-ties may fall the other way, so a count, not a check
    equal_lib = int((toks == step()).sum())
    ms_lib = event_times_ms(step, steps, stream)
    ms_lib = sum(ms_lib) / len(ms_lib)
    model.skinny_linear = True
    step()
    ms = event_times_ms(step, steps, stream)
    ms = sum(ms) / len(ms)
    # the same step captured once in a HIP graph and replayed: no launch gaps between its ~400 kernels
    ms_graph, same_graph = None, None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):  # the stream whose scratch buffers the warm-up step sized
            toks_graph = step()
        graph.replay()
        torch.cuda.synchronize()
        same_graph = bool(torch.equal(toks_graph, toks))
        ms_graph = event_times_ms(graph.replay, steps, stream)
        ms_graph = round(sum(ms_graph) / len(ms_graph), 3)
    except Exception as e:  # reported, not fatal: the eager figures above stand on their own
        ms_graph = f"capture failed: {type(e).__name__}: {e}"[:200]
    elt = 2
    kv_bytes = int(ctx.sum()) * 2 * cfg.num_key_value_heads * cfg.head_dim * elt * layers
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    kvd = cfg.num_key_value_heads * cfg.head_dim
    weight_bytes = elt * (layers * (H * (H + 2 * kvd) + H * H + 3 * H * I) + V * H)
    return {"ms_per_step": round(ms, 3), "steps": steps, "tokens_per_s": round(S / (ms * 1e-3), 1),
            "kv_bytes_per_step": kv_bytes, "weight_bytes_per_step": weight_bytes,
            "hbm_gbs": round((kv_bytes + weight_bytes) / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round((kv_bytes + weight_bytes) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "constrained_tokens_all_allowed": ok,
            "ms_per_step_reference_call_sequence": round(ms_ref, 3), "same_tokens_either_way": same,
            "ms_per_step_library_gemms_only": round(ms_lib, 3), "tokens_equal_with_library_gemms": f"{equal_lib} of {S}",
            "ms_per_step_hip_graph_replay": ms_graph, "same_tokens_from_graph": same_graph,
            "config": {"workload": f"Llama-3-8B-shaped decode step, {layers} layers, 128 seqs, ctx U[1024,16384] "
                                   "(seed 5), bf16, per-layer paged KV"
                                   + (" (one cache shared by all layers)" if share_cache else "")
                                   + ", AICI 5% allow-mask + greedy",
                       "context_tokens": int(ctx.sum())}}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--kv-pools", type=int, default=3, help="copies of the KV pool cycled through by the decode leg")
    ap.add_argument("--streaming", action="store_true",
                    help="also time the HBM-bound helper kernels (cache scatter/gather, rotary, norms, "
                         "activation, bias + arg-max) against the HBM roofline")
    ap.add_argument("--no-mixed-step", action="store_true",
                    help="skip one layer's attention for the mixed prefill-chunk + decode step (Phi-2 shape)")
    ap.add_argument("--no-llama-step", action="store_true",
                    help="skip the full Llama-3-8B-shaped decode step with the AICI mask + greedy stage "
                         "(it allocates about 170 GB of HBM)")
    ap.add_argument("--no-short-rows", action="store_true",
                    help="drop the 16 x 2048-token prefill leg (two kernels in turns): keeps a kernel trace's prefill "
                         "row to the headline configuration")
    ap.add_argument("--no-decode-c5-shape", action="store_true",
                    help="skip the decode attention of the full-model configuration at its own shape (one layer)")
    ap.add_argument("--mixed-step", action="store_true", help="(default; kept for old command lines)")
    ap.add_argument("--llama-step", action="store_true", help="(default; kept for old command lines)")
    ap.add_argument("--llama-layers", type=int, default=32)
    ap.add_argument("--llama-share-cache", action="store_true",
                    help="all layers read one layer's KV cache (taken by itself when the device is short of memory)")
    ap.add_argument("--no-memory-system", action="store_true",
                    help="skip the plain read / copy / fill kernels and the shuffled 4 KiB-chunk read (the "
                         "attainable rates reported beside the 8 TB/s peak)")
    ap.add_argument("--memory-system", action="store_true", help="(default; kept for old command lines)")
    ap.add_argument("--no-sustained", action="store_true",
                    help="skip the runs of about 1.5 s each (prefill, and a bare stream of MFMAs) that show what the card "
                         "holds once its power management has settled, with the card's power beside them")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (torch copy_) so that FETCH_SIZE / WRITE_SIZE "
                         "read under rocprofv3 --pmc can be scaled against a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the attention path has no cross-GPU step in this build "
                 "(run with --gpus 1)")
    import torch

    from aici_amd import kernels as K
    from aici_amd import workloads as W
    from aici_amd import paged

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream(dev)
    K.init()

    # ---- decode leg (headline) ------------------------------------------------------------
    c_cpu = W.config2()
    c = c_cpu.to(dev)
    out = torch.empty_like(c.q)
    # Several copies of the KV pool, used round-robin: between two uses of one copy
    # (pools - 1) x 1.3 GB of other K/V pass through the 256 MB Infinity Cache, so every
    # step really streams its 634 MB from HBM.
    pools = [(c.key_cache, c.value_cache)] + [(c.key_cache.clone(), c.value_cache.clone())
                                              for _ in range(args.kv_pools - 1)]
    step_no = [0]

    def decode_step():
        kc, vc = pools[step_no[0] % len(pools)]
        step_no[0] += 1
        K.paged_attention_v1(out, c.q, kc, vc, c.num_kv_heads, c.scale, c.block_tables, c.context_lens, 16,
                             c.max_ctx)

    for _ in range(max(args.warmup, 1)):
        decode_step()
    wall = timed_blocks(decode_step, args.steps)
    import statistics

    wall_ms = statistics.median(wall)
    # HIP events on the launch stream around blocks of steps (both kernels of every call), and around every call
    block_ms = event_blocks_ms(decode_step, args.steps, stream)
    avg_step_ms = sum(block_ms) / len(block_ms)
    call_ms = event_times_ms(decode_step, max(args.steps, 100), stream)
    nbytes = c_cpu.algorithmic_bytes()
    value = nbytes / (wall_ms * 1e-3) / 1e9
    achieved = nbytes / (avg_step_ms * 1e-3) / 1e9
    main_us = PROFILED["decode_main_kernel_us"]

    line = {
        "metric": "prefill attn TFLOP/s + paged-decode attn HBM GB/s (1 GPU, % roofline)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "ms_per_step_spread": spread(wall),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "paged decode attention: 64 seqs, ctx U[512,4096] (seed 2), 32 q / 8 kv heads, "
                               "d 128, bf16, block 16, tables from a shuffled 20k-block pool",
                   "algorithmic_bytes_per_step": nbytes,
                   "context_tokens": int(c_cpu.context_lens.sum()), "kv_pool_copies": len(pools)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": PROFILED["decode_traffic_bytes"],
                     "traffic_source": PROFILED["decode_traffic_source"],
                     "kernel": "the whole decode step: paged_decode_flat_kernel + paged_decode_flat_reduce_kernel, "
                               "HIP events on the launch stream around blocks of `steps` calls",
                     "avg_step_us": round(avg_step_ms * 1e3, 2),
                     "avg_step_us_with_an_event_between_calls": round(sum(call_ms) / len(call_ms) * 1e3, 2),
                     "dominant_kernel_alone": {
                         "kernel": "paged_decode_flat_kernel", "avg_launch_us": main_us,
                         "achieved": round(nbytes / main_us / 1e3, 1),
                         "frac": round(nbytes / main_us / 1e3 / HBM_PEAK_GBS, 4),
                         "source": PROFILED["decode_kernels_source"] + " (rocprofv3 kernel trace of this command; "
                                   "not measured in this run)"}},
        "host_cores": host_cores(),
    }

    if not args.no_sustained:
        # the same step for about a second, with the card's power beside it (a memory-bound step leaves the card
        # well inside its power limit; the prefill leg below does not)
        with PowerSampler() as power:
            sus = sustained(decode_step, 1.0, avg_step_ms, power)
        line["roofline"]["sustained"] = {**sus, "achieved": round(nbytes / (sus["ms_per_step"] * 1e-3) / 1e9, 1),
                                         "frac": round(nbytes / (sus["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if args.copy_calibration:
        src = torch.empty((1 << 30,), dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"bytes_read": 1 << 30, "bytes_written": 1 << 30, "launches": 3}
        del src, dst

    # ---- prefill leg ------------------------------------------------------------------------
    if not args.no_prefill:
        p_cpu = W.config3(1.0)
        p = p_cpu.to(dev)

        def prefill_step():
            K.flash_attn_varlen(p.q, p.k, p.v, p.cu_q, p.cu_k, p.max_q, p.max_k, p.scale, True)

        # The part raises its clock over the first tens of milliseconds of MFMA load: warm up for that long.
        psteps = max(3, min(args.steps, 50))
        for _ in range(max(25, args.warmup)):
            prefill_step()
        pwall = timed_blocks(prefill_step, psteps)
        pl = event_times_ms(prefill_step, psteps, stream)
        pms = sum(pl) / len(pl)
        tflops = p.flops() / (pms * 1e-3) / 1e12
        line["prefill"] = {
            "value": round(p.flops() / (statistics.median(pwall) * 1e-3) / 1e12, 1), "unit": "TFLOP/s",
            "ms_per_step": round(statistics.median(pwall), 4), "ms_per_step_spread": spread(pwall), "steps": psteps,
            "config": {"workload": "varlen causal prefill: 8 x 4096 tokens, 32 q / 8 kv heads, d 128, bf16, N(0,1)",
                       "algorithmic_flops_per_step": p.flops()},
            "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                         "traffic": PROFILED["prefill_traffic_bytes"], "traffic_source": PROFILED["prefill_traffic_source"],
                         "kernel": "prefill_varlen_w8_kernel, HIP events on the launch stream",
                         "avg_launch_us": round(pms * 1e3, 1)},
        }
        if not args.no_sustained:
            # ... and once the card's power management has settled: about 1.5 s of launches back to back
            with PowerSampler() as power:
                sus = sustained(prefill_step, 1.5, pms, power)
            sus_tf = p.flops() / (sus["ms_per_step"] * 1e-3) / 1e12
            line["prefill"]["sustained"] = {**sus, "value": round(sus_tf, 1), "unit": "TFLOP/s",
                                            "frac": round(sus_tf / MFMA_BF16_PEAK_TFLOPS, 4)}
            time.sleep(0.5)
        # The same rows with K/V read from the paged cache they were scattered into (what an engine step
        # has at hand: rLLM writes the cache first, llm/mod.rs:147-164, and gathers back from it).
        nb = sum((l + 15) // 16 for l in p.lens_k)
        perm = torch.randperm(nb + 64, generator=torch.Generator().manual_seed(3)).tolist()
        tables = torch.zeros((len(p.lens_k), max((l + 15) // 16 for l in p.lens_k)), dtype=torch.int32)
        slots, pos = [], 0
        for i, l in enumerate(p.lens_k):
            n = (l + 15) // 16
            tables[i, :n] = torch.tensor(perm[pos:pos + n], dtype=torch.int32)
            slots += W.slots_for(perm[pos:pos + n], l)
            pos += n
        kc, vc = paged.alloc_gpu_cache_layer(nb + 64, p.k.shape[1], p.k.shape[2], 16, p.k.dtype, dev)
        K.reshape_and_cache(p.k, p.v, kc, vc, torch.tensor(slots, dtype=torch.int64, device=dev))
        tb, ctx = tables.to(dev), torch.tensor(p.lens_k, dtype=torch.int32, device=dev)

        def paged_step():
            K.flash_attn_varlen_paged(p.q, kc, vc, tb, p.cu_q, ctx, p.max_q, p.max_k, p.scale, True)

        for _ in range(10):
            paged_step()
        torch.cuda.synchronize()
        ql = event_times_ms(paged_step, max(psteps, 90), stream)
        qms = sum(ql) / len(ql)
        line["prefill"]["from_paged_cache"] = {
            "value": round(p.flops() / (qms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "ms_per_step": round(qms, 4),
            "frac": round(p.flops() / (qms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "kernel": "prefill_varlen_w8_kernel, block images copied global -> LDS (hipattn_mha_varlen_fwd_paged)"}
        del p, kc, vc
        if not args.no_short_rows:
            # The same number of tokens in sequences half as long, on the library's choice of kernel (eight
            # wavefronts) and on the kernel that rotates three groups of four wavefronts through the matrix pipe;
            # the two take turns, because whichever runs later finds the part at a higher clock.
            p = W.config3(1.0, batch=16, L=2048).to(dev)
            for _ in range(40):
                prefill_step()
            turns = {0: [], 4: []}
            try:
                for rnd in range(6):
                    for kern in ((0, 4) if rnd % 2 == 0 else (4, 0)):
                        K.tuning_set("prefill_kernel", kern)
                        prefill_step()
                        prefill_step()
                        turns[kern].append(sum(event_times_ms(prefill_step, 20, stream)) / 20)
            finally:
                K.tuning_set("prefill_kernel", 0)
            sms, rms = statistics.median(turns[0]), statistics.median(turns[4])
            line["prefill"]["rows_of_2048"] = {
                "value": round(p.flops() / (sms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "ms_per_step": round(sms, 4),
                "frac": round(p.flops() / (sms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                "config": {"workload": "varlen causal prefill: 16 x 2048 tokens, 32 q / 8 kv heads, d 128, bf16, N(0,1)",
                           "algorithmic_flops_per_step": p.flops()},
                "kernel": "prefill_varlen_w8_kernel (the library's choice), HIP events on the launch stream",
                "three_group_kernel_forced": {
                    "kernel": "prefill_varlen_r3_kernel (prefill_kernel = 4)", "ms_per_step": round(rms, 4),
                    "value": round(p.flops() / (rms * 1e-3) / 1e12, 1), "unit": "TFLOP/s"}}
            del p

        if not args.no_sustained:
            with PowerSampler() as power:
                line["prefill"]["matrix_pipe"] = matrix_pipe_leg(dev, power)

    # ---- optional: the streaming helpers -------------------------------------------------------------
    if args.streaming:
        line["streaming"] = streaming_leg(dev, stream, max(20, min(args.steps, 100)))

    if not args.no_memory_system:
        line["memory_system"] = memory_system_leg(dev, stream, 100)

    if not args.no_mixed_step:
        line["mixed_step"] = mixed_step_leg(dev, stream, max(100, args.steps))

    if not args.no_decode_c5_shape:
        line["decode_c5_shape"] = decode_c5_shape_leg(dev, stream, args.steps)

    # ---- the full engine step the decode kernel sits in -------------------------------------------
    if not args.no_llama_step:
        del pools, c
        torch.cuda.empty_cache()
        free_b, _total = torch.cuda.mem_get_info(dev)
        need = 175e9 * args.llama_layers / 32
        share = args.llama_share_cache or free_b < need
        try:
            line["llama_step"] = llama_step_leg(dev, stream, max(4, min(args.steps, 10)), args.llama_layers, share)
            if share and not args.llama_share_cache:
                line["llama_step"]["note"] = (f"one KV cache shared by all layers: {free_b / 1e9:.0f} GB free on the "
                                              f"device, {need / 1e9:.0f} GB needed for a cache per layer")
        except torch.OutOfMemoryError as e:
            line["llama_step"] = {"skipped": f"out of device memory: {str(e)[:160]}"}
        torch.cuda.empty_cache()

    # ---- CPU baselines: the reference's CPU route on this box's host cores ------------------------
    if not args.no_cpu_baseline:
        threads = host_cores()["threads_used"]
        line["cpu_baseline"] = cpu_baseline_decode(c_cpu, list(range(0, 64, 2)), threads)
        if "prefill" in line:
            line["prefill"]["cpu_baseline"] = cpu_baseline_prefill(p_cpu, 0, threads)

    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
