#!/usr/bin/env python3
"""Benchmark of the paged KV-cache attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one decode step of one layer over the synthetic batch of BASELINE.json
configs[1]: 64 sequences, contexts uniform in [1024, 8192], 32 query / 8 kv heads, head_dim
128, page 16, pages drawn from a seeded permutation of a 65536-page pool; every step appends
one token per sequence (split + RoPE, append scatter) and runs split-KV decode attention.
All inputs, page tables of every step included, are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is the algorithmic GB/s of the whole step; `roofline` is the
decode-attention entry point alone against the 8 TB/s HBM peak; `cpu_baseline` is the CPU
oracle (restatement of the reference's llvm decode kernel) on this host.  A chunked-prefill
figure (configs[2]) is reported under `prefill`.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16

HQ, HKV, D, PS = 32, 8, 128, 16
TOKEN_BYTES = 2 * HKV * D * 2  # K and V rows of every kv head, fp16


# --------------------------------------------------------------------------------------------
# workload builders (also imported by tests/)
# --------------------------------------------------------------------------------------------
def decode_workload(batch=64, ctx_lo=1024, ctx_hi=8192, pool_pages=65536, steps=16, seed=1):
    """Page tables of `steps` consecutive decode steps.  Step s sees contexts ctx + s + 1 (the
    appended token included, as the cache builds them when it appends before attention)."""
    rng = np.random.default_rng(seed)
    ctx = rng.integers(ctx_lo, ctx_hi, size=batch, endpoint=True)
    perm = rng.permutation(pool_pages).astype(np.int32)
    max_pages = [(int(c) + steps + PS - 1) // PS for c in ctx]
    starts = np.concatenate([[0], np.cumsum(max_pages)])
    assert starts[-1] <= pool_pages, "pool too small for the batch"
    owned = [perm[starts[i]:starts[i + 1]] for i in range(batch)]
    tables = []
    for s in range(steps):
        kv_len = ctx + s + 1
        npages = (kv_len + PS - 1) // PS
        indptr = np.concatenate([[0], np.cumsum(npages)]).astype(np.int32)
        values = np.concatenate([owned[i][:npages[i]] for i in range(batch)]).astype(np.int32)
        last = ((kv_len - 1) % PS + 1).astype(np.int32)
        pos = (kv_len - 1).astype(np.int32)
        slots = np.array([owned[i][(kv_len[i] - 1) // PS] * PS + (kv_len[i] - 1) % PS for i in range(batch)], np.int32)
        tables.append(dict(kv_len=kv_len.astype(np.int64), page_indptr=indptr, page_values=values,
                           last_page_len=last, q_rope_position=pos, append_position_map=slots))
    return dict(ctx=ctx, owned=owned, tables=tables, pool_pages=pool_pages, batch=batch)


def prefill_workload(batch=8, prefix_hi=4096, chunk_lo=128, chunk_hi=2048, seed=2):
    rng = np.random.default_rng(seed)
    prefix = rng.integers(0, prefix_hi, size=batch, endpoint=True)
    chunk = rng.integers(chunk_lo, chunk_hi, size=batch, endpoint=True)
    npages = (prefix + PS - 1) // PS              # pages the attention reads (the cached prefix)
    npages_after = (prefix + chunk + PS - 1) // PS  # pages owned once the chunk is appended
    pool_pages = int(npages_after.sum()) + 8
    perm = rng.permutation(pool_pages).astype(np.int32)
    starts = np.concatenate([[0], np.cumsum(npages_after)])
    owned = [perm[starts[i]:starts[i + 1]] for i in range(batch)]
    page_values = np.concatenate([owned[i][:npages[i]] for i in range(batch)])
    append_map = np.concatenate([[owned[i][t // PS] * PS + t % PS for t in range(prefix[i], prefix[i] + chunk[i])]
                                 for i in range(batch)]).astype(np.int32)
    flops = 4.0 * HQ * D * float(np.sum(chunk * (chunk + 1) / 2 + chunk * prefix))
    return dict(prefix=prefix, chunk=chunk, pool_pages=pool_pages,
                q_indptr=np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32),
                page_indptr=np.concatenate([[0], np.cumsum(npages)]).astype(np.int32),
                page_values=page_values.astype(np.int32), append_position_map=append_map,
                last_page_len=np.where(prefix == 0, 0, (prefix - 1) % PS + 1).astype(np.int32), flops=flops)


def make_prefill_step(torch, K, pw, gen, dev):
    """The chunked-prefill step that this file times, on the workload `pw` of prefill_workload():
    returns (step, tensors).  step(_) runs RoPE of k and the append of the new K/V rows (one launch) and
    causal attention over the cached prefix and the new chunk in one pass, with the queries read from
    the fused qkv tensor and rotated inside the kernel (one launch) -- what the cache object runs for
    such a step; `tensors` holds every device array it reads and writes (the full-size parity test
    checks `out` / `lse`)."""
    def i32(a):
        return torch.tensor(np.asarray(a), dtype=torch.int32, device=dev)

    n = int(pw["q_indptr"][-1])
    t = dict(
        pages=torch.randn((pw["pool_pages"], 2, HKV, PS, D), generator=gen, device=dev).to(torch.float16),
        qkv=torch.randn((n, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16),
        q=torch.empty((n, HQ, D), dtype=torch.float16, device=dev),
        k=torch.empty((n, HKV, D), dtype=torch.float16, device=dev),
        v=torch.empty((n, HKV, D), dtype=torch.float16, device=dev),
        out=torch.empty((n, HQ, D), dtype=torch.float16, device=dev),
        lse=torch.empty((n, HQ), dtype=torch.float32, device=dev),
        q_indptr=i32(pw["q_indptr"]), page_indptr=i32(pw["page_indptr"]), page_values=i32(pw["page_values"]),
        last_page_len=i32(pw["last_page_len"]),
        q_rope_position=i32(np.concatenate([p + np.arange(c) for p, c in zip(pw["prefix"], pw["chunk"])])),
        append_position_map=i32(pw["append_position_map"]))
    sm_scale = D ** -0.5

    def prefill_step(_):
        K.fused_rope_append(t["qkv"], t["q_rope_position"], None, t["k"], t["v"], 1, t["pages"],
                            t["append_position_map"], 1.0, 1e4)
        K.batch_prefill_cached_and_new_kv_fused_q(t["qkv"], t["q_rope_position"], 1, 1.0, 1e4, t["q_indptr"], t["k"],
                                                  t["v"], t["pages"], t["page_indptr"], t["page_values"],
                                                  t["last_page_len"], t["out"], t["lse"], sm_scale)

    return prefill_step, t


# --------------------------------------------------------------------------------------------
# Seconds of untimed, back-to-back calls in front of every timed region.  The shader clock of this chip
# is managed by the power the running kernel draws and takes tens of milliseconds of continuous load to
# settle: ten 0.5 ms launches after an idle gap measure the ramp, not the kernel (the chunked-prefill
# step reads 0.57 ms that way and 0.46 ms from the 100th call on).
SETTLE_S = 0.3


def settle(torch, fn, seconds=SETTLE_S):
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(16):
            fn(i)
            i += 1
        torch.cuda.synchronize()


def time_region(torch, fn, iters, settle_s=0.0):
    """Milliseconds per call of fn, by HIP events on the stream the kernels run on; with settle_s > 0
    after that many seconds of the same calls, untimed."""
    if settle_s > 0:
        settle(torch, lambda i: fn(i % iters), settle_s)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def calibrate(num_bytes=2 << 30, iters=10, quiet=False):
    """Plain streaming read and copy of `num_bytes`, and a loop of nothing but fp16 MFMA: what the
    memory system and the matrix cores of this box deliver to the simplest possible kernels.
    Prints one JSON line unless `quiet`."""
    import torch

    from tvm_amd import bench_aids as K  # libtvmkv_bench.so: the measurement aids, not the product library

    dev = "cuda:0"
    src = torch.empty(num_bytes // 2, dtype=torch.float16, device=dev).normal_()
    dst = torch.empty_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    K.stream_read(src, sink)
    K.stream_copy(src, dst)
    ms_read = time_region(torch, lambda i: K.stream_read(src, sink), iters)
    K.stream_read_nt(src, sink)
    ms_read_nt = time_region(torch, lambda i: K.stream_read_nt(src, sink), iters)
    ms_copy = time_region(torch, lambda i: K.stream_copy(src, dst), iters)
    # matrix cores: a loop of nothing but fp16 MFMA, one round of workgroups per wave slot
    wgs, mfma_iters = 256 * 2, 4096
    sums = torch.empty((wgs, 256), dtype=torch.float32, device=dev)
    mfma = {}
    for name, ops in (("constant", torch.full((256, 16), 0.5, dtype=torch.float16, device=dev)),
                      ("random", torch.randn((256, 16), device=dev).to(torch.float16))):
        K.mfma_loop(ops, sums, 16)
        ms = time_region(torch, lambda i: K.mfma_loop(ops, sums, mfma_iters), 10, SETTLE_S)
        mfma[name] = round(2.0 * 32 * 32 * 16 * 8 * mfma_iters * 4 * wgs / ms / 1e9, 1)
    out = {"calibration": "plain streaming kernels and an MFMA-only loop", "bytes": num_bytes,
           "mfma_f16_TFLOPs_constant_operands": mfma["constant"], "mfma_f16_TFLOPs_random_operands": mfma["random"],
           "read_GBps": round(num_bytes / ms_read / 1e6, 1), "read_ms": round(ms_read, 4),
           "read_nt_GBps": round(num_bytes / ms_read_nt / 1e6, 1), "read_nt_ms": round(ms_read_nt, 4),
           "copy_GBps_read_plus_write": round(2 * num_bytes / ms_copy / 1e6, 1), "copy_ms": round(ms_copy, 4)}
    if not quiet:
        print(json.dumps(out))
    return out


def bare_step_over_layer_pools(torch, dev, layers, seed):
    """The decode step of configs[1] as bare launches (tvmkv_fused_decode_step), one page pool per layer
    as a model has them: what the memory system makes of `layers` x 1.2 GB that are read once per step
    (nothing of a layer's pages is left in the memory-side cache or the TLBs when its turn comes again),
    without the cache object around the launches.  Returns ms per layer."""
    from tvm_amd import kernels as K

    wl = decode_workload(pool_pages=20480, steps=1, seed=seed)
    B = wl["batch"]
    t = {key: torch.tensor(wl["tables"][0][key], dtype=torch.int32, device=dev)
         for key in ("page_indptr", "page_values", "last_page_len", "q_rope_position", "append_position_map")}
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    first = torch.empty((wl["pool_pages"], 2, HKV, PS, D), dtype=torch.float16, device=dev)
    for lo in range(0, wl["pool_pages"], 4096):
        first[lo:lo + 4096].copy_(torch.randn(first[lo:lo + 4096].shape, generator=gen, device=dev))
    pools = [first] + [first.clone() for _ in range(layers - 1)]
    qkv = torch.randn((B, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    out = torch.empty((B, HQ, D), dtype=torch.float16, device=dev)
    lse = torch.empty((B, HQ), dtype=torch.float32, device=dev)

    def step(_):
        for pool in pools:
            K.fused_decode_step(qkv, pool, t["page_indptr"], t["page_values"], t["last_page_len"], t["q_rope_position"],
                                t["append_position_map"], out, lse, 1, 1.0, 1e4, D ** -0.5)

    settle(torch, step)
    return time_region(torch, step, 8) / layers


def cache_object_decode(torch, dev, layers=32, seed=1):
    """configs[1] through the cache OBJECT, the way a model drives it (the reference's call order,
    src/runtime/vm/kv_state.cc:33-116): per decode step one begin_forward for all layers, then
    attention_with_fused_qkv layer by layer, then end_forward.  The cache is filled through the same
    interface (chunked prefill steps).  What this leg shows beside the kernel legs: the host
    bookkeeping, the single auxiliary upload per step and the launches of `layers` layers do not
    slow the kernels down."""
    from tvm_amd import get_global_func as gf

    rng = np.random.default_rng(seed)
    B = 64
    ctx = rng.integers(1024, 8192, size=B, endpoint=True)
    steps = 12
    capacity = int(ctx.sum()) + B * (steps + 4) + B * PS
    cache = gf("vm.builtin.paged_attention_kv_cache_create")(
        [B, capacity, 4096, PS, 0], [0, layers], HQ, HKV, D, D, [0] * layers, False, 1, 1.0, 1e4, None,
        torch.empty((), dtype=torch.float16, device=dev))
    cache.set_stream(torch.cuda.current_stream().cuda_stream)
    f_add = gf("vm.builtin.kv_state_add_sequence")
    f_begin = gf("vm.builtin.kv_state_begin_forward")
    f_end = gf("vm.builtin.kv_state_end_forward")
    f_attn = gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")
    sm_scale = D ** -0.5
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    chunk_qkv = torch.randn((4096, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    chunk_out = torch.empty((4096, HQ, D), dtype=torch.float16, device=dev)
    for b in range(B):
        f_add(cache, b)
        left = int(ctx[b])
        while left > 0:
            n = min(left, 4096)
            f_begin(cache, [b], [n], None)
            for layer in range(layers):
                f_attn(cache, layer, sm_scale, chunk_qkv[:n], chunk_out[:n])
            f_end(cache)
            left -= n
    qkv = torch.randn((B, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    out = torch.empty((B, HQ, D), dtype=torch.float16, device=dev)
    ids, ones = list(range(B)), [1] * B

    def step():
        f_begin(cache, ids, ones, None)
        for layer in range(layers):
            f_attn(cache, layer, sm_scale, qkv, out)
        f_end(cache)

    for _ in range(4):
        step()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps - 4):
        step()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / (steps - 4)
    gpu_ms = start.elapsed_time(stop) / (steps - 4)
    t0 = time.perf_counter()  # the host's share: how long it takes to enqueue a step on an idle device
    step()
    enqueue_ms = (time.perf_counter() - t0) * 1e3
    torch.cuda.synchronize()
    kv_tokens = float(ctx.sum()) + B * (4 + (steps - 4) / 2.0)  # cached tokens an average timed step attends to
    step_bytes = layers * (kv_tokens * TOKEN_BYTES + B * HQ * D * 2 * 2 + B * (HQ + 2 * HKV) * D * 2 + B * TOKEN_BYTES)
    del cache
    torch.cuda.empty_cache()
    bare_ms = bare_step_over_layer_pools(torch, dev, layers, seed)
    return {"ms_per_layer_bare_launches_over_one_pool_per_layer": round(bare_ms, 4),
            "workload": f"configs[1] through the cache object: {layers} layers, B=64, ctx U[1024,8192], one begin_forward + "
                        f"{layers} x attention_with_fused_qkv + end_forward per decode step, cache filled by chunked prefill "
                        "steps through the same interface",
            "layers": layers, "ms_per_step": round(gpu_ms, 4), "ms_per_layer": round(gpu_ms / layers, 4),
            "host_wall_ms_per_step": round(wall_ms, 4), "host_enqueue_ms_per_step": round(enqueue_ms, 4),
            "GBps": round(step_bytes / gpu_ms / 1e6, 1),
            "frac_of_hbm_peak": round(step_bytes / gpu_ms / 1e6 / HBM_PEAK_GBPS, 4),
            "tokens_per_s": round(B / (gpu_ms * 1e-3), 1)}


def cache_object_shared_prefix_decode(torch, dev, layers=8, seed=5):
    """Decode with a shared prompt through the cache object: 64 sequences forked from one parent that holds a
    4096-token prefix (kv_state_fork_sequence: the children share the parent's pages, src/runtime/vm/
    paged_kv_cache.cc:653-770), each with U[256,2048] tokens of its own.  A decode step then has two depths
    (BeginForward, :884-1212): the shared prefix once for all 64 queries (the paged prefill kernel, 64 x group rows
    per kv head), every sequence's own tokens (the decode kernel), and the merge of the two states -- the
    reference's flow for prefix sharing (:2161-2335).  Algorithmic bytes count the prefix once."""
    from tvm_amd import get_global_func as gf

    rng = np.random.default_rng(seed)
    B, prefix = 64, 4096
    own = rng.integers(256, 2048, size=B, endpoint=True)
    steps = 8
    capacity = prefix + int(own.sum()) + B * (steps + 8) + (B + 2) * PS
    cache = gf("vm.builtin.paged_attention_kv_cache_create")(
        [B + 1, capacity, 4096, PS, 0], [0, layers], HQ, HKV, D, D, [0] * layers, False, 1, 1.0, 1e4, None,
        torch.empty((), dtype=torch.float16, device=dev))
    cache.set_stream(torch.cuda.current_stream().cuda_stream)
    f_add, f_fork = gf("vm.builtin.kv_state_add_sequence"), gf("vm.builtin.kv_state_fork_sequence")
    f_begin, f_end = gf("vm.builtin.kv_state_begin_forward"), gf("vm.builtin.kv_state_end_forward")
    f_popn = gf("vm.builtin.kv_state_popn")
    f_attn = gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")
    sm_scale = D ** -0.5
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    chunk_qkv = torch.randn((4096, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    chunk_out = torch.empty((4096, HQ, D), dtype=torch.float16, device=dev)

    def forward(ids, lens, qkv_, out_):
        f_begin(cache, ids, lens, None)
        for layer in range(layers):
            f_attn(cache, layer, sm_scale, qkv_, out_)
        f_end(cache)

    parent = B
    f_add(cache, parent)
    forward([parent], [prefix], chunk_qkv[:prefix], chunk_out[:prefix])
    for b in range(B):
        f_fork(cache, parent, b)
        n = int(own[b])
        forward([b], [n], chunk_qkv[:n], chunk_out[:n])
    qkv = torch.randn((B, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    out = torch.empty((B, HQ, D), dtype=torch.float16, device=dev)
    ids, ones = list(range(B)), [1] * B

    def step(_):
        forward(ids, ones, qkv, out)
        for b in ids:
            f_popn(cache, b, 1)

    for _ in range(3):
        step(0)
    flags = cache.flags()
    ms = time_region(torch, step, steps, SETTLE_S)
    nbytes = layers * ((prefix + float(own.sum()) + B) * TOKEN_BYTES + B * HQ * D * 2 * 2 + B * (HQ + 2 * HKV) * D * 2)
    unshared = layers * ((B * prefix + float(own.sum()) + B) * TOKEN_BYTES + B * HQ * D * 2 * 2)
    return {"workload": f"64 sequences forked from one 4096-token prompt, U[256,2048] tokens of their own, one token each per "
                        f"step, {layers} layers through the cache object: per layer split + RoPE + append, the shared prefix "
                        "for all queries in one paged-prefill launch, the sequences' own tokens in the decode kernel, merge",
            "layers": layers, "depths": flags["num_depths"], "ms_per_step": round(ms, 4), "ms_per_layer": round(ms / layers, 4),
            "MB_per_layer": round(nbytes / layers / 1e6, 1), "GBps": round(nbytes / ms / 1e6, 1),
            "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
            "MB_per_layer_without_sharing": round(unshared / layers / 1e6, 1)}


def cache_object_prefill(torch, dev, layers=8):
    """configs[2] through the cache object: the prefixes are cached by chunked-prefill steps, then every
    timed step appends the 8 chunks in one begin_forward, runs attention_with_fused_qkv on every layer
    and pops the chunks again (popn), so that all timed steps see the same cache."""
    from tvm_amd import get_global_func as gf

    pw = prefill_workload()
    prefix, chunk = [int(x) for x in pw["prefix"]], [int(x) for x in pw["chunk"]]
    B = len(prefix)
    total = sum(chunk)
    capacity = sum(prefix) + total + 2 * B * PS
    chunk_cap = (total + 255) // 256 * 256
    cache = gf("vm.builtin.paged_attention_kv_cache_create")(
        [B, capacity, chunk_cap, PS, 0], [0, layers], HQ, HKV, D, D, [0] * layers, False, 1, 1.0, 1e4, None,
        torch.empty((), dtype=torch.float16, device=dev))
    cache.set_stream(torch.cuda.current_stream().cuda_stream)
    f_add = gf("vm.builtin.kv_state_add_sequence")
    f_begin = gf("vm.builtin.kv_state_begin_forward")
    f_end = gf("vm.builtin.kv_state_end_forward")
    f_popn = gf("vm.builtin.kv_state_popn")
    f_attn = gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")
    sm_scale = D ** -0.5
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    qkv = torch.randn((chunk_cap, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    out = torch.empty((chunk_cap, HQ, D), dtype=torch.float16, device=dev)
    for b in range(B):
        f_add(cache, b)
        if prefix[b] > 0:
            f_begin(cache, [b], [prefix[b]], None)
            for layer in range(layers):
                f_attn(cache, layer, sm_scale, qkv[:prefix[b]], out[:prefix[b]])
            f_end(cache)
    ids = list(range(B))

    def step(_):
        f_begin(cache, ids, chunk, None)
        for layer in range(layers):
            f_attn(cache, layer, sm_scale, qkv[:total], out[:total])
        f_end(cache)
        for b in range(B):
            f_popn(cache, b, chunk[b])

    for _ in range(2):
        step(0)
    ms = time_region(torch, step, 10, SETTLE_S)
    tflops = layers * pw["flops"] / (ms * 1e-3) / 1e12
    return {"workload": f"configs[2] through the cache object: {layers} layers; per step one begin_forward that appends the 8 "
                        f"chunks, {layers} x attention_with_fused_qkv, end_forward, and popn of the chunks",
            "layers": layers, "ms_per_step": round(ms, 4), "ms_per_layer": round(ms / layers, 4),
            "tflops": round(tflops, 1), "frac_of_mfma_peak": round(tflops / MFMA_F16_PEAK_TFLOPS, 4)}


# HBM bytes per launch of the decode entry point, from rocprofv3 counter runs of this file.  The one
# place the figures live is the rocprofv3 summary profiles/decode_mfma_kernel_cfg2_batched_decode.txt,
# which carries them on a line `traffic_record: {...}` (FETCH_SIZE and WRITE_SIZE in KiB per dispatch of
# decode_mfma_kernel, which merges the chunks itself, the scale of each counter from the plain copy
# kernel of known size, profiles/stream_copy_kernel_2GiB_calibration.txt, and the algorithmic bytes of
# the launch they were measured on).  They are kept as bytes of traffic per algorithmic byte: the kernel
# reads every K/V row once whatever the context lengths are, and the rest (q, outputs, split-KV partial
# states) scales with the same page tables, so the ratio carries over to the page tables of any
# --steps / --warmup of this workload.  Without the file the traffic is reported as null.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "decode_mfma_kernel_cfg2_batched_decode.txt")


def traffic_per_algorithmic_byte():
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith("traffic_record:"):
                    r = json.loads(line[len("traffic_record:"):])
                    kib = r["fetch_size_kib"] * r["fetch_scale"] + r["write_size_kib"] * r["write_scale"]
                    return kib * 1024.0 / r["algorithmic_bytes"]
    except (OSError, ValueError, KeyError):
        pass
    return None


def measured_traffic(algorithmic_bytes):
    ratio = traffic_per_algorithmic_byte()
    return None if ratio is None else int(round(ratio * algorithmic_bytes))


def prefill_cpu_baseline(torch, pw, t, budget_s=10.0):
    """The chunked-prefill step of configs[2] on the CPU oracle (split + RoPE, ragged causal attention of
    the chunk, attention over the cached prefix, merge: the reference's llvm kernels restated, one
    thread), on a bounded sample: kv head 0 with its 4 query heads (1/8 of the heads) of the sequences
    with the least work first, until `budget_s` seconds are spent; its outputs are compared with the
    rows the GPU step wrote."""
    from oracle import kernels as ok

    group = HQ // HKV
    flops_seq = 4.0 * group * D * (pw["chunk"] * (pw["chunk"] + 1) / 2 + pw["chunk"] * pw["prefix"])
    qkv, pos_all, out_gpu = t["qkv"], t["q_rope_position"].cpu().numpy(), t["out"]
    spent, flops, seqs, err = 0.0, 0.0, [], 0.0
    for b in np.argsort(flops_seq):
        c, pre = int(pw["chunk"][b]), int(pw["prefix"][b])
        r0, r1 = int(pw["q_indptr"][b]), int(pw["q_indptr"][b + 1])
        heads = list(range(group)) + [HQ, HQ + HKV]
        sub = qkv[r0:r1][:, heads].cpu().numpy()
        ids = pw["page_values"][int(pw["page_indptr"][b]):int(pw["page_indptr"][b + 1])]
        pool = t["pages"][torch.tensor(ids, dtype=torch.int64, device=qkv.device)][:, :, 0:1].contiguous().cpu().numpy()
        if len(ids) == 0:
            pool = np.zeros((1, 2, 1, PS, D), np.float16)
        q = np.zeros((c, group, D), np.float16)
        k = np.zeros((c, 1, D), np.float16)
        v = np.zeros((c, 1, D), np.float16)
        eo, el = np.zeros((c, group, D), np.float16), np.zeros((c, group), np.float32)
        to, tl = np.zeros((c, group, D), np.float16), np.zeros((c, group), np.float32)
        ind = np.array([0, c], np.int32)
        zq, zb = np.zeros(c, np.int32), np.zeros(1, np.int32)
        c0 = time.perf_counter()
        ok.fused_rope(sub, pos_all[r0:r1], q, k, v, 1)
        ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, D ** -0.5)
        ok.prefill_paged(q, ind, pool, np.array([0, len(ids)], np.int32), np.arange(len(ids), dtype=np.int32),
                         pw["last_page_len"][b:b + 1], zb, zq, to, tl, 0, 0, 1.0, 1e4, D ** -0.5)
        ok.merge_state_inplace(eo, el, to, tl)
        spent += time.perf_counter() - c0
        flops += float(flops_seq[b])
        seqs.append(int(b))
        err = max(err, float(np.max(np.abs(out_gpu[r0:r1, :group].cpu().numpy().astype(np.float32) - eo.astype(np.float32)))))
        if spent > budget_s:
            break
    return {"value": round(flops / spent / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"kv head 0 with its {group} query heads (1/{HKV} of the heads) of sequences {seqs} of the same "
                      f"workload, least work first ({flops / 1e9:.1f} of {pw['flops'] / 1e9:.1f} GFLOP), split+RoPE, ragged "
                      f"causal + paged + merge as the reference composes the step, 1 thread, {spent:.1f} s",
            "gpu_vs_cpu_max_abs_err": err}


def cfg1_decode(torch, dev, steps=16):
    """configs[0] (the reference's CPU-runnable case): 4 sequences with contexts 512/1024/1500/2048 built
    through the cache verbs in a 1024-page pool (pages in allocation order), then decode steps that
    append one token per sequence.  Checked against the committed golden fixture (page table and append
    indices bit for bit, output within atol = rtol = 1e-2), timed on the GPU, and the same decode step
    (split + RoPE + decode attention) timed on the CPU oracle, one thread."""
    from oracle import kernels as ok
    from tests.golden import make_fixtures as mf
    from tests.gpu_util import GpuCache
    from tvm_amd import get_global_func as gf

    c = mf.CFG1
    gold = np.load(os.path.join(ROOT, "tests", "golden", "cfg1_decode.npz"))
    cache = GpuCache(mf.cfg1_cache_config(), 1, c["hq"], c["hkv"], c["d"], c["d"], rope_mode=1)
    seen = {}

    def grab():
        for name in mf.PER_DEPTH:
            seen[name] = cache.cache.aux(name, 0)
        for name in mf.GLOBAL:
            seen[name] = cache.cache.aux(name)

    _, out = mf.cfg1_drive(cache, grab)
    tables_equal = all(seen[name] == list(gold[name]) for name in mf.PER_DEPTH + mf.GLOBAL)
    tol = 1e-2 + 1e-2 * np.abs(gold["out"].astype(np.float32))
    err = np.abs(out.astype(np.float32) - gold["out"].astype(np.float32))
    B, heads = len(c["ctx"]), c["hq"] + 2 * c["hkv"]
    ids, ones = list(range(B)), [1] * B
    sm = c["d"] ** -0.5
    qkv = torch.randn((B, heads, c["d"]), device=dev).to(torch.float16)
    o = torch.empty((B, c["hq"], c["d"]), dtype=torch.float16, device=dev)
    cache.cache.set_stream(torch.cuda.current_stream().cuda_stream)
    f_begin, f_end = gf("vm.builtin.kv_state_begin_forward"), gf("vm.builtin.kv_state_end_forward")
    f_attn = gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")

    def step(_):
        f_begin(cache.cache, ids, ones, None)
        f_attn(cache.cache, 0, sm, qkv, o)
        f_end(cache.cache)

    for _ in range(3):
        step(0)
    ms = time_region(torch, step, steps)
    # CPU: the same kind of step on the fixture's page table (contexts + 1), K/V values do not matter for time
    rng = np.random.default_rng(0)
    ip = np.asarray(gold["page_indptr"], np.int32)
    pv = np.asarray(gold["page_indices"], np.int32)
    pages = rng.standard_normal((c["pool_pages"], 2, c["hkv"], c["page"], c["d"])).astype(np.float16)
    qh = np.zeros((B, c["hq"], c["d"]), np.float16)
    kh = np.zeros((B, c["hkv"], c["d"]), np.float16)
    vh = np.zeros((B, c["hkv"], c["d"]), np.float16)
    eo, el = np.zeros((B, c["hq"], c["d"]), np.float16), np.zeros((B, c["hq"]), np.float32)
    z = np.zeros(B, np.int32)
    c0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        ok.fused_rope(gold["qkv"], gold["q_rope_position_map"], qh, kh, vh, 1)
        ok.decode(qh, pages, ip, pv, np.asarray(gold["last_page_len"], np.int32), z, z, eo, el, 0, 1.0, 1e4, sm)
    cpu_s = (time.perf_counter() - c0) / reps
    kv_tokens = sum(c["ctx"]) + B
    return {"workload": "configs[0]: 4 seqs, ctx 512/1024/1500/2048, Hq32/Hkv8/D128, page 16, 1024-page pool, pages in "
                        "allocation order through add_sequence / begin_forward; decode steps through the cache object",
            "parity": {"page_table_and_append_indices_bit_exact_vs_fixture": bool(tables_equal),
                       "output_within_atol_rtol_1e-2_of_fixture": bool(np.all(err <= tol)),
                       "max_abs_err": float(err.max())},
            "ms_per_step": round(ms, 4), "tokens_per_s": round(B / (ms * 1e-3), 1),
            "note": "20.8 MB of K/V per step sit in the 256 MB memory-side cache: a parity configuration, not a bandwidth claim",
            "cpu_baseline": {"value": round(B / cpu_s, 2), "unit": "tokens/s", "cores": 1, "kind": "port",
                             "GBps": round(kv_tokens * TOKEN_BYTES / cpu_s / 1e9, 3),
                             "sample": f"{reps} decode steps of this configuration (split+RoPE and decode attention over "
                                       f"{kv_tokens} cached tokens), 1 thread, {cpu_s * reps:.2f} s"}}


def mla_cpu_baseline(heads_sample=4, budget_s=8.0):
    """The oracle's restatement of the reference's absorbed-MLA paged kernel (a GPU-only TIR kernel: the
    reference has no CPU kernel for MLA, python/tvm/relax/frontend/nn/llm/kv_cache.py:676-677) on a
    sample of configs[4]'s decode batch: `heads_sample` of the 128 heads of the first sequences, until
    `budget_s` seconds are spent."""
    from oracle import kernels as ok

    rng = np.random.default_rng(4)
    ctx = rng.integers(2048, 8192, size=32, endpoint=True)
    dl, dr, ps = 512, 64, 64
    spent, flops, nbytes, done = 0.0, 0.0, 0.0, 0
    for b in range(len(ctx)):
        n = int(ctx[b])
        npg = (n + ps - 1) // ps
        pages = (rng.standard_normal((npg, ps, dl + dr)) * 0.5).astype(np.float16)
        q = (rng.standard_normal((1, heads_sample, dl + dr)) * 0.5).astype(np.float16)
        eo, el = np.zeros((1, heads_sample, dl), np.float16), np.zeros((1, heads_sample), np.float32)
        c0 = time.perf_counter()
        ok.prefill_paged_mla(q, np.array([0, 1], np.int32), pages, np.array([0, npg], np.int32),
                             np.arange(npg, dtype=np.int32), np.array([(n - 1) % ps + 1], np.int32), eo, el, 0,
                             (128 + 64) ** -0.5, d_latent=dl)
        spent += time.perf_counter() - c0
        flops += 2.0 * heads_sample * (2 * dl + dr) * n
        nbytes += n * (dl + dr) * 2.0
        done += 1
        if spent > budget_s:
            break
    return {"value": round(flops / spent / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "note": "no reference CPU kernel exists for MLA; this is the oracle's CPU restatement of the reference's GPU-only TIR kernel",
            "sample": f"{heads_sample} of 128 heads of the first {done} sequences of configs[4]'s decode batch, one query "
                      f"token each, 1 thread, {spent:.1f} s",
            "tokens_per_s_scaled_to_128_heads": round(done / spent * heads_sample / 128.0, 4)}


def extras(torch, K, dev):
    """configs[3] and configs[4] of BASELINE.json, and the sliding-window and token-tree variants of the
    attention kernels on configs[1]'s shape; kernels only (inputs resident, HIP events)."""
    out = {}

    def i32(a):
        return torch.tensor(np.asarray(a), dtype=torch.int32, device=dev)

    # ---- configs[3]: long-context split-KV decode, 64 q heads / 8 kv heads, 8 sequences ---------
    rng = np.random.default_rng(3)
    hq, hkv, d, ps = 64, 8, 128, 16
    ctx = rng.integers(32768, 131072, size=8, endpoint=True)
    npages = (ctx + ps - 1) // ps
    pool = int(npages.sum()) + 64
    perm = rng.permutation(pool).astype(np.int32)
    pages = torch.empty((pool, 2, hkv, ps, d), dtype=torch.float16, device=dev)
    for lo in range(0, pool, 8192):
        pages[lo:lo + 8192].normal_()
    indptr = np.concatenate([[0], np.cumsum(npages)])
    q = torch.randn((8, hq, d), device=dev).to(torch.float16)
    o = torch.empty_like(q)
    lse = torch.empty((8, hq), dtype=torch.float32, device=dev)
    z = torch.zeros(8, dtype=torch.int32, device=dev)
    args = (q, pages, i32(indptr), i32(perm[:indptr[-1]]), i32((ctx - 1) % ps + 1), z, z, o, lse, 0, 1.0, 1e4,
            d ** -0.5)
    K.batch_decode_paged_kv(*args)
    ms = time_region(torch, lambda i: K.batch_decode_paged_kv(*args), 20, SETTLE_S)
    nbytes = float(ctx.sum()) * 2 * hkv * d * 2 + 2 * 8 * hq * d * 2
    # the same call with the chunk merge as a second kernel: the difference is what merging inside
    # the kernel saves
    import tvm_amd
    tvm_amd.set_option("decode_separate_merge", 1)
    K.batch_decode_paged_kv(*args)
    ms_two_kernels = time_region(torch, lambda i: K.batch_decode_paged_kv(*args), 20, SETTLE_S)
    tvm_amd.set_option("decode_separate_merge", 0)
    out["long_context_decode"] = {"workload": "configs[3]: 8 seqs, ctx U[32768,131072] seed 3, Hq64/Hkv8/D128, page 16",
                                  "kv_tokens": int(ctx.sum()), "algorithmic_bytes": int(nbytes), "ms": round(ms, 4),
                                  "ms_with_separate_merge_kernel": round(ms_two_kernels, 4),
                                  "GBps": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    del pages
    torch.cuda.empty_cache()

    # ---- decode away from configs[1]: one long sequence, few long ones, many short ones, one kv head ----
    def decode_shape(batch, lo, hi, hq_, hkv_, seed):
        rng_ = np.random.default_rng(seed)
        ctx_ = rng_.integers(lo, hi, size=batch, endpoint=True)
        npg_ = (ctx_ + 15) // 16
        ip_ = np.concatenate([[0], np.cumsum(npg_)])
        pool_ = int(ip_[-1]) + 64
        perm_ = rng_.permutation(pool_).astype(np.int32)
        pages_ = torch.empty((pool_, 2, hkv_, 16, 128), dtype=torch.float16, device=dev)
        for lo_ in range(0, pool_, 8192):
            pages_[lo_:lo_ + 8192].normal_()
        q_ = torch.randn((batch, hq_, 128), device=dev).to(torch.float16)
        o_ = torch.empty_like(q_)
        l_ = torch.empty((batch, hq_), dtype=torch.float32, device=dev)
        z_ = torch.zeros(batch, dtype=torch.int32, device=dev)
        a_ = (q_, pages_, i32(ip_), i32(perm_[:ip_[-1]]), i32((ctx_ - 1) % 16 + 1), z_, z_, o_, l_, 0, 1.0, 1e4, 128 ** -0.5)
        K.batch_decode_paged_kv(*a_)
        ms_ = time_region(torch, lambda i: K.batch_decode_paged_kv(*a_), 20, SETTLE_S)
        nb_ = float(ctx_.sum()) * 2 * hkv_ * 128 * 2 + 2 * batch * hq_ * 128 * 2
        return {"ms": round(ms_, 4), "MB": round(nb_ / 1e6, 1), "frac_of_hbm_peak": round(nb_ / ms_ / 1e6 / HBM_PEAK_GBPS, 4)}

    out["decode_other_shapes"] = {
        "workload": "batch x context, query / kv heads, D128, page 16, permuted pool: the split-KV chunk rule, the chunk merge "
                    "and the search for a work item's sequence away from configs[1]",
        "1 x 131072, 32/8": decode_shape(1, 131072, 131072, 32, 8, 11),
        "4 x 32768, 32/8": decode_shape(4, 32768, 32768, 32, 8, 12),
        "2048 x U[64,512], 32/8": decode_shape(2048, 64, 512, 32, 8, 13),
        "64 x U[1024,8192], 32/1": decode_shape(64, 1024, 8192, 32, 1, 14),
        "64 x U[1024,8192], 64/1": decode_shape(64, 1024, 8192, 64, 1, 15),
        "64 x U[1024,8192], 64/2": decode_shape(64, 1024, 8192, 64, 2, 16),
        "16 x U[100,4000], 32/8": decode_shape(16, 100, 4000, 32, 8, 5),
        "8 x U[2000,6000], 32/8": decode_shape(8, 2000, 6000, 32, 8, 17)}
    torch.cuda.empty_cache()

    # ---- sliding window + attention sinks, and a token-tree verify step, on configs[1]'s shape ----
    hq, hkv, d, ps, nseq = 32, 8, 128, 16, 64
    rng = np.random.default_rng(7)
    sink, window = 4, 4096
    offset = rng.integers(sink, sink + ps, size=nseq)           # physical slot of the first window token
    phys = offset + window                                       # slots in use: sinks, a gap, the window
    npages = (phys + ps - 1) // ps
    pool = 65536
    perm = rng.permutation(pool).astype(np.int32)
    pages = torch.empty((pool, 2, hkv, ps, d), dtype=torch.float16, device=dev)
    for lo in range(0, pool, 8192):
        pages[lo:lo + 8192].normal_()
    indptr = np.concatenate([[0], np.cumsum(npages)])
    q = torch.randn((nseq, hq, d), device=dev).to(torch.float16)
    o = torch.empty_like(q)
    lse = torch.empty((nseq, hq), dtype=torch.float32, device=dev)
    z = torch.zeros(nseq, dtype=torch.int32, device=dev)
    info = i32(np.stack([(phys - 1) % ps + 1, offset, np.full(nseq, sink)]))
    args = (q, pages, i32(indptr), i32(perm[:indptr[-1]]), info, z, z, o, lse, 0, 1.0, 1e4, d ** -0.5)
    K.batch_decode_paged_kv(*args)
    ms = time_region(torch, lambda i: K.batch_decode_paged_kv(*args), 20, SETTLE_S)
    nbytes = float(nseq * (sink + window)) * 2 * hkv * d * 2 + 2 * nseq * hq * d * 2
    out["sliding_window_decode"] = {"workload": "64 seqs, 4 sink tokens + a 4096-token window each (length_info with 3 rows), "
                                                "Hq32/Hkv8/D128, page 16",
                                    "ms": round(ms, 4), "GBps": round(nbytes / ms / 1e6, 1),
                                    "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}

    # ---- paged prefill through the sliding-window form of the kernel (three-row length_info, per-layer
    # window) against the plain form on the same keys: configs[2]'s sequences, every key visible --------
    rng2 = np.random.default_rng(2)
    pre = rng2.integers(0, 4096, size=8, endpoint=True)
    chunk = rng2.integers(128, 2048, size=8, endpoint=True)
    kvp = pre + chunk
    npg = (kvp + ps - 1) // ps
    ipp = np.concatenate([[0], np.cumsum(npg)])
    qip = np.concatenate([[0], np.cumsum(chunk)])
    nq = int(qip[-1])
    qp = torch.randn((nq, hq, d), device=dev).to(torch.float16)
    op = torch.empty_like(qp)
    lp = torch.empty((nq, hq), dtype=torch.float32, device=dev)
    z8, zq = torch.zeros(8, dtype=torch.int32, device=dev), torch.zeros(nq, dtype=torch.int32, device=dev)
    last = (kvp - 1) % ps + 1
    plain = (qp, i32(qip), pages, i32(ipp), i32(perm[:ipp[-1]]), i32(last), z8, zq, op, lp, 0, 0, 1.0, 1e4, d ** -0.5)
    three = i32(np.stack([last, np.zeros(8, dtype=np.int64), np.zeros(8, dtype=np.int64)]))
    slid = (qp, i32(qip), pages, i32(ipp), i32(perm[:ipp[-1]]), three, z8, zq, op, lp, 1, 0, 1.0, 1e4, d ** -0.5)
    K.batch_prefill_paged_kv(*plain)
    ms_plain = time_region(torch, lambda i: K.batch_prefill_paged_kv(*plain), 20, SETTLE_S)
    K.batch_prefill_paged_kv(*slid, sliding_window_size=1 << 20)
    ms_slid = time_region(torch, lambda i: K.batch_prefill_paged_kv(*slid, sliding_window_size=1 << 20), 20, SETTLE_S)
    flops = 4.0 * hq * d * float(np.sum(chunk * kvp))
    out["sliding_window_prefill"] = {"workload": "configs[2]'s 8 sequences (prefix U[0,4096] + chunk U[128,2048], seed 2), the chunk's "
                                                 "queries against all cached keys: plain kernel, and the sliding-window form "
                                                 "(length_info with 3 rows, per-layer window mask) with a window that covers them",
                                     "ms_plain": round(ms_plain, 4), "ms_sliding_form": round(ms_slid, 4),
                                     "sliding_over_plain": round(ms_slid / ms_plain, 3),
                                     "tflops_sliding_form": round(flops / ms_slid / 1e9, 1),
                                     "frac_of_mfma_peak": round(flops / ms_slid / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}

    # ---- uniform long prefill work: no short sequences, no causal diagonal, no ragged tail ----------
    uq, uk = 2048, 4096
    unp = uk // ps
    uip = np.arange(9) * unp
    uqi = np.arange(9) * uq
    uqt = torch.randn((8 * uq, hq, d), device=dev).to(torch.float16)
    uo = torch.empty_like(uqt)
    ul = torch.empty((8 * uq, hq), dtype=torch.float32, device=dev)
    uzq = torch.zeros(8 * uq, dtype=torch.int32, device=dev)
    uargs = (uqt, i32(uqi), pages, i32(uip), i32(perm[:uip[-1]]), i32(np.full(8, ps)), z8, uzq, uo, ul, 0, 0, 1.0, 1e4,
             d ** -0.5)
    K.batch_prefill_paged_kv(*uargs)
    settle(torch, lambda i: K.batch_prefill_paged_kv(*uargs))
    ms_u = time_region(torch, lambda i: K.batch_prefill_paged_kv(*uargs), 20)
    uflops = 4.0 * hq * d * 8 * uq * uk
    out["prefill_uniform"] = {"workload": f"8 seqs x {uq} query tokens against {uk} cached tokens each, every key visible "
                                          "(paged prefill kernel, Hq32/Hkv8/D128, page 16, permuted pool): the attention "
                                          "kernel without configs[2]'s short sequences, diagonal and tail",
                              "ms": round(ms_u, 4), "tflops": round(uflops / ms_u / 1e9, 1),
                              "frac_of_mfma_peak": round(uflops / ms_u / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
    del uqt, uo, ul

    def preorder(depth):  # (first, second) labels of a complete binary tree listed in depth-first order
        labels = []

        def walk(level):
            me = len(labels)
            labels.append([me, 0])
            if level + 1 < depth:
                walk(level + 1)
                walk(level + 1)
            labels[me][1] = len(labels)
        walk(0)
        return np.asarray(labels, dtype=np.int32)

    ctx = rng.integers(1024, 8192, size=nseq, endpoint=True)    # cached tokens before the tree

    def tree_verify(depth):
        labels = preorder(depth)                                  # 2^depth - 1 draft tokens per sequence
        nodes = len(labels)
        kv = ctx + nodes                                          # the tree's tokens are appended already
        npages = (kv + ps - 1) // ps
        indptr = np.concatenate([[0], np.cumsum(npages)])
        qi = np.arange(nseq + 1) * nodes
        q = torch.randn((nseq * nodes, hq, d), device=dev).to(torch.float16)
        o = torch.empty_like(q)
        lse = torch.empty((nseq * nodes, hq), dtype=torch.float32, device=dev)
        zq = torch.zeros(nseq * nodes, dtype=torch.int32, device=dev)
        args = (q, i32(qi), pages, i32(indptr), i32(perm[:indptr[-1]]), i32((kv - 1) % ps + 1), z, zq, o, lse, 0, 1.0,
                1e4, d ** -0.5, i32(qi), i32(np.tile(labels, (nseq, 1)).reshape(-1)))
        K.tree_attn_paged_kv(*args)
        settle(torch, lambda i: K.tree_attn_paged_kv(*args))
        ms = time_region(torch, lambda i: K.tree_attn_paged_kv(*args), 20)
        depth_sum = float(sum((lv + 1) * 2 ** lv for lv in range(depth)))  # visible tree tokens summed over the nodes
        flops = 4.0 * hq * d * (float(ctx.sum()) * nodes + nseq * depth_sum)
        nbytes = float(kv.sum()) * 2 * hkv * d * 2 + 2 * nseq * nodes * hq * d * 2
        return {"workload": f"64 seqs, ctx U[1024,8192], a {nodes}-node binary draft tree each (appended), one launch of the "
                            f"tree-masked paged kernel, Hq32/Hkv8/D128: {nodes * hq // hkv} query rows per kv head",
                "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                "GBps": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}

    out["token_tree_verify"] = tree_verify(6)            # 63 nodes: 252 rows per kv head, two row tiles, compute-bound
    out["token_tree_verify_15_nodes"] = tree_verify(4)   # 60 rows per kv head: one row tile, the K/V stream decides

    # ---- a short chunk against a long cached sequence: few row tiles, split over the keys ----------
    plen, clen = 100000, 64
    npg = (plen + ps - 1) // ps
    qs = torch.randn((clen, hq, d), device=dev).to(torch.float16)
    ks_ = torch.randn((clen, hkv, d), device=dev).to(torch.float16)
    vs_ = torch.randn((clen, hkv, d), device=dev).to(torch.float16)
    os_ = torch.empty_like(qs)
    ls_ = torch.empty((clen, hq), dtype=torch.float32, device=dev)
    sargs = (qs, i32([0, clen]), ks_, vs_, pages, i32([0, npg]), i32(perm[:npg]), i32([(plen - 1) % ps + 1]), os_, ls_,
             d ** -0.5)
    ms_split = time_region(torch, lambda i: K.batch_prefill_cached_and_new_kv(*sargs), 20, SETTLE_S)
    prev = tvm_amd.set_option("prefill_kv_splits", 1)
    try:
        ms_whole = time_region(torch, lambda i: K.batch_prefill_cached_and_new_kv(*sargs), 20, SETTLE_S)
    finally:
        tvm_amd.set_option("prefill_kv_splits", prev)
    nbytes = float(plen) * 2 * hkv * d * 2
    out["short_chunk_long_context"] = {
        "workload": f"one sequence, a {clen}-token chunk on {plen} cached tokens, Hq32/Hkv8/D128, one-pass chunked prefill: "
                    "2 row tiles per kv head, their keys split over the workgroups of the launch and merged",
        "ms": round(ms_split, 4), "ms_one_workgroup_per_row_tile": round(ms_whole, 4),
        "speedup": round(ms_whole / ms_split, 2), "GBps": round(nbytes / ms_split / 1e6, 1),
        "frac_of_hbm_peak": round(nbytes / ms_split / 1e6 / HBM_PEAK_GBPS, 4)}
    del pages
    torch.cuda.empty_cache()

    # ---- the other head dims: decode on configs[1]'s lengths, the one-pass chunked prefill on configs[2]'s ----
    def head_dim_leg(d_, hq_, hkv_):
        rng_ = np.random.default_rng(1)
        ctx_ = rng_.integers(1024, 8192, size=64, endpoint=True)
        npg_ = (ctx_ + ps - 1) // ps
        ip_ = np.concatenate([[0], np.cumsum(npg_)])
        pw_ = prefill_workload()
        pool_ = max(int(ip_[-1]), pw_["pool_pages"]) + 8
        perm_ = rng_.permutation(pool_).astype(np.int32)
        pages_ = torch.empty((pool_, 2, hkv_, ps, d_), dtype=torch.float16, device=dev)
        for lo_ in range(0, pool_, 8192):
            pages_[lo_:lo_ + 8192].normal_()
        q_ = torch.randn((64, hq_, d_), device=dev).to(torch.float16)
        o_ = torch.empty_like(q_)
        l_ = torch.empty((64, hq_), dtype=torch.float32, device=dev)
        z_ = torch.zeros(64, dtype=torch.int32, device=dev)
        a_ = (q_, pages_, i32(ip_), i32(perm_[:ip_[-1]]), i32((ctx_ - 1) % ps + 1), z_, z_, o_, l_, 0, 1.0, 1e4, d_ ** -0.5)
        K.batch_decode_paged_kv(*a_)
        ms_d = time_region(torch, lambda i: K.batch_decode_paged_kv(*a_), 20, SETTLE_S)
        nb_ = float(ctx_.sum()) * 2 * hkv_ * d_ * 2 + 2 * 64 * hq_ * d_ * 2
        n_ = int(pw_["q_indptr"][-1])
        qp_ = torch.randn((n_, hq_, d_), device=dev).to(torch.float16)
        kp_ = torch.randn((n_, hkv_, d_), device=dev).to(torch.float16)
        vp_ = torch.randn((n_, hkv_, d_), device=dev).to(torch.float16)
        op_ = torch.empty_like(qp_)
        lp_ = torch.empty((n_, hq_), dtype=torch.float32, device=dev)
        b_ = (qp_, i32(pw_["q_indptr"]), kp_, vp_, pages_, i32(pw_["page_indptr"]), i32(pw_["page_values"]),
              i32(pw_["last_page_len"]), op_, lp_, d_ ** -0.5)
        K.batch_prefill_cached_and_new_kv(*b_)
        ms_p = time_region(torch, lambda i: K.batch_prefill_cached_and_new_kv(*b_), 20, SETTLE_S)
        fl_ = pw_["flops"] / (HQ * D) * (hq_ * d_)
        return {"decode_ms": round(ms_d, 4), "decode_frac_of_hbm_peak": round(nb_ / ms_d / 1e6 / HBM_PEAK_GBPS, 4),
                "prefill_ms": round(ms_p, 4), "prefill_tflops": round(fl_ / ms_p / 1e9, 1),
                "prefill_frac_of_mfma_peak": round(fl_ / ms_p / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}

    # ---- the generic kernels: float32 storage, pages that are not a power of two ---------------------------
    def generic_leg():
        from tvm_amd import dlpack as dl
        rng_ = np.random.default_rng(1)
        ctx_ = rng_.integers(1024, 8192, size=64, endpoint=True)
        res = {"workload": "what the tuned fp16 kernels are not built for, on the generic matrix-core kernels (K/V rows "
                           "straight from their pages into the operands of v_mfma_f32_16x16x4_f32, or of the fp16 "
                           "instructions of that shape for fp16 storage): decode of 64 seqs ctx U[1024,8192] Hq32/Hkv8/D128 "
                           "with float32 storage (page 16) and with fp16 pages of 24 tokens; causal self-attention of "
                           "4 x 2048 tokens with float32 storage (D128) and with fp16 storage at head dims 160 and 96 (the latter with RoPE inside the kernel)"}
        for name, tdt, ps_ in (("decode_float32_storage", torch.float32, 16), ("decode_fp16_pages_of_24_tokens", torch.float16, 24)):
            npg_ = (ctx_ + ps_ - 1) // ps_
            ip_ = np.concatenate([[0], np.cumsum(npg_)])
            pool_ = int(ip_[-1]) + 8
            perm_ = rng_.permutation(pool_).astype(np.int32)
            pages_ = torch.empty((pool_, 2, HKV, ps_, D), dtype=tdt, device=dev)
            for lo_ in range(0, pool_, 4096):
                pages_[lo_:lo_ + 4096].normal_()
            q_ = torch.randn((64, HQ, D), device=dev).to(tdt)
            o_ = torch.empty_like(q_)
            l_ = torch.empty((64, HQ), dtype=torch.float32, device=dev)
            z_ = torch.zeros(64, dtype=torch.int32, device=dev)
            ints = [i32(ip_), i32(perm_[:ip_[-1]]), i32((ctx_ - 1) % ps_ + 1)]
            a_ = (dl.tensor(q_), dl.tensor(pages_), dl.tensor(ints[0]), dl.tensor(ints[1]), dl.tensor(ints[2]), dl.tensor(z_),
                  dl.tensor(z_), dl.tensor(o_), dl.tensor(l_), 0, 1.0, 1e4, D ** -0.5)
            dl.call("batch_decode_paged_kv", *a_)
            ms_ = time_region(torch, lambda i: dl.call("batch_decode_paged_kv", *a_), 20, SETTLE_S)
            nb_ = float(ctx_.sum()) * 2 * HKV * D * q_.element_size() + 2 * 64 * HQ * D * q_.element_size()
            res[name] = {"ms": round(ms_, 4), "GBps": round(nb_ / ms_ / 1e6, 1),
                         "frac_of_hbm_peak": round(nb_ / ms_ / 1e6 / HBM_PEAK_GBPS, 4)}
            del pages_
        n_, c_ = 4, 2048
        q_, k_, v_ = (torch.randn((n_ * c_, h_, D), device=dev) for h_ in (HQ, HKV, HKV))
        o_ = torch.empty_like(q_)
        l_ = torch.empty((n_ * c_, HQ), dtype=torch.float32, device=dev)
        ind_ = i32(np.arange(n_ + 1) * c_)
        zq_, zb_ = torch.zeros(n_ * c_, dtype=torch.int32, device=dev), torch.zeros(n_, dtype=torch.int32, device=dev)
        a_ = (dl.tensor(q_), dl.tensor(ind_), dl.tensor(k_), dl.tensor(v_), dl.tensor(ind_), dl.tensor(zq_), dl.tensor(zb_),
              dl.tensor(o_), dl.tensor(l_), 1, 0, 1.0, 1e4, D ** -0.5)
        dl.call("batch_prefill_ragged_kv", *a_)
        ms_ = time_region(torch, lambda i: dl.call("batch_prefill_ragged_kv", *a_), 5, SETTLE_S)
        fl_ = 4.0 * HQ * D * n_ * c_ * (c_ + 1) / 2
        res["causal_prefill_float32_storage"] = {"ms": round(ms_, 4), "tflops": round(fl_ / ms_ / 1e9, 1),
                                                 "frac_of_fp32_mfma_peak": round(fl_ / ms_ / 1e9 / 157.3, 4)}
        for d_, rotary_ in ((160, 0), (96, 1)):  # head dim 96 with RoPE inside the kernel: a sliding-window cache's prefill
            q_, k_, v_ = (torch.randn((n_ * c_, h_, d_), device=dev).to(torch.float16) for h_ in (HQ, HKV, HKV))
            o_ = torch.empty_like(q_)
            pos_ = i32(np.tile(np.arange(c_), n_))
            a_ = (dl.tensor(q_), dl.tensor(ind_), dl.tensor(k_), dl.tensor(v_), dl.tensor(ind_), dl.tensor(pos_), dl.tensor(zb_),
                  dl.tensor(o_), dl.tensor(l_), 1, rotary_, 1.0, 1e4, d_ ** -0.5)
            dl.call("batch_prefill_ragged_kv", *a_)
            ms_ = time_region(torch, lambda i: dl.call("batch_prefill_ragged_kv", *a_), 5, SETTLE_S)
            fl_ = 4.0 * HQ * d_ * n_ * c_ * (c_ + 1) / 2
            name_ = f"causal_prefill_fp16_head_dim_{d_}" + ("_rope_in_kernel" if rotary_ else "")
            res[name_] = {"ms": round(ms_, 4), "tflops": round(fl_ / ms_ / 1e9, 1),
                          "frac_of_mfma_peak": round(fl_ / ms_ / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)}
        return res

    out["generic_kernels"] = generic_leg()
    torch.cuda.empty_cache()

    out["other_head_dims"] = {
        "workload": "decode of 64 seqs ctx U[1024,8192] (configs[1]'s lengths) and the one-pass chunked-prefill kernel on "
                    "configs[2]'s 8 sequences, page 16, at the head dims beside 128 (query / kv heads)",
        "D64, 32/8": head_dim_leg(64, 32, 8),
        "D256, 16/8": head_dim_leg(256, 16, 8)}
    torch.cuda.empty_cache()

    # ---- configs[4]: MLA, 128 heads, latent 512 + rope 64, page 64 ------------------------------
    hq, dl, dr, ps = 128, 512, 64, 64
    sm = (128 + 64) ** -0.5

    def mla_case(name, prefix, chunk, seed, causal):
        rng = np.random.default_rng(seed)
        kv = prefix + chunk
        npg = (kv + ps - 1) // ps
        pool = int(npg.sum()) + 8
        perm = rng.permutation(pool).astype(np.int32)
        pg = (torch.randn((pool, ps, dl + dr), device=dev) * 0.5).to(torch.float16)
        ip = np.concatenate([[0], np.cumsum(npg)])
        qi = np.concatenate([[0], np.cumsum(chunk)])
        n = int(qi[-1])
        q = (torch.randn((n, hq, dl + dr), device=dev) * 0.5).to(torch.float16)
        o = torch.empty((n, hq, dl), dtype=torch.float16, device=dev)
        lse = torch.empty((n, hq), dtype=torch.float32, device=dev)
        a = (q, i32(qi), pg, i32(ip), i32(perm[:ip[-1]]), i32((kv - 1) % ps + 1), o, lse, causal, sm)
        K.batch_prefill_paged_kv_mla(*a)
        ms = time_region(torch, lambda i: K.batch_prefill_paged_kv_mla(*a), 20, SETTLE_S)
        if causal:
            pairs = float(np.sum(chunk * prefix + chunk * (chunk + 1) / 2))
        else:
            pairs = float(np.sum(chunk * kv))
        flops = 2.0 * hq * (2 * dl + dr) * pairs  # QK^T over 576 features + PV over 512
        nbytes = float(kv.sum()) * (dl + dr) * 2 + n * hq * (2 * dl + dr) * 2
        out[name] = {"ms": round(ms, 4), "algorithmic_flops": flops, "algorithmic_bytes": int(nbytes),
                     "tflops": round(flops / ms / 1e9, 1),
                     "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                     "GBps": round(nbytes / ms / 1e6, 1),
                     "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}

    def mla_prefill_step(name, prefix_len, chunk_len, nseq, seed):
        """A chunked-prefill step of an MLA layer as the reference composes it
        (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_mla_tir.py:293-349):
        causal self-attention of the chunk on expanded heads (d_qk 192, d_v 128, ragged kernel),
        attention of the absorbed query over the cached latent prefix (paged MLA kernel, all
        visible), and the merge of the two states in the 128-wide value space (the projection of
        the latent output that sits between them in a model is not part of the path)."""
        rng = np.random.default_rng(seed)
        n = nseq * chunk_len
        qi = i32(np.arange(nseq + 1) * chunk_len)
        qe = (torch.randn((n, hq, 192), device=dev) * 0.5).to(torch.float16)
        ke = (torch.randn((n, hq, 192), device=dev) * 0.5).to(torch.float16)
        ve = (torch.randn((n, hq, 128), device=dev) * 0.5).to(torch.float16)
        o_self = torch.empty((n, hq, 128), dtype=torch.float16, device=dev)
        l_self = torch.empty((n, hq), dtype=torch.float32, device=dev)
        zq, zb = torch.zeros(n, dtype=torch.int32, device=dev), torch.zeros(nseq, dtype=torch.int32, device=dev)
        npg = (prefix_len + ps - 1) // ps
        pool = nseq * npg + 8
        perm = rng.permutation(pool).astype(np.int32)
        pg = (torch.randn((pool, ps, dl + dr), device=dev) * 0.5).to(torch.float16)
        ip = i32(np.arange(nseq + 1) * npg)
        qa = (torch.randn((n, hq, dl + dr), device=dev) * 0.5).to(torch.float16)
        o_lat = torch.empty((n, hq, dl), dtype=torch.float16, device=dev)
        l_lat = torch.empty((n, hq), dtype=torch.float32, device=dev)
        o_cross = torch.empty((n, hq, 128), dtype=torch.float16, device=dev).normal_()
        pv_ = i32(perm[:nseq * npg])
        last = i32(np.full(nseq, (prefix_len - 1) % ps + 1))

        def step(_):
            K.batch_prefill_ragged_kv(qe, qi, ke, ve, qi, zq, zb, o_self, l_self, 1, 0, 1.0, 1e4, sm)
            K.batch_prefill_paged_kv_mla(qa, qi, pg, ip, pv_, last, o_lat, l_lat, 0, sm)
            K.merge_state_inplace(o_self, l_self, o_cross, l_lat)

        step(0)
        ms = time_region(torch, step, 20, SETTLE_S)
        flops = float(hq) * nseq * (640.0 * chunk_len * (chunk_len + 1) / 2 + 2176.0 * chunk_len * prefix_len)
        out[name] = {"ms": round(ms, 4), "algorithmic_flops": flops, "tflops": round(flops / ms / 1e9, 1),
                     "frac_of_mfma_peak": round(flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                     "workload": f"configs[4] prefill step: {nseq} seqs, {chunk_len}-token chunk on a {prefix_len}-token "
                                 "prefix: ragged causal (192/128) + absorbed paged (576->512) + merge, three launches"}

    rng = np.random.default_rng(4)
    ctx = rng.integers(2048, 8192, size=32, endpoint=True)
    mla_prefill_step("mla_prefill_step", 2048, 1024, 4, 8)
    mla_case("mla_decode", ctx - 1, np.ones(32, dtype=np.int64), 5, 0)
    out["mla_decode"]["workload"] = "configs[4] decode: batch 32, ctx U[2048,8192] seed 4, 128 heads, 576-wide latent rows, page 64"
    mla_case("mla_prefill", np.full(4, 2048), np.full(4, 1024), 6, 1)
    out["mla_prefill"]["workload"] = "configs[4] prefill: 4 seqs, 1024-token chunk on a 2048-token prefix (chunk already appended), causal"
    mla_case("mla_verify_4_tokens", ctx - 4, np.full(32, 4, dtype=np.int64), 7, 1)
    out["mla_verify_4_tokens"]["workload"] = ("configs[4]'s decode batch with 4 tokens per sequence (a draft to verify), causal: every token is "
                                              "planned as a one-token sequence and the KV is split as in a decode step")
    ctx200 = np.random.default_rng(8).integers(2048, 8192, size=200, endpoint=True)
    mla_case("mla_decode_200_sequences", ctx200 - 1, np.ones(200, dtype=np.int64), 9, 0)
    out["mla_decode_200_sequences"]["workload"] = ("200 sequences, ctx U[2048,8192], one token each: more than one split launch plans, "
                                                   "cut into two split launches of 100")
    return out


def hold(which, seconds):
    """Runs one kernel back to back for `seconds` and prints its rate over the last second."""
    import torch

    from tvm_amd import kernels as K

    dev = "cuda:0"
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    if which == "prefill":
        pw = prefill_workload()
        fn, _ = make_prefill_step(torch, K, pw, gen, dev)
        unit, work = "TFLOP/s", pw["flops"] / 1e12
    elif which == "mfma":
        ops = torch.randn((256, 16), device=dev).to(torch.float16)
        sums = torch.empty((512, 256), dtype=torch.float32, device=dev)
        from tvm_amd import bench_aids
        fn = lambda i: bench_aids.mfma_loop(ops, sums, 4096)
        unit, work = "TFLOP/s (random operands)", 2.0 * 32 * 32 * 16 * 8 * 4096 * 4 * 512 / 1e12
    elif which in ("mla_prefill", "mla_decode"):
        hq, dl, dr, ps = 128, 512, 64, 64
        rng = np.random.default_rng(4)
        if which == "mla_decode":
            prefix, chunk, causal = rng.integers(2048, 8192, size=32, endpoint=True) - 1, np.ones(32, dtype=np.int64), 0
        else:
            prefix, chunk, causal = np.full(4, 2048), np.full(4, 1024), 1
        kv = prefix + chunk
        npg = (kv + ps - 1) // ps
        pool = int(npg.sum()) + 8
        perm = rng.permutation(pool).astype(np.int32)
        pg = (torch.randn((pool, ps, dl + dr), device=dev) * 0.5).to(torch.float16)
        ip = np.concatenate([[0], np.cumsum(npg)])
        qi = np.concatenate([[0], np.cumsum(chunk)])
        n = int(qi[-1])
        i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=dev)
        q = (torch.randn((n, hq, dl + dr), device=dev) * 0.5).to(torch.float16)
        o = torch.empty((n, hq, dl), dtype=torch.float16, device=dev)
        lse = torch.empty((n, hq), dtype=torch.float32, device=dev)
        a = (q, i32(qi), pg, i32(ip), i32(perm[:ip[-1]]), i32((kv - 1) % ps + 1), o, lse, causal, (128 + 64) ** -0.5)
        fn = lambda i: K.batch_prefill_paged_kv_mla(*a)
        pairs = float(np.sum(chunk * prefix + chunk * (chunk + 1) / 2)) if causal else float(np.sum(chunk * kv))
        unit, work = "TFLOP/s", 2.0 * hq * (2 * dl + dr) * pairs / 1e12
    else:
        wl = decode_workload(steps=1)
        t = wl["tables"][0]
        B = wl["batch"]
        pages = torch.randn((wl["pool_pages"], 2, HKV, PS, D), generator=gen, device=dev, dtype=torch.float16)
        q = torch.randn((B, HQ, D), generator=gen, device=dev, dtype=torch.float16)
        out = torch.empty_like(q)
        lse = torch.empty((B, HQ), dtype=torch.float32, device=dev)
        z = torch.zeros(B, dtype=torch.int32, device=dev)
        tabs = {k: torch.tensor(t[k], dtype=torch.int32, device=dev) for k in ("page_indptr", "page_values", "last_page_len")}
        fn = lambda i: K.batch_decode_paged_kv(q, pages, tabs["page_indptr"], tabs["page_values"], tabs["last_page_len"],
                                               z, z, out, lse, 0, 1.0, 1e4, D ** -0.5)
        unit, work = "TB/s", (float(t["kv_len"].sum()) * TOKEN_BYTES + B * HQ * D * 4) / 1e12
    settle(torch, fn, max(seconds - 1.0, 0.5))
    ms = time_region(torch, fn, 200)
    print(json.dumps({"held": which, "seconds": seconds, "ms": round(ms, 4), "rate": round(work / (ms * 1e-3), 2), "unit": unit}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=16)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-CPU leg (profiling runs)")
    ap.add_argument("--no-prefill", action="store_true", help="skip the chunked-prefill leg (profiling runs)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip configs[3] (long-context decode), configs[4] (MLA decode / prefill) and the "
                         "sliding-window / token-tree variants, which are otherwise reported under \"extras\" "
                         "(not part of the headline value)")
    ap.add_argument("--extras", action="store_true", help="accepted for compatibility: the extras run by default")
    ap.add_argument("--calibrate", action="store_true",
                    help="only run the plain 2 GiB streaming read and copy kernels (bandwidth calibration; "
                         "known-size dispatches for scaling rocprofv3 traffic counters)")
    ap.add_argument("--hold", choices=["prefill", "mfma", "decode", "mla_prefill", "mla_decode"],
                    help="only run one kernel back to back for --hold-seconds and print its rate: a steady load to "
                         "read the board's power and clocks under from another shell (rocm-smi)")
    ap.add_argument("--hold-seconds", type=float, default=6.0)
    args = ap.parse_args()
    if args.calibrate:
        calibrate()
        return
    if args.hold:
        hold(args.hold, args.hold_seconds)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; the path shards per kv head without any exchange "
                 "step, and no multi-GPU figure is produced. Use --gpus 1.")

    import torch

    from tvm_amd import kernels as K  # raises if libtvmkv.so is missing: there is no fallback
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    K_steps, W = args.steps, args.warmup
    total_steps = K_steps + W

    # ---- decode workload, resident in HBM ---------------------------------------------------
    wl = decode_workload(steps=total_steps)
    B = wl["batch"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    pages = torch.empty((wl["pool_pages"], 2, HKV, PS, D), dtype=torch.float16, device=dev)
    for lo in range(0, wl["pool_pages"], 8192):  # fill in slices: randn makes an fp32 temporary
        pages[lo:lo + 8192].copy_(torch.randn(pages[lo:lo + 8192].shape, generator=gen, device=dev))
    qkv = torch.randn((total_steps, B, HQ + 2 * HKV, D), generator=gen, device=dev).to(torch.float16)
    q = torch.empty((B, HQ, D), dtype=torch.float16, device=dev)
    k = torch.empty((B, HKV, D), dtype=torch.float16, device=dev)
    v = torch.empty((B, HKV, D), dtype=torch.float16, device=dev)
    out = torch.empty((B, HQ, D), dtype=torch.float16, device=dev)
    lse = torch.empty((B, HQ), dtype=torch.float32, device=dev)
    zeros_b = torch.zeros(B, dtype=torch.int32, device=dev)

    def i32(a):
        return torch.tensor(a, dtype=torch.int32, device=dev)

    tabs = [{key: i32(t[key]) for key in ("page_indptr", "page_values", "last_page_len", "q_rope_position",
                                          "append_position_map")} for t in wl["tables"]]
    sm_scale = D ** -0.5

    def rope_append(s):  # split + RoPE and the append of the new k / v rows, one launch
        t = tabs[s]
        K.fused_rope_append(qkv[s], t["q_rope_position"], q, k, v, 1, pages, t["append_position_map"], 1.0, 1e4)

    def decode_only(s):
        t = tabs[s]
        K.batch_decode_paged_kv(q, pages, t["page_indptr"], t["page_values"], t["last_page_len"], zeros_b,
                                t["q_rope_position"], out, lse, 0, 1.0, 1e4, sm_scale)

    def step(s):  # the decode step of a layer as the cache object runs it: one launch
        t = tabs[s]
        K.fused_decode_step(qkv[s], pages, t["page_indptr"], t["page_values"], t["last_page_len"], t["q_rope_position"],
                            t["append_position_map"], out, lse, 1, 1.0, 1e4, sm_scale)

    def step_two_launches(s):
        rope_append(s)
        decode_only(s)

    settle(torch, lambda i: step(i % total_steps))  # clocks settle under the workload itself, then W + K steps
    for s in range(W):
        step(s)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms_step = time_region(torch, lambda i: step(W + i), K_steps)
    wall_ms = (time.perf_counter() - t0) * 1e3 / K_steps
    # (0.1 s of the same calls first: the first launches of a kernel load its code and wake a second queue slot)
    ms_two = time_region(torch, lambda i: step_two_launches(W + i), K_steps, 0.1)
    # the decode entry point alone (split-KV kernel with the fused chunk merge), same page tables
    ms_decode = time_region(torch, lambda i: decode_only(W + i), K_steps)
    # for the comparison with the CPU: the last step's output of the one-launch step, and of the two launches
    step(total_steps - 1)
    out_fused = out.clone()
    step_two_launches(total_steps - 1)
    torch.cuda.synchronize()

    kv_tokens = np.array([t["kv_len"].sum() for t in wl["tables"][W:]], dtype=np.float64)
    qo_bytes = B * HQ * D * 2 * 2
    step_bytes = kv_tokens.mean() * TOKEN_BYTES + qo_bytes + B * (HQ + 2 * HKV) * D * 2 + B * TOKEN_BYTES
    decode_bytes = kv_tokens.mean() * TOKEN_BYTES + qo_bytes
    gbps_step = step_bytes / (ms_step * 1e-3) / 1e9
    gbps_decode = decode_bytes / (ms_decode * 1e-3) / 1e9

    result = {
        "metric": "paged decode attn GB/s",
        "value": round(gbps_step, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K_steps,
        "warmup": W,
        "settle_s": SETTLE_S,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: batched paged decode, 1 layer, B=64, ctx U[1024,8192] seed 1, "
                               "Hq32/Hkv8/D128 fp16, page 16, permuted 65536-page pool, append 1 token/seq/step "
                               "(split + RoPE + append + split-KV decode with the chunk merge in ONE launch, "
                               "tvmkv_fused_decode_step, as the cache object runs a decode step)",
                   "kv_tokens_per_step": int(kv_tokens.mean()), "bytes_per_step": int(step_bytes)},
        "tokens_per_s": round(B / (ms_step * 1e-3), 1),
        "host_wall_ms_per_step": round(wall_ms, 4),
        "ms_per_step_as_two_launches": round(ms_two, 4),
        "roofline": {"bound": "hbm", "achieved": round(gbps_decode, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps_decode / HBM_PEAK_GBPS, 4),
                     "traffic": measured_traffic(int(decode_bytes)),
                     "traffic_per_algorithmic_byte": (None if traffic_per_algorithmic_byte() is None
                                                      else round(traffic_per_algorithmic_byte(), 4)),
                     "kernel": "tvmkv_batch_decode_paged_kv (decode_mfma_kernel, chunk merge fused)",
                     "ms": round(ms_decode, 4), "algorithmic_bytes": int(decode_bytes)},
    }

    # ---- chunked prefill (configs[2]): ragged causal + paged non-causal + merge + append -------
    if not args.no_prefill:
        pw = prefill_workload()
        prefill_step, prefill_tensors = make_prefill_step(torch, K, pw, gen, dev)

        for _ in range(3):
            prefill_step(0)
        ms_cold = time_region(torch, prefill_step, 10)  # ten launches as they come, clocks still ramping
        settle(torch, prefill_step)
        ms_prefill = time_region(torch, prefill_step, max(K_steps, 10))
        tflops = pw["flops"] / (ms_prefill * 1e-3) / 1e12
        result["prefill"] = {"workload": "configs[2]: chunked causal prefill, 8 seqs, prefix U[0,4096], chunk "
                                         "U[128,2048] seed 2 (RoPE of k + append of the new K/V rows in one launch; causal attention over the new chunk and attention over the cached prefix in one pass that rotates q itself)",
                             "tflops": round(tflops, 2), "ms": round(ms_prefill, 4),
                             "algorithmic_flops": pw["flops"],
                             "frac_of_mfma_peak": round(tflops / MFMA_F16_PEAK_TFLOPS, 4),
                             "ms_first_ten_launches": round(ms_cold, 4)}

    # What the simplest kernels reach on this box, next to the datasheet peaks.  After the timed legs:
    # the MFMA loop heats the chip and the clock of what follows drops.
    cal = calibrate(num_bytes=1 << 30, iters=5, quiet=True)
    result["calibration"] = {"hbm_read_GBps": cal["read_GBps"], "hbm_read_nontemporal_GBps": cal["read_nt_GBps"],
                             "mfma_f16_TFLOPs_constant_operands": cal["mfma_f16_TFLOPs_constant_operands"],
                             "mfma_f16_TFLOPs_random_operands": cal["mfma_f16_TFLOPs_random_operands"],
                             "what": "1 GiB streaming read (plain / non-temporal loads); a loop of fp16 MFMA only"}
    result["roofline"]["frac_of_calibrated_read"] = round(gbps_decode / cal["read_nt_GBps"], 4)
    if "prefill" in result:
        result["prefill"]["frac_of_calibrated_mfma_random_operands"] = round(
            result["prefill"]["tflops"] / cal["mfma_f16_TFLOPs_random_operands"], 4)

    # ---- CPU baseline: the oracle's restatement of the reference's llvm decode kernel ---------
    if not args.no_cpu_baseline:
        from oracle import kernels as ok

        # The timed decode steps, last one first, until about 12 s of CPU time are spent.  The pages of
        # the last step hold every earlier step's tokens too (steps only append), so one compact host
        # copy (same bytes, renumbered page ids) serves all of them with each step's own page table.
        last = W + K_steps - 1
        used = wl["tables"][last]["page_values"]
        host_pages = pages[torch.tensor(used, dtype=torch.int64, device=dev)].cpu().numpy()
        renumber = {int(pid): i for i, pid in enumerate(used)}
        qkv_host = qkv[W:].cpu().numpy()
        z = np.zeros(B, np.int32)
        cpu_s, cpu_bytes, steps_done, err = 0.0, 0.0, 0, None
        for s in range(last, W - 1, -1):
            t = wl["tables"][s]
            values = np.array([renumber[int(pid)] for pid in t["page_values"]], np.int32)
            qh = np.zeros((B, HQ, D), np.float16)
            kh = np.zeros((B, HKV, D), np.float16)
            vh = np.zeros((B, HKV, D), np.float16)
            eo = np.zeros((B, HQ, D), np.float16)
            el = np.zeros((B, HQ), np.float32)
            c0 = time.perf_counter()
            ok.fused_rope(qkv_host[s - W], t["q_rope_position"], qh, kh, vh, 1)
            ok.decode(qh, host_pages, t["page_indptr"], values, t["last_page_len"], z, z, eo, el, 0, 1.0, 1e4,
                      sm_scale)
            cpu_s += time.perf_counter() - c0
            cpu_bytes += float(t["kv_len"].sum()) * TOKEN_BYTES + qo_bytes
            steps_done += 1
            if s == last:  # the GPU buffers hold the last step's result
                eo_last = eo
                err = float(np.max(np.abs(out.cpu().numpy().astype(np.float32) - eo.astype(np.float32))))
                err_fused = float(np.max(np.abs(out_fused.cpu().numpy().astype(np.float32) - eo.astype(np.float32))))
            if cpu_s > 12.0:
                break
        result["cpu_baseline"] = {"value": round(cpu_bytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1,
                                  "kind": "port",
                                  "sample": f"{steps_done} full decode steps of the same workload (split+RoPE and "
                                            f"decode attention of 64 sequences, ~{int(cpu_bytes / steps_done / TOKEN_BYTES)} "
                                            f"kv tokens each), 1 thread, {cpu_s:.1f} s; the reference kernel is T.serial",
                                  "tokens_per_s": round(B * steps_done / cpu_s, 2), "host_cpus": os.cpu_count(),
                                  "gpu_vs_cpu_max_abs_err": err_fused,
                                  "gpu_two_launches_vs_cpu_max_abs_err": err}

        # The same kernel on all of the box's host cores: one task per sequence (sequences are
        # independent in the reference kernel), the C calls run outside the interpreter lock.
        from concurrent.futures import ThreadPoolExecutor
        threads = max(1, min(16, len(os.sched_getaffinity(0))))
        par_s, par_bytes, par_steps = 0.0, 0.0, 0
        with ThreadPoolExecutor(threads) as pool:
            for s in range(last, last - steps_done, -1):
                t = wl["tables"][s]
                values = np.array([renumber[int(pid)] for pid in t["page_values"]], np.int32)
                qh = np.zeros((B, HQ, D), np.float16)
                kh = np.zeros((B, HKV, D), np.float16)
                vh = np.zeros((B, HKV, D), np.float16)
                po = np.zeros((B, HQ, D), np.float16)
                pl = np.zeros((B, HQ), np.float32)
                order = np.argsort(-t["kv_len"])  # longest first
                c0 = time.perf_counter()
                ok.fused_rope(qkv_host[s - W], t["q_rope_position"], qh, kh, vh, 1)
                list(pool.map(lambda b: ok.decode_range(qh, host_pages, t["page_indptr"], values, t["last_page_len"], z, z,
                                                        po, pl, int(b), int(b) + 1, sm_scale), order))
                par_s += time.perf_counter() - c0
                par_bytes += float(t["kv_len"].sum()) * TOKEN_BYTES + qo_bytes
                par_steps += 1
                if s == last:
                    assert np.array_equal(po, eo_last), "threaded CPU run differs from the serial one"
        result["cpu_baseline_all_cores"] = {"value": round(par_bytes / par_s / 1e9, 3), "unit": "GB/s", "cores": threads,
                                            "kind": "port",
                                            "sample": f"the same {par_steps} decode steps, one task per sequence on "
                                                      f"{threads} threads, {par_s:.1f} s",
                                            "tokens_per_s": round(B * par_steps / par_s, 2)}
        if "prefill" in result:
            result["prefill"]["cpu_baseline"] = prefill_cpu_baseline(torch, pw, prefill_tensors)
        result["cfg1_decode"] = cfg1_decode(torch, dev)


    if not args.no_extras:
        del pages, qkv
        torch.cuda.empty_cache()
        result["extras"] = extras(torch, K, dev)
        if not args.no_cpu_baseline:
            cpu_mla = mla_cpu_baseline()
            result["extras"]["mla_decode"]["cpu_baseline"] = cpu_mla
            result["extras"]["mla_prefill"]["cpu_baseline"] = dict(cpu_mla, sample=cpu_mla["sample"] + " (the same kernel "
                                                                   "serves prefill-shaped calls: the per-flop rate carries over)")
        torch.cuda.empty_cache()
        result["extras"]["cache_object_decode"] = cache_object_decode(torch, dev)
        torch.cuda.empty_cache()
        result["extras"]["cache_object_prefill"] = cache_object_prefill(torch, dev)
        torch.cuda.empty_cache()
        result["extras"]["cache_object_shared_prefix_decode"] = cache_object_shared_prefix_decode(torch, dev)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
