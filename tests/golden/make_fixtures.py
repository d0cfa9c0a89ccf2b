#!/usr/bin/env python3
"""Writes the golden fixtures of this folder.

    python tests/golden/make_fixtures.py

The fixtures are produced by the repository's own CPU oracle (oracle/), which is pinned to closed
forms, invariants and hand-derived examples in tests/test_oracle_kernels.py and
tests/test_host_cache_oracle.py; nothing of the reference implementation is imported or run.  They
therefore guard against regressions of the oracle, of the C++ host cache and of the HIP kernels,
on inputs that are fixed once and for all:

  rope_vectors.npz      split + rotary embedding at positions 0, 1, 2047, 131071
                        (position_embedding.py:525-565 of the reference)
  cfg1_decode.npz       4 sequences with contexts 512/1024/1500/2048 built through the cache verbs,
                        then one decode step: its page table, append indices and attention output
  host_scenarios.json   the verb sequences of the reference's KV-cache tests
                        (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:706-909)
                        with every auxiliary array after each begin_forward and the final pool state
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import host_cache as hc  # noqa: E402
from oracle import kernels as ok  # noqa: E402
from oracle.paged_kv_cache import OraclePagedKVCache  # noqa: E402
from tests import scenario as S  # noqa: E402

PER_DEPTH = ["qo_indptr", "page_indptr", "page_indices", "last_page_len", "sliding_window_offset", "sink_size",
             "k_rope_pos_offset"]
GLOBAL = ["q_rope_position_map", "append_position_map", "cur_append_lengths_indptr", "k_ragged_rope_pos_offset"]

CFG1 = dict(ctx=[512, 1024, 1500, 2048], hq=32, hkv=8, d=128, page=16, pool_pages=1024, seed=0)


def rope_inputs():
    rng = np.random.default_rng(11)
    qkv = rng.standard_normal((4, 2 + 2 * 1, 128)).astype(np.float16)
    pos = np.array([0, 1, 2047, 131071], np.int32)
    return qkv, pos


def make_rope():
    qkv, pos = rope_inputs()
    q = np.zeros((4, 2, 128), np.float16)
    k = np.zeros((4, 1, 128), np.float16)
    v = np.zeros((4, 1, 128), np.float16)
    ok.fused_rope(qkv, pos, q, k, v, 1, theta=1e4, scale=1.0)
    np.savez_compressed(os.path.join(HERE, "rope_vectors.npz"), qkv=qkv, pos=pos, q=q, k=k, v=v)


def cfg1_drive(cache, on_decode_begin=None):
    """Prefills the four contexts (one sequence per begin_forward, chunks of 512) and runs one
    decode step.  Returns (qkv of the decode step, output of the decode step).  `cache` has the
    method names of OraclePagedKVCache."""
    c = CFG1
    rng = np.random.default_rng(c["seed"])
    heads = c["hq"] + 2 * c["hkv"]
    sm = c["d"] ** -0.5
    for sid, ctx in enumerate(c["ctx"]):
        cache.add_sequence(sid)
        done = 0
        while done < ctx:
            n = min(512, ctx - done)
            qkv = rng.standard_normal((n, heads, c["d"])).astype(np.float16)
            out = np.zeros((n, c["hq"], c["d"]), np.float16)
            cache.begin_forward([sid], [n])
            cache.attention_with_fused_qkv(0, sm, qkv, out)
            cache.end_forward()
            done += n
    ids = list(range(len(c["ctx"])))
    qkv = rng.standard_normal((len(ids), heads, c["d"])).astype(np.float16)
    out = np.zeros((len(ids), c["hq"], c["d"]), np.float16)
    cache.begin_forward(ids, [1] * len(ids))
    if on_decode_begin is not None:
        on_decode_begin()
    cache.attention_with_fused_qkv(0, sm, qkv, out)
    cache.end_forward()
    return qkv, out


def cfg1_cache_config():
    c = CFG1
    return [len(c["ctx"]), c["pool_pages"] * c["page"] - c["page"], 512, c["page"], 0]


def make_cfg1():
    c = CFG1
    cache = OraclePagedKVCache(cfg1_cache_config(), 1, c["hq"], c["hkv"], c["d"], c["d"], rope_mode=1)
    aux = {}

    def grab():
        a = cache.host.aux
        for name in PER_DEPTH:
            aux[name] = np.array(a[name][0], np.int32)
        for name in GLOBAL:
            aux[name] = np.array(a[name], np.int32)

    qkv, out = cfg1_drive(cache, grab)
    np.savez_compressed(os.path.join(HERE, "cfg1_decode.npz"), qkv=qkv, out=out, **aux)


class Recorder:
    """Host-cache facade that records every verb, the auxiliary arrays after each begin_forward,
    and the pool state at the end."""

    def __init__(self, cache_config):
        self.host = hc.HostCache(list(cache_config), [0], 1)
        self.ops = []

    def add_sequence(self, sid):
        self.host.add_sequence(sid)
        self.ops.append({"op": "add", "args": [sid]})

    def fork_sequence(self, parent, child, pos):
        self.host.fork_sequence(parent, child, pos)
        self.ops.append({"op": "fork", "args": [parent, child, pos]})

    def remove_sequence(self, sid):
        self.host.remove_sequence(sid)
        self.ops.append({"op": "remove", "args": [sid]})

    def popn(self, sid, n):
        self.host.popn(sid, n)
        self.ops.append({"op": "popn", "args": [sid, n]})

    def begin_forward(self, ids, lens):
        self.host.begin_forward(list(ids), list(lens), None)
        a = self.host.aux
        rec = {"op": "begin_forward", "args": [list(map(int, ids)), list(map(int, lens))],
               "num_depths": a["num_depths"], "append_before_attn": bool(a["append_before_attn"]),
               "use_decode_kernel": [bool(x) for x in a["use_decode_kernel"][:a["num_depths"]]]}
        for name in PER_DEPTH:
            rec[name] = [list(map(int, a[name][d])) for d in range(a["num_depths"])]
        for name in GLOBAL:
            rec[name] = list(map(int, a[name]))
        self.ops.append(rec)

    def empty(self):
        return self.host.empty()

    def final(self):
        st = self.host.state()
        return {"free_page_ids": list(map(int, st["free_page_ids"])), "free_block_idx": list(map(int, st["free_block_idx"])),
                "blocks": [list(b) for b in st["blocks"]],
                "seqs": {str(k): list(v) for k, v in st["seqs"].items()},
                "copies": [list(c) for c in self.host.copies]}


class VerbsOnly(S.Scenario):
    """tests.scenario.Scenario without tensors."""

    def step(self, batch):
        ids, lens = [], []
        for item, n in batch:
            if isinstance(item, tuple):
                sid, parent, pos = item
                self.cache.fork_sequence(parent, sid, pos)
                self.cached_k[sid] = True
            else:
                sid = item
                if sid not in self.cached_k:
                    self.cache.add_sequence(sid)
                    self.cached_k[sid] = True
            ids.append(sid)
            lens.append(n)
        self.cache.begin_forward(ids, lens)

    def verify_cached_kv(self, seq_ids):
        pass

    def remove(self, sid):
        self.cache.remove_sequence(sid)
        self.cached_k.pop(sid)

    def popn(self, sid, n):
        self.cache.popn(sid, n)


SCENARIOS = {"prefill_and_decode": S.run_prefill_and_decode, "remove_sequence": S.run_remove_sequence,
             "fork_sequence": S.run_fork_sequence, "unlimited_depth": S.run_unlimited_depth, "popn": S.run_popn}
SCENARIO_CACHE_CONFIG = [32, 2048, 512, 16, 0]


def make_host_scenarios():
    out = {"cache_config": SCENARIO_CACHE_CONFIG, "scenarios": {}}
    for name, runner in SCENARIOS.items():
        rec = Recorder(SCENARIO_CACHE_CONFIG)
        runner(VerbsOnly(rec, 1, 8, 2, 64))
        out["scenarios"][name] = {"ops": rec.ops, "final": rec.final()}
    with open(os.path.join(HERE, "host_scenarios.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    make_rope()
    make_cfg1()
    make_host_scenarios()
    for name in ("rope_vectors.npz", "cfg1_decode.npz", "host_scenarios.json"):
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")
