"""The committed golden fixtures (tests/golden/, written by tests/golden/make_fixtures.py) against
the CPU oracle and against the shipped C++ host cache in host-only mode: the verb sequences of the
reference's KV-cache tests must reproduce every recorded auxiliary array and the final pool state
bit for bit."""
import json
import os

import numpy as np
import pytest

from oracle import kernels as ok
from tests.golden import make_fixtures as mf
from tvm_amd import get_global_func as gf

GOLD = os.path.dirname(os.path.abspath(mf.__file__))


def test_oracle_rope_matches_fixture():
    g = np.load(os.path.join(GOLD, "rope_vectors.npz"))
    qkv, pos = mf.rope_inputs()
    assert np.array_equal(qkv, g["qkv"]) and np.array_equal(pos, g["pos"])
    q, k, v = np.zeros_like(g["q"]), np.zeros_like(g["k"]), np.zeros_like(g["v"])
    ok.fused_rope(qkv, pos, q, k, v, 1, theta=1e4, scale=1.0)
    assert np.array_equal(q, g["q"]) and np.array_equal(k, g["k"]) and np.array_equal(v, g["v"])
    # position 0 is the identity, v is never rotated
    assert np.array_equal(g["q"][0], qkv[0, :2]) and np.array_equal(g["v"], qkv[:, 3:])


def _scenarios():
    with open(os.path.join(GOLD, "host_scenarios.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("name", sorted(mf.SCENARIOS))
def test_oracle_host_cache_matches_fixture(name):
    gold = _scenarios()
    rec = mf.Recorder(gold["cache_config"])
    mf.SCENARIOS[name](mf.VerbsOnly(rec, 1, 8, 2, 64))
    assert json.loads(json.dumps(rec.ops)) == gold["scenarios"][name]["ops"]
    assert json.loads(json.dumps(rec.final())) == gold["scenarios"][name]["final"]


@pytest.mark.parametrize("name", sorted(mf.SCENARIOS))
def test_library_host_cache_matches_fixture(name):
    gold = _scenarios()
    cfg = gold["cache_config"]
    cache = gf("vm.builtin.paged_attention_kv_cache_create")(cfg, [0, 1], 8, 2, 64, 64, [0], False, 1, 1.0, 1e4, None,
                                                             "host")
    verbs = {"add": "vm.builtin.kv_state_add_sequence", "fork": "vm.builtin.kv_state_fork_sequence",
             "remove": "vm.builtin.kv_state_remove_sequence", "popn": "vm.builtin.kv_state_popn"}
    for op in gold["scenarios"][name]["ops"]:
        if op["op"] != "begin_forward":
            gf(verbs[op["op"]])(cache, *op["args"])
            continue
        gf("vm.builtin.kv_state_begin_forward")(cache, op["args"][0], op["args"][1], None)
        flags = cache.flags()
        assert flags["num_depths"] == op["num_depths"]
        assert bool(flags["append_before_attn"]) == op["append_before_attn"]
        for d in range(op["num_depths"]):
            assert bool(flags[f"use_decode_kernel_{d}"]) == op["use_decode_kernel"][d]
            for arr in mf.PER_DEPTH:
                assert cache.aux(arr, d) == op[arr][d], f"{name}: {arr}[{d}]"
        for arr in mf.GLOBAL:
            assert cache.aux(arr) == op[arr], f"{name}: {arr}"
    final = gold["scenarios"][name]["final"]
    st = cache.state()
    assert st["free_page_ids"] == final["free_page_ids"]
    assert st["free_block_idx"] == final["free_block_idx"]
    assert [list(b) for b in st["blocks"]] == final["blocks"]
    assert {str(k): list(v) for k, v in st["seqs"].items()} == final["seqs"]
    assert [list(c) for c in cache.copy_log()] == final["copies"]


def test_cfg1_page_table_is_the_closed_form():
    """No forks, no sliding window: pages are popped from the free list in begin_forward
    order, so the table and the append indices of the decode step can be written down by hand."""
    g = np.load(os.path.join(GOLD, "cfg1_decode.npz"))
    c = mf.CFG1
    ps = c["page"]
    next_page = 0  # the free list is filled from the highest id down and handed out from its back
    owned = []
    for ctx in c["ctx"]:
        pages, done = [], 0
        while done < ctx:  # one begin_forward per 512-token chunk
            n = min(512, ctx - done)
            need = (done + n + ps - 1) // ps - len(pages)
            pages += [next_page + i for i in range(need)]
            next_page += need
            done += n
        owned.append(pages)
    for b, ctx in enumerate(c["ctx"]):  # the decode step appends one token
        if (ctx + 1 + ps - 1) // ps > len(owned[b]):
            owned[b].append(next_page)
            next_page += 1
    assert list(g["page_indices"]) == [p for pages in owned for p in pages]
    assert list(g["page_indptr"]) == list(np.concatenate([[0], np.cumsum([len(p) for p in owned])]))
    assert list(g["last_page_len"]) == [ctx % ps + 1 for ctx in c["ctx"]]
    assert list(g["q_rope_position_map"]) == c["ctx"]
    assert list(g["append_position_map"]) == [owned[b][ctx // ps] * ps + ctx % ps for b, ctx in enumerate(c["ctx"])]
    assert list(g["k_rope_pos_offset"]) == [0] * 4
