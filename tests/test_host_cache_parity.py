"""Bit-exact parity of the shipped C++ host cache (libtvmkv.so, host-only mode) with the Python
oracle of the reference's bookkeeping: page tables, append indices, every other auxiliary
array, the fork copy log and the whole pool state, after every operation of the reference's
scenario batches and of seeded random operation sequences (forks at arbitrary positions,
popn into shared prefixes, removals, page recycling, sliding windows, token trees)."""
import numpy as np
import pytest

import tvm_amd
from oracle import host_cache as hc
from tests import scenario as S
from tests.invariants import check_pool_invariants
from tvm_amd import get_global_func as gf

PER_DEPTH = ["qo_indptr", "page_indptr", "page_indices", "last_page_len", "sliding_window_offset", "sink_size",
             "k_rope_pos_offset", "page_indptr_sliding_window", "page_indices_sliding_window",
             "k_rope_pos_offset_sliding_window"]
GLOBAL = ["q_rope_position_map", "append_position_map", "cur_append_lengths_indptr", "k_ragged_rope_pos_offset"]


class Pair:
    """Drives the oracle and the C++ cache with the same calls and compares after each."""

    def __init__(self, cache_config, attn_kinds=(0,), rope_mode=1):
        self.oracle = hc.HostCache(list(cache_config), list(attn_kinds), rope_mode)
        self.cache = gf("vm.builtin.paged_attention_kv_cache_create")(
            list(cache_config), [0, len(attn_kinds)], 8, 2, 64, 64, list(attn_kinds), False, rope_mode, 1.0, 1e4,
            None, "host")
        self.page_size = cache_config[3]

    def both(self, oracle_call, name, *args):
        o_err = c_err = None
        try:
            oracle_call(*args)
        except hc.CacheError as e:
            o_err = str(e)
        try:
            gf(name)(self.cache, *args)
        except tvm_amd.KVError as e:
            c_err = str(e)
        assert (o_err is None) == (c_err is None), f"{name}{args}: oracle error {o_err!r} vs library error {c_err!r}"
        return o_err is None

    def compare_state(self):
        so, sc = self.oracle.state(), self.cache.state()
        assert sc["free_page_ids"] == so["free_page_ids"]
        assert sc["free_block_idx"] == so["free_block_idx"]
        assert [tuple(b) for b in sc["blocks"]] == [tuple(b) for b in so["blocks"]]
        assert sc["seqs"] == so["seqs"]
        assert self.cache.copy_log() == self.oracle.copies
        assert gf("vm.builtin.attention_kv_cache_empty")(self.cache) == self.oracle.empty()
        assert gf("vm.builtin.attention_kv_cache_get_num_available_pages")(self.cache) == self.oracle.get_num_available_pages()
        assert gf("vm.builtin.attention_kv_cache_get_total_sequence_length")(self.cache) == self.oracle.get_total_sequence_length()

    def compare_aux(self):
        aux = self.oracle.aux
        flags = self.cache.flags()
        assert flags["num_depths"] == aux["num_depths"]
        assert bool(flags["append_before_attn"]) == aux["append_before_attn"]
        for d in range(aux["num_depths"]):
            assert bool(flags[f"use_decode_kernel_{d}"]) == aux["use_decode_kernel"][d]
            assert bool(flags[f"is_chain_{d}"]) == aux["is_chain_on_depths"][d]
            for name in PER_DEPTH:
                assert self.cache.aux(name, d) == aux[name][d], f"{name}[{d}]"
            if not aux["is_chain_on_depths"][d]:
                assert self.cache.aux("tree_attn_mask", d) == aux["tree_attn_mask"][d]
                assert self.cache.aux("tree_attn_mn_indptr", d) == aux["tree_attn_mn_indptr"][d]
        for name in GLOBAL:
            assert self.cache.aux(name) == aux[name], name

    def add(self, sid):
        ok = self.both(self.oracle.add_sequence, "vm.builtin.kv_state_add_sequence", sid)
        self.compare_state()
        return ok

    def remove(self, sid):
        ok = self.both(self.oracle.remove_sequence, "vm.builtin.kv_state_remove_sequence", sid)
        self.compare_state()
        return ok

    def fork(self, parent, child, pos):
        ok = self.both(self.oracle.fork_sequence, "vm.builtin.kv_state_fork_sequence", parent, child, pos)
        self.compare_state()
        return ok

    def popn(self, sid, n):
        ok = self.both(self.oracle.popn, "vm.builtin.kv_state_popn", sid, n)
        self.compare_state()
        return ok

    def begin_forward(self, ids, lens, tree=None):
        ok = self.both(self.oracle.begin_forward, "vm.builtin.kv_state_begin_forward", ids, lens, tree)
        self.compare_state()
        if ok:
            self.compare_aux()
        return ok


class ScenarioAdapter:
    """Lets tests.scenario drive a Pair: only the bookkeeping verbs matter here."""

    def __init__(self, pair):
        self.p = pair

    def add_sequence(self, sid):
        assert self.p.add(sid)

    def fork_sequence(self, parent, child, pos):
        assert self.p.fork(parent, child, pos)

    def remove_sequence(self, sid):
        assert self.p.remove(sid)

    def popn(self, sid, n):
        assert self.p.popn(sid, n)

    def begin_forward(self, ids, lens):
        assert self.p.begin_forward(ids, lens)

    def empty(self):
        return self.p.oracle.empty()


class BookkeepingOnly(S.Scenario):
    """tests.scenario.Scenario without tensors: replays the verbs of the reference's batches."""

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


@pytest.mark.parametrize("runner", [S.run_prefill_and_decode, S.run_remove_sequence, S.run_fork_sequence,
                                    S.run_unlimited_depth, S.run_popn])
def test_reference_scenarios_bit_exact(runner):
    pair = Pair([32, 2048, 512, 16, 0])
    runner(BookkeepingOnly(ScenarioAdapter(pair), 1, 8, 2, 64))


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("page_size,sliding", [(16, 0), (4, 0), (16, 1)])
def test_random_operation_sequences(seed, page_size, sliding):
    rng = np.random.default_rng(1000 * page_size + seed + 7 * sliding)
    rope = 0 if sliding else 1
    pair = Pair([16, 40 * page_size, 64 * page_size, page_size, sliding], rope_mode=rope)
    live, lengths, windowed = [], {}, set()
    next_id = 0
    consistent = True  # a begin_forward that fails half way leaves lengths bumped, in both implementations
    for _ in range(120):
        op = rng.choice(["add", "forward", "forward", "decode", "decode", "fork", "popn", "remove", "bad"])
        if op == "add" or not live:
            if pair.add(next_id):
                live.append(next_id)
                lengths[next_id] = 0
                if sliding and rng.random() < 0.5:
                    w, sink = int(rng.integers(2, 3 * page_size)), int(rng.integers(0, 4))
                    o_ok = pair.both(pair.oracle.enable_sliding_window_for_seq,
                                     "vm.builtin.attention_kv_cache_enable_sliding_window_for_seq", next_id, w, sink)
                    if o_ok:
                        windowed.add(next_id)
            next_id += 1
        elif op in ("forward", "decode"):
            k = int(rng.integers(1, min(len(live), 5) + 1))
            ids = [int(x) for x in rng.permutation(live)[:k]]
            lens = [1 if op == "decode" else int(rng.integers(1, 3 * page_size)) for _ in ids]
            ok = pair.begin_forward(ids, lens)
            # lengths are only tracked for choosing fork/pop positions; the oracle is the truth
            for s in live:
                lengths[s] = pair.oracle.seq_map[s].seq_length if s in pair.oracle.seq_map else 0
            if not ok:
                # a failed begin_forward (pool exhausted, shared block) leaves both sides in the same
                # partially updated state (the reference bumps seq_length before reserving pages,
                # src/runtime/vm/paged_kv_cache.cc:919); keep comparing, stop checking invariants
                consistent = False
        elif op == "fork":
            parent = int(rng.choice(live))
            pos = int(rng.integers(-1, lengths[parent] + 1))
            if pair.fork(parent, next_id, pos):
                live.append(next_id)
                lengths[next_id] = pair.oracle.seq_map[next_id].seq_length
            else:
                consistent = False  # "cache is full" strikes after the child block was linked in
            next_id += 1
        elif op == "popn":
            sid = int(rng.choice(live))
            n = int(rng.integers(0, lengths[sid] + 2))
            if sid in windowed:
                continue  # the reference drops the window settings on a re-forking pop
            if pair.popn(sid, n):
                lengths[sid] = pair.oracle.seq_map[sid].seq_length
            elif n <= lengths[sid]:
                consistent = False  # failed inside the re-fork
        elif op == "remove":
            sid = int(rng.choice(live))
            if pair.remove(sid):
                live.remove(sid)
        else:
            pair.add(int(rng.choice(live)))            # duplicate id
            pair.remove(next_id + 1000)                # unknown id
            pair.begin_forward([next_id + 1000], [1])  # unknown id
        if not consistent:
            # the half-applied operation left the pool in a state the reference does not define
            # either (it would index an empty page list next); both sides agreed up to here
            return
        if not sliding:
            check_pool_invariants(pair.cache.state(), pair.oracle.num_total_pages, page_size)
    for sid in list(live):
        pair.remove(sid)
    assert pair.oracle.empty() and gf("vm.builtin.attention_kv_cache_empty")(pair.cache)


def test_token_tree_bookkeeping():
    pair = Pair([8, 512, 256, 16, 0])
    pair.add(0)
    pair.add(1)
    assert pair.begin_forward([0, 1], [10, 20])
    # a chain for seq 1 and a tree for seq 0 (0 -> {1, 2}, 1 -> 3); the reference decides "is a
    # chain" from the LAST sequence of the commit (src/runtime/vm/paged_kv_cache.cc:1580), so the
    # tree goes last
    assert pair.begin_forward([1, 0], [3, 4], [-1, 0, 1, -1, 0, 0, 2])
    leaf = [2, 3]
    o = pair.oracle.commit_accepted_token_tree_nodes([1, 0], leaf)
    # accepted path 0 -> 2 -> 3 moves node 2 to position 1 and node 3 to position 2 (in that order);
    # seq 0 holds 10 tokens in page 0, so tree node i sits in slot 10 + i
    assert o == ([0, 0, 2], [12, 13], [11, 12])
    # host-only cache: the device copy is skipped, the bookkeeping is not
    gf("vm.builtin.attention_kv_cache_commit_accepted_token_tree_nodes")(pair.cache, [1, 0], leaf)
    assert pair.cache.aux("commit_copy_length_indptr") == o[0]
    assert pair.cache.aux("commit_copy_src_pos") == o[1]
    assert pair.cache.aux("commit_copy_dst_pos") == o[2]
    pair.compare_state()
    assert pair.begin_forward([0, 1], [1, 1])


def test_error_messages_match_the_reference_text():
    c = gf("vm.builtin.paged_attention_kv_cache_create")([4, 64, 64, 16, 0], [0, 1], 8, 2, 64, 64, [0], False, 1,
                                                          1.0, 1e4, None, "host")
    add = gf("vm.builtin.kv_state_add_sequence")
    add(c, 0)
    with pytest.raises(tvm_amd.KVError, match='The sequence "0" is already in the KV cache.'):
        add(c, 0)
    with pytest.raises(tvm_amd.KVError, match='The sequence "9" cannot be found in KV cache.'):
        gf("vm.builtin.kv_state_remove_sequence")(c, 9)
    gf("vm.builtin.kv_state_begin_forward")(c, [0], [40])
    with pytest.raises(tvm_amd.KVError, match="exceeds the whole sequence length"):
        gf("vm.builtin.kv_state_popn")(c, 0, 41)
    add(c, 1)
    with pytest.raises(tvm_amd.KVError, match="The KV cache is full. No page can be allocated."):
        gf("vm.builtin.kv_state_begin_forward")(c, [1], [64])
    # the failed step had already bumped the sequence's length (as the reference does before it reserves pages,
    # src/runtime/vm/paged_kv_cache.cc:919): the object refuses everything but clear until it has been cleared
    with pytest.raises(tvm_amd.KVError, match="call clear before using the cache again"):
        gf("vm.builtin.kv_state_begin_forward")(c, [0], [1])
    with pytest.raises(tvm_amd.KVError, match="call clear"):
        add(c, 2)
    gf("vm.builtin.kv_state_clear")(c)
    add(c, 0)
    with pytest.raises(tvm_amd.KVError, match="Append with length 0 is not allowed."):
        gf("vm.builtin.kv_state_begin_forward")(c, [0], [0])
    # ... while a step that fails before it has changed anything leaves the cache usable
    with pytest.raises(tvm_amd.KVError, match="cannot be found in KV cache"):
        gf("vm.builtin.kv_state_begin_forward")(c, [7], [1])
    gf("vm.builtin.kv_state_begin_forward")(c, [0], [3])
    with pytest.raises(tvm_amd.KVError) as info:
        gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")(c, 0, 1.0, _Fake(), _Fake())
    assert info.value.code == -4  # host-only cache: no device work, no CPU fallback
    with pytest.raises(tvm_amd.KVError, match="not part of the paged KV-cache path"):
        gf("vm.builtin.attention_kv_cache_debug_set_kv")


class _Fake:
    shape = (1, 12, 64)

    def data_ptr(self):
        return 0

    def is_contiguous(self):
        return True


def test_storage_types_and_shapes_a_cache_accepts():
    """float16 and float32 storage (the reference's tests run both); float32, pages other than 16 / 32 / 64 / 128
    tokens and other head dims run on the generic kernels, sliding windows and RoPE inside the attention kernels
    included (that rotation needs a head dim that is a multiple of 16, of 8 with float32)."""
    import torch
    create = tvm_amd.get_global_func("vm.builtin.paged_attention_kv_cache_create")

    def make(config, d, rope_mode, dtype):
        return create(config, [0, 1], 8, 2, d, d, [0], False, rope_mode, 1.0, 1e4, None, torch.empty((), dtype=dtype))

    for dtype in (torch.float16, torch.float32):
        cache = make([4, 64, 32, 16, 0], 128, 1, dtype)
        assert cache.dtype_bits == (16 if dtype == torch.float16 else 32)
        tvm_amd.get_global_func("vm.builtin.kv_state_add_sequence")(cache, 0)
    make([4, 64, 32, 24, 0], 72, 1, torch.float16)           # pages of 24 tokens, head dim 72: the generic kernels
    make([4, 64, 32, 24, 1], 128, 0, torch.float16)          # pages of 24 tokens with a sliding window
    make([4, 64, 32, 16, 1], 128, 1, torch.float32)          # float32 with a sliding window (which rotates in the kernels)
    make([4, 64, 32, 24, 0], 128, 2, torch.float16)          # pages of 24 tokens with RoPE inside the kernels
    make([4, 64, 32, 16, 1], 96, 1, torch.float16)           # head dim 96 with a sliding window
    with pytest.raises(tvm_amd.KVError, match="multiple of 16"):
        make([4, 64, 32, 16, 0], 72, 2, torch.float16)       # RoPE inside the kernels at head dim 72
    with pytest.raises(tvm_amd.KVError, match="multiple of 8"):
        make([4, 64, 32, 16, 1], 68, 1, torch.float32)
    with pytest.raises(tvm_amd.KVError, match="float16 and float32"):
        make([4, 64, 32, 16, 0], 128, 1, torch.bfloat16)
