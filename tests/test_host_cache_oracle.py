"""Pins oracle/host_cache.py (the Python restatement of the reference's host bookkeeping).

* hand-derived examples: worked out on paper from src/runtime/vm/paged_kv_cache.cc
  (:606-719 fork, :803-862 popn, :884-1212 begin_forward); the expected values below are typed
  from that derivation, not produced by the code under test;
* the closed form for fork-free runs: pages leave the LIFO free list as 0,1,2,... in
  BeginForward order;
* structural invariants after every operation of the reference's scenario tests;
* end-to-end: the same scenarios through oracle host cache + oracle kernels must reproduce the
  numpy closed-form attention and the cached K/V (what the reference's CPU test asserts).
"""
import numpy as np
import pytest

from oracle import host_cache as hc
from oracle.paged_kv_cache import OraclePagedKVCache
from tests import scenario as S
from tests.invariants import check_pool_invariants
from tests.util import assert_close


def make(capacity=16368, reserved=32, chunk=8192, ps=16, sliding=0):
    return hc.HostCache([reserved, capacity, chunk, ps, sliding])


def test_pool_size_formula():
    assert make().num_total_pages == 1024  # ceil(16368/16) + 1
    assert hc.HostCache([4, 100, 10, 16, 1]).num_total_pages == 7 + 1 + 8
    c = make()
    assert c.free_page_ids[-1] == 0 and c.free_page_ids[0] == 1023 and c.empty()


def test_cfg1_prefill_then_decode_hand_derived():
    c = make()
    for s in range(4):
        c.add_sequence(s)
    aux = c.begin_forward([0, 1, 2, 3], [512, 1024, 1500, 2048])
    assert aux["append_before_attn"] is False and aux["use_decode_kernel"] == [False]
    assert aux["num_depths"] == 1
    assert aux["page_indptr"][0] == [0, 0, 0, 0, 0] and aux["page_indices"][0] == []
    assert aux["qo_indptr"][0] == [0, 512, 1536, 3036, 5084]
    assert aux["last_page_len"][0] == [0, 0, 0, 0]
    assert c.pool[0].page_ids == list(range(0, 32))
    assert c.pool[1].page_ids == list(range(32, 96))
    assert c.pool[2].page_ids == list(range(96, 190))
    assert c.pool[3].page_ids == list(range(190, 318))
    apm = aux["append_position_map"]
    assert apm[:512] == list(range(512))
    assert apm[512:1536] == list(range(512, 1536))
    assert apm[1536:3036] == list(range(1536, 3036))
    assert apm[3036:] == list(range(3040, 5088))
    assert aux["q_rope_position_map"][512:515] == [0, 1, 2]
    assert aux["k_ragged_rope_pos_offset"] == [0, 0, 0, 0]
    aux = c.begin_forward([0, 1, 2, 3], [1, 1, 1, 1])
    assert aux["append_before_attn"] is True and aux["use_decode_kernel"] == [True]
    assert aux["qo_indptr"][0] == [0, 1, 2, 3, 4]
    assert aux["page_indptr"][0] == [0, 33, 98, 192, 321]
    assert aux["page_indices"][0] == (list(range(32)) + [318] + list(range(32, 96)) + [319]
                                      + list(range(96, 190)) + list(range(190, 318)) + [320])
    assert aux["last_page_len"][0] == [1, 1, 13, 1]
    assert aux["k_rope_pos_offset"][0] == [0, 0, 0, 0]
    assert aux["q_rope_position_map"] == [512, 1024, 1500, 2048]
    assert aux["append_position_map"] == [5088, 5104, 3036, 5120]
    assert aux["cur_append_lengths_indptr"] == [0, 1, 2, 3, 4]
    assert aux["k_ragged_rope_pos_offset"] == [512, 1024, 1500, 2048]
    assert c.get_num_available_pages() == 703
    assert c.get_total_sequence_length() == 5088


def _prefill(c, sid, n):
    c.add_sequence(sid)
    c.begin_forward([sid], [n])


def test_fork_inside_a_page_hand_derived():
    c = make()
    _prefill(c, 0, 40)
    assert c.pool[0].as_tuple() == ([0, 1, 2], 40, 0, 0, 0, -1, 1)
    c.fork_sequence(0, 1, -1)
    assert c.pool[2].as_tuple() == ([0, 1], 32, 0, 0, 0, -1, 2)
    assert c.pool[0].as_tuple() == ([2], 8, 32, 0, 0, 2, 1)
    assert c.pool[1].as_tuple() == ([3], 8, 32, 0, 0, 2, 1)
    assert c.copies == [(2, 3, 8)]
    assert (c.seq_map[1].last_block_idx, c.seq_map[1].seq_length) == (1, 40)
    aux = c.begin_forward([0, 1], [1, 1])
    assert aux["num_depths"] == 2
    assert aux["use_decode_kernel"] == [True, True] and aux["append_before_attn"] is True
    assert aux["page_indices"][0] == [0, 1, 0, 1] and aux["page_indptr"][0] == [0, 2, 4]
    assert aux["page_indices"][1] == [2, 3] and aux["page_indptr"][1] == [0, 1, 2]
    assert aux["last_page_len"] == [[16, 16], [9, 9]]
    assert aux["k_rope_pos_offset"] == [[0, 0], [32, 32]]
    assert aux["q_rope_position_map"] == [40, 40]
    assert aux["append_position_map"] == [2 * 16 + 8, 3 * 16 + 8]


def test_fork_at_page_aligned_end_hand_derived():
    c = make()
    _prefill(c, 0, 32)
    c.fork_sequence(0, 1, -1)
    assert c.pool[0].as_tuple() == ([0, 1], 32, 0, 0, 0, -1, 2)
    assert c.pool[1].as_tuple() == ([], 0, 32, 0, 0, 0, 1)   # parent's empty tail block
    assert c.pool[2].as_tuple() == ([], 0, 32, 0, 0, 0, 1)   # child block
    assert c.seq_map[0].last_block_idx == 1 and c.seq_map[1].last_block_idx == 2
    assert c.copies == [] and c.get_num_available_pages() == 1024 - 2
    aux = c.begin_forward([0, 1], [1, 1])
    assert aux["num_depths"] == 2
    assert aux["page_indices"] == [[0, 1, 0, 1], [2, 3]]


def test_fork_at_interior_page_boundary_hand_derived():
    c = make()
    _prefill(c, 0, 40)
    c.fork_sequence(0, 1, 16)
    assert c.pool[2].as_tuple() == ([0], 16, 0, 0, 0, -1, 2)
    assert c.pool[0].as_tuple() == ([1, 2], 24, 16, 0, 0, 2, 1)
    assert c.pool[1].as_tuple() == ([], 0, 16, 0, 0, 2, 1)
    assert c.copies == []
    assert c.seq_map[1].seq_length == 16


def test_popn_inside_unshared_block_hand_derived():
    c = make()
    _prefill(c, 0, 40)
    c.popn(0, 10)
    assert c.pool[0].as_tuple() == ([0, 1], 30, 0, 0, 0, -1, 1)
    assert c.free_page_ids[-1] == 2 and c.seq_map[0].seq_length == 30
    c.begin_forward([0], [3])       # 30 -> 33 tokens: needs page index 2 again, which is next out
    assert c.pool[0].page_ids == [0, 1, 2]


def test_popn_into_shared_prefix_hand_derived():
    # seq0: 40 tokens; fork seq1 at the end (mid-page) -> shared block2 [0,1], block0 [2], block1 [3].
    # popn(1, 20): block1 (8 tokens, unshared) is freed whole (n=12 left); seq1 now ends at shared
    # block2 (ref 2) -> re-fork at 32-12=20 under temp id -2: in_page_offset 4, moved_offset 16,
    # moved_pages 1 -> split block2: new parent block1' (recycled index 1) {pages [0], len 16,
    # ref 2}, block2 {pages [1], len 16, start 16, parent 1}; child block gets a fresh page with a
    # 4-slot copy from page 1.  Free blocks pop LIFO: the freed block index 1 is reused first for
    # the child, so the new parent takes index 3.
    c = make()
    _prefill(c, 0, 40)
    c.fork_sequence(0, 1, -1)
    c.popn(1, 20)
    st = c.state()
    check_pool_invariants(st, 1024, 16)
    seq1 = c.seq_map[1]
    assert seq1.seq_length == 20
    child = c.pool[seq1.last_block_idx]
    assert child.seq_length == 4 and child.start_pos == 16 and len(child.page_ids) == 1
    parent = c.pool[child.parent_idx]
    assert parent.as_tuple()[:3] == ([0], 16, 0) and parent.external_ref_cnt == 2
    assert c.copies[-1] == (1, child.page_ids[0], 4)
    assert child.page_ids[0] == 3  # page 3 was freed by the pop and is the next page handed out
    assert c.seq_map[0].seq_length == 40
    assert c.position_map_of(0) == list(range(40))
    assert c.position_map_of(1) == list(range(16)) + [48, 49, 50, 51]
    assert -2 not in c.seq_map


def test_fork_free_closed_form():
    """No forks, no sliding window: sequence i owns the consecutive page ids popped from the
    free list in BeginForward order, and append slots follow page_ids[t // ps] * ps + t % ps."""
    rng = np.random.default_rng(0)
    c = make(capacity=4096)
    ps = 16
    lengths = {}
    pages = {}
    next_page = 0
    for step in range(12):
        ids = [int(s) for s in rng.permutation(6)[: rng.integers(1, 6)]]
        decode = step % 3 == 2
        lens = [1 if decode else int(rng.integers(1, 40)) for _ in ids]
        for s in ids:
            if s not in lengths:
                c.add_sequence(s)
                lengths[s], pages[s] = 0, []
        aux = c.begin_forward(ids, lens)
        expect_map = []
        for s, n in zip(ids, lens):
            need = (lengths[s] + n + ps - 1) // ps
            while len(pages[s]) < need:
                pages[s].append(next_page)
                next_page += 1
        for s, n in zip(ids, lens):
            for t in range(lengths[s], lengths[s] + n):
                expect_map.append(pages[s][t // ps] * ps + t % ps)
            lengths[s] += n
        assert aux["append_position_map"] == expect_map
        assert aux["q_rope_position_map"] == [t for s, n in zip(ids, lens) for t in range(lengths[s] - n, lengths[s])]
        assert aux["num_depths"] == 1
        if aux["append_before_attn"]:
            assert decode
            assert aux["page_indices"][0] == [p for s in ids for p in pages[s]]
            assert aux["last_page_len"][0] == [(lengths[s] - 1) % ps + 1 for s in ids]
        else:
            # page table excludes the tokens being appended
            old = [lengths[s] - n for s, n in zip(ids, lens)]
            assert aux["page_indptr"][0] == list(np.concatenate([[0], np.cumsum([(o + ps - 1) // ps for o in old])]))
            assert aux["last_page_len"][0] == [0 if o == 0 else (o - 1) % ps + 1 for o in old]
        check_pool_invariants(c.state(), c.num_total_pages, ps)


def test_error_paths():
    c = make(capacity=64, reserved=4, chunk=64)
    c.add_sequence(0)
    with pytest.raises(hc.CacheError, match="already in the KV cache"):
        c.add_sequence(0)
    with pytest.raises(hc.CacheError, match="cannot be found"):
        c.remove_sequence(7)
    with pytest.raises(hc.CacheError, match="cannot be found"):
        c.begin_forward([3], [1])
    c.begin_forward([0], [40])
    with pytest.raises(hc.CacheError, match="exceeds"):
        c.popn(0, 41)
    c.fork_sequence(0, 1, 32)
    c.add_sequence(2)
    with pytest.raises(hc.CacheError, match="full"):
        c.begin_forward([2], [64])          # pool has 5 pages, 3 in use
    c2 = make()
    c2.add_sequence(0)
    c2.begin_forward([0], [16])
    c2.fork_sequence(0, 1, 8)               # fork inside the first page: child shares no block
    c2.begin_forward([0], [1])              # block 0 is still unshared -> fine
    c3 = make()
    c3.add_sequence(0)
    c3.begin_forward([0], [32])
    c3.fork_sequence(0, 1, 16)              # block0 split; seq0's last block [1] len 16 unshared
    c3.fork_sequence(0, 2, 32)              # page-aligned end: seq0 gets an empty tail block
    with pytest.raises(hc.CacheError, match="Append with length 0"):
        c3.begin_forward([0], [0])


@pytest.mark.parametrize("rope_mode", [S.ROPE_NORMAL, S.ROPE_NONE])
@pytest.mark.parametrize("runner", [S.run_prefill_and_decode, S.run_remove_sequence, S.run_fork_sequence,
                                    S.run_unlimited_depth, S.run_popn])
def test_reference_scenarios_on_the_oracle(runner, rope_mode):
    layers, hq, hkv, d, ps = 2, 8, 2, 64, 16
    cache = OraclePagedKVCache([32, 2048, 512, ps, 0], layers, hq, hkv, d, d, rope_mode=rope_mode)

    def on_step(seq_ids, lens):
        check_pool_invariants(cache.host.state(), cache.host.num_total_pages, ps)

    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=rope_mode, seed=3, on_step=on_step)
    runner(sc)
    check_pool_invariants(cache.host.state(), cache.host.num_total_pages, ps)


def _attended_slots(aux, depth, row, page_size):
    """Slots the step's page table lets sequence `row` attend to at `depth`: sink tokens, then the
    window (python/tvm/relax/frontend/nn/llm/_kernel_common.py:155-170)."""
    lo, hi = aux["page_indptr"][depth][row], aux["page_indptr"][depth][row + 1]
    pages = aux["page_indices"][depth][lo:hi]
    if not pages:
        return set()
    phys_len = (len(pages) - 1) * page_size + aux["last_page_len"][depth][row]
    sink, win_lo = aux["sink_size"][depth][row], aux["sliding_window_offset"][depth][row]
    tokens = list(range(sink)) + list(range(win_lo, phys_len))
    return {pages[t // page_size] * page_size + t % page_size for t in tokens}


def test_sliding_window_reuses_attended_slots_within_a_step():
    """Why a sliding-window cache must append AFTER attention: in this batch the new tokens of one
    sequence are given slots that the same step's page table of another sequence attends to.  The
    oracle (which follows the reference's order) and the closed form still agree on every output."""
    ps = 16
    host = hc.HostCache([32, 2048, 512, ps, 1], [hc.ATTN_MHA], hc.ROPE_NORMAL)
    for sid in range(4):
        host.add_sequence(sid)
        host.enable_sliding_window_for_seq(sid, 40, 4)
    clashes = []
    for _ in range(6):
        host.begin_forward([0, 1, 2, 3], [17] * 4)
        assert not host.aux["append_before_attn"]
        attended = [_attended_slots(host.aux, 0, row, ps) for row in range(4)]
        new = [s for s in host.aux["append_position_map"] if s != -1]
        indptr = host.aux["cur_append_lengths_indptr"]
        clash = 0
        for row in range(4):
            mine = set(host.aux["append_position_map"][indptr[row]:indptr[row + 1]]) - {-1}
            clash += sum(len(mine & attended[other]) for other in range(4) if other != row)
        clashes.append(clash)
        assert len(new) == len(set(new)), "two new tokens share a slot"
        host.end_forward()
    assert clashes[:3] == [0, 0, 0] and all(c > 0 for c in clashes[3:]), clashes


@pytest.mark.parametrize("runner", [S.run_sliding_window, S.run_sliding_window_fork, S.run_sliding_window_page_reuse])
def test_sliding_window_scenarios_on_the_oracle(runner):
    """Sliding-window cache with attention sinks: RoPE is applied inside the kernels at positions
    counted inside the cache (the reference switches such caches to INLINE mode,
    src/runtime/vm/paged_kv_cache.cc:343-345)."""
    layers, hq, hkv, d, ps = 2, 8, 2, 64, 16
    cache = OraclePagedKVCache([32, 2048, 512, ps, 1], layers, hq, hkv, d, d, rope_mode=S.ROPE_INLINE)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=S.ROPE_INLINE, seed=4)
    runner(sc)


@pytest.mark.parametrize("rope_mode", [S.ROPE_NORMAL, S.ROPE_NONE])
def test_token_tree_scenario_on_the_oracle(rope_mode):
    """Speculative decoding: tree-masked attention over new tokens and over appended tree nodes,
    commit of an accepted path (slots compacted, the rest popped), then plain decode."""
    layers, hq, hkv, d, ps = 2, 8, 2, 64, 16
    cache = OraclePagedKVCache([32, 2048, 512, ps, 0], layers, hq, hkv, d, d, rope_mode=rope_mode)

    def on_step(seq_ids, lens):
        check_pool_invariants(cache.host.state(), cache.host.num_total_pages, ps)

    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=rope_mode, seed=6, on_step=on_step)
    S.run_tree_attn(sc)
    check_pool_invariants(cache.host.state(), cache.host.num_total_pages, ps)


def test_attention_with_shared_kv_on_the_oracle():
    """src/runtime/vm/paged_kv_cache.cc:1487-1525: queries of another layer attend to layer 0's cached
    K/V plus the step's own rows; equals the closed form over layer 0's K/V, in prefill and decode."""
    from oracle import closed_form as cf
    layers, hq, hkv, d = 2, 4, 2, 64
    cache = OraclePagedKVCache([4, 256, 64, 16, 0], layers, hq, hkv, d, d, rope_mode=S.ROPE_NONE)
    rng = np.random.default_rng(5)
    cache.add_sequence(0)
    ks, vs = np.zeros((0, hkv, d), np.float16), np.zeros((0, hkv, d), np.float16)
    for n in (21, 12, 1, 1):
        qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(np.float16)
        q2 = rng.standard_normal((n, hq, d)).astype(np.float16)
        k_cur, v_cur = np.ascontiguousarray(qkv[:, hq:hq + hkv]), np.ascontiguousarray(qkv[:, hq + hkv:])
        cache.begin_forward([0], [n])
        o1, o2 = np.zeros((n, hq, d), np.float16), np.zeros((n, hq, d), np.float16)
        cache.attention_with_fused_qkv(0, d ** -0.5, qkv, o1)
        cache.attention_with_shared_kv(0, d ** -0.5, q2, k_cur, v_cur, o2)
        cache.end_forward()
        ks, vs = np.concatenate([ks, k_cur]), np.concatenate([vs, v_cur])
        expected, _ = cf.attention(q2, ks, vs, d ** -0.5, causal=True)
        assert_close(o2, expected, atol=2e-3, rtol=2e-3, what=f"shared-kv attention, append {n}")
