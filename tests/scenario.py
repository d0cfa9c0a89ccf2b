"""Scenario driver shared by the CPU-oracle tests and the GPU parity tests.

It replays the batches of the reference's own KV-cache tests
(tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:327-593, :706-909):
every step forks / adds sequences, calls begin_forward, pushes seeded q/k/v through
``attention_with_fused_qkv`` for every layer, checks the outputs against the numpy closed form
(softmax(QK^T/sqrt(D) + causal) V with RoPE applied up front) and checks the cached K/V of
every touched sequence through ``debug_get_kv``.

``cache`` is any object with the method names of ``oracle.paged_kv_cache.OraclePagedKVCache``;
``tests/test_gpu_*.py`` wrap the HIP-backed cache in the same interface.
"""
import numpy as np

from oracle import closed_form as cf
from tests.util import assert_close

ROPE_NONE, ROPE_NORMAL, ROPE_INLINE = 0, 1, 2


class Scenario:
    def __init__(self, cache, num_layers, hq, hkv, d, rope_mode=ROPE_NORMAL, rope_scale=1.0,
                 rope_theta=1e4, seed=0, tol=2e-3, normal=False, on_step=None, dtype=np.float16):
        self.cache = cache
        self.dtype = dtype  # storage type of the cache under test (float16 or float32)
        self.num_layers, self.hq, self.hkv, self.d = num_layers, hq, hkv, d
        self.rope_mode, self.rope_scale, self.rope_theta = rope_mode, rope_scale, rope_theta
        self.rng = np.random.default_rng(seed)
        self.sm_scale = d ** -0.5
        self.cached_k = {}
        self.cached_v = {}
        self.tol = tol
        self.normal = normal
        self.on_step = on_step
        self.window = {}  # seq_id -> (window, sink)

    def _rand(self, *shape):
        if self.normal:
            return self.rng.standard_normal(shape).astype(self.dtype)
        return self.rng.random(shape).astype(self.dtype)  # the reference test draws uniform [0,1)

    def verify_cached_kv(self, seq_ids):
        for sid in seq_ids:
            ek, ev = self.cached_k[sid], self.cached_v[sid]
            n = ek.shape[1]
            if n == 0:
                continue
            k = np.zeros((self.num_layers, n, self.hkv, self.d), self.dtype)
            v = np.zeros_like(k)
            self.cache.debug_get_kv(sid, 0, n, k, v)
            assert_close(k, ek, atol=2e-3, rtol=2e-3, what=f"cached k of seq {sid}")
            assert np.array_equal(v, ev), f"cached v of seq {sid} differs"

    def step(self, batch, trees=None, accepted=None):
        """batch: list of (seq_id, append_length) or ((seq_id, parent, fork_pos), append_length).

        trees: per sequence the parent pointers of its whole token tree, whose last append_length
        nodes are the new tokens; accepted: per sequence the leaf whose root path is kept when the
        step is committed, -1 for none (test_runtime_builtin_paged_attention_kv_cache_tir.py:396-668).
        """
        cache = self.cache
        seq_ids, append_lengths = [], []
        for item, n in batch:
            if isinstance(item, tuple):
                sid, parent, fork_pos = item
                cache.fork_sequence(parent, sid, fork_pos)
                if fork_pos == -1:
                    self.cached_k[sid] = self.cached_k[parent]
                    self.cached_v[sid] = self.cached_v[parent]
                else:
                    self.cached_k[sid] = self.cached_k[parent][:, :fork_pos]
                    self.cached_v[sid] = self.cached_v[parent][:, :fork_pos]
            else:
                sid = item
                if sid not in self.cached_k:
                    cache.add_sequence(sid)
                    self.cached_k[sid] = np.zeros((self.num_layers, 0, self.hkv, self.d), self.dtype)
                    self.cached_v[sid] = np.zeros((self.num_layers, 0, self.hkv, self.d), self.dtype)
            seq_ids.append(sid)
            append_lengths.append(n)

        depths = [None] * len(seq_ids)
        if trees is not None:
            assert self.rope_mode != ROPE_INLINE, "tree attention has no inline RoPE"
            flat = []
            for i, (tree, n) in enumerate(zip(trees, append_lengths)):
                assert len(tree) >= n
                flat += tree[-n:]
                depths[i] = []
                for parent in tree:
                    depths[i].append(0 if parent == -1 else depths[i][parent] + 1)
            cache.begin_forward(seq_ids, append_lengths, flat)
        else:
            cache.begin_forward(seq_ids, append_lengths)
        if self.on_step is not None:
            self.on_step(seq_ids, append_lengths)

        new_q, new_k, new_v, positions = [], [], [], []
        for i, (sid, n) in enumerate(zip(seq_ids, append_lengths)):
            q = self._rand(self.num_layers, n, self.hq, self.d)
            k = self._rand(self.num_layers, n, self.hkv, self.d)
            v = self._rand(self.num_layers, n, self.hkv, self.d)
            if trees is None:
                pos = self.cached_k[sid].shape[1] + np.arange(n)
            else:  # a tree node sits at its depth behind the tokens in front of the tree
                tree_begin = self.cached_k[sid].shape[1] - (len(trees[i]) - n)
                pos = tree_begin + np.array(depths[i][-n:])
            positions.append(pos)
            if self.rope_mode == ROPE_NORMAL:
                k_store = np.stack([cf.apply_rotary(k[l], pos, self.rope_scale, self.rope_theta)
                                    for l in range(self.num_layers)]).astype(self.dtype)
            else:
                k_store = k
            self.cached_k[sid] = np.concatenate([self.cached_k[sid], k_store], axis=1)
            self.cached_v[sid] = np.concatenate([self.cached_v[sid], v], axis=1)
            new_q.append(q)
            new_k.append(k)
            new_v.append(v)

        total = sum(append_lengths)
        for layer in range(self.num_layers):
            qkv = np.concatenate([np.concatenate([q[layer] for q in new_q]),
                                  np.concatenate([k[layer] for k in new_k]),
                                  np.concatenate([v[layer] for v in new_v])], axis=1)
            out = np.zeros((total, self.hq, self.d), self.dtype)
            cache.attention_with_fused_qkv(layer, self.sm_scale, np.ascontiguousarray(qkv), out)
            cursor = 0
            for i, (sid, n) in enumerate(zip(seq_ids, append_lengths)):
                q_seq = new_q[i][layer]
                k_seq = self.cached_k[sid][layer]
                if self.rope_mode != ROPE_NONE:
                    q_seq = cf.apply_rotary(q_seq, positions[i], self.rope_scale, self.rope_theta)
                if self.rope_mode == ROPE_INLINE:
                    k_seq = cf.apply_rotary(k_seq, np.arange(k_seq.shape[0]), self.rope_scale, self.rope_theta)
                mask = None
                if trees is not None:
                    total_kv, tree_size = k_seq.shape[0], len(trees[i])
                    mask = np.ones((n, total_kv), bool)
                    mask[:, total_kv - tree_size:] = cf.tree_ancestor_mask(trees[i])[tree_size - n:]
                expected, _ = cf.attention(q_seq, k_seq, self.cached_v[sid][layer], self.sm_scale, causal=True,
                                           mask=mask)
                assert_close(out[cursor:cursor + n], expected, atol=self.tol, rtol=self.tol,
                             what=f"attention output, layer {layer}, seq {sid}")
                cursor += n
        cache.end_forward()
        if accepted is not None:
            cache.commit_accepted_token_tree_nodes(seq_ids, accepted)
            for i, (sid, n) in enumerate(zip(seq_ids, append_lengths)):
                path, node = [], accepted[i]
                while node != -1:
                    path.append(node)
                    node = trees[i][node]
                begin = self.cached_k[sid].shape[1] - n
                for dst, src in enumerate(reversed(path)):
                    self.cached_k[sid][:, begin + dst] = self.cached_k[sid][:, begin + src]
                    self.cached_v[sid][:, begin + dst] = self.cached_v[sid][:, begin + src]
                if n - len(path) > 0:
                    self.cached_k[sid] = self.cached_k[sid][:, :len(path) - n]
                    self.cached_v[sid] = self.cached_v[sid][:, :len(path) - n]
        # the sliding window takes effect after the step: keep the attention sink and the newest tokens
        # (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:566-590)
        for sid in seq_ids:
            window, sink = self.window.get(sid, (0, 0))
            n = self.cached_k[sid].shape[1]
            if window and n > window:
                cut = sink + (n - window)
                self.cached_k[sid] = np.concatenate([self.cached_k[sid][:, :sink], self.cached_k[sid][:, cut:]], axis=1)
                self.cached_v[sid] = np.concatenate([self.cached_v[sid][:, :sink], self.cached_v[sid][:, cut:]], axis=1)
        self.verify_cached_kv(seq_ids)

    def add_with_window(self, sid, window, sink):
        self.cache.add_sequence(sid)
        self.cache.enable_sliding_window_for_seq(sid, window, sink)
        self.cached_k[sid] = np.zeros((self.num_layers, 0, self.hkv, self.d), self.dtype)
        self.cached_v[sid] = np.zeros((self.num_layers, 0, self.hkv, self.d), self.dtype)
        self.window[sid] = (window, sink)

    def fork_with_window(self, parent, sid, pos, window, sink):
        self.cache.fork_sequence(parent, sid, pos)
        self.cache.enable_sliding_window_for_seq(sid, window, sink)
        self.cached_k[sid] = self.cached_k[parent][:, :pos]
        self.cached_v[sid] = self.cached_v[parent][:, :pos]
        self.window[sid] = (window, sink)

    def remove(self, sid):
        self.cache.remove_sequence(sid)
        self.cached_k.pop(sid)
        self.cached_v.pop(sid)

    def popn(self, sid, n):
        self.cache.popn(sid, n)
        if n:
            self.cached_k[sid] = self.cached_k[sid][:, :-n]
            self.cached_v[sid] = self.cached_v[sid][:, :-n]


# The batches of the reference's scenario tests, as data ------------------------------------
PREFILL_AND_DECODE = (
    [[(0, 6)], [(1, 8)], [(2, 11)], [(3, 16)], [(4, 19), (5, 20)]]
    + [[(6, 21), (7, 24)], [(2, 5), (4, 7), (8, 24)]]
    + [[(6, 13)], [(8, 19)], [(0, 1)], [(1, 3), (3, 8), (5, 12), (7, 11)]]
    + [[(i, 1) for i in range(9)]] * 2
    + [[(0, 1), (2, 1), (4, 1), (6, 1), (8, 1)]]
    + [[(4, 1), (5, 1), (6, 1), (7, 1), (8, 1)]]
)


def run_prefill_and_decode(sc):
    for batch in PREFILL_AND_DECODE:
        sc.step(list(batch))


def run_remove_sequence(sc):
    n = 5
    for victim in range(n):
        sc.step([(sid, 1) for sid in range(n)])
        sc.remove(victim)
        sc.verify_cached_kv([s for s in range(n) if s != victim])
        # the reference test re-adds the sequence on the next round through apply_attention


def run_fork_sequence(sc):
    sc.step([(0, 60), (1, 88), (2, 17), (3, 4)])
    sc.step([((4, 3, -1), 35)])
    sc.step([((5, 0, -1), 20)])
    sc.step([((6, 5, -1), 102)])
    sc.step([((7, 0, -1), 3)])
    sc.step([((8, 5, -1), 71), ((9, 5, -1), 20)])
    for batch in [
        [(2, 1), (4, 1), (7, 1), (6, 1), (8, 1), (9, 1)],
        [(7, 1), (6, 1), (8, 1), (9, 1)],
        [(7, 1), (1, 1), (6, 1), (2, 1), (8, 1), (4, 1), (9, 1)],
        [(7, 10), (6, 2), (8, 3), (9, 4)],
    ]:
        sc.step(batch)
    sc.step([((10, 1, 33), 11)])
    sc.step([((11, 0, 60), 45), ((12, 0, 15), 14)])
    sc.step([((13, 0, 16), 19), ((14, 0, 17), 19)])
    sc.step([((15, 5, 60), 8), ((16, 5, 80), 10)])
    sc.step([((17, 5, 75), 11), ((18, 5, 76), 45), ((19, 5, 77), 14)])
    for batch in [
        [(6, 1), (11, 1), (13, 1), (9, 1)],
        [(10, 1), (16, 1), (18, 1), (19, 1)],
        [(8, 1), (15, 1), (17, 1), (12, 1), (14, 1)],
        [(10, 10), (6, 2), (8, 3), (19, 4)],
    ]:
        sc.step(batch)
    for i in range(20):
        sc.remove(i)
        sc.verify_cached_kv(list(range(i + 1, 20)))
    assert sc.cache.empty(), "The KV cache is not empty after removing all sequences"
    # fork after page recycle
    sc.step([(0, 7), (1, 24)])
    sc.step([((2, 1, -1), 10)])
    sc.step([((3, 0, -1), 20)])
    sc.step([(2, 1), (3, 1)])
    sc.step([(10, 7), (11, 24)])
    sc.step([((12, 11, -1), 200)])
    sc.step([(10, 1), (12, 1)])


def run_unlimited_depth(sc):
    sc.step([(0, 30)])
    for child, parent, n in [(1, 0, 15), (2, 1, 5), (3, 2, 20), (4, 3, 26), (5, 3, 18), (6, 5, 22),
                             (7, 5, 12), (8, 7, 29), (9, 7, 9), (10, 9, 31), (11, 9, 4)]:
        sc.step([((child, parent, -1), n)])
    for batch in [[(3, 1), (6, 1), (9, 1)], [(4, 1), (8, 1), (10, 1)], [(5, 1), (7, 1), (11, 1)]]:
        sc.step(batch)
    for i in range(12):
        sc.remove(i)
        sc.verify_cached_kv(list(range(i + 1, 12)))
    assert sc.cache.empty()


def run_popn(sc):
    sc.step([(0, 35), (1, 88), (2, 17), (3, 4)])
    sc.step([((4, 3, -1), 35)])
    for sid, n in [(0, 17), (1, 57), (2, 16), (3, 0), (4, 37)]:
        sc.popn(sid, n)
        sc.verify_cached_kv(list(range(4)))
    for sid in range(5):
        sc.remove(sid)
        sc.verify_cached_kv(list(range(sid + 1, 5)))
    assert sc.cache.empty()


def run_sliding_window(sc):
    """tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:912-955"""
    for sid, (window, sink) in enumerate(zip([20, 25, 30, 35, 40], [6, 4, 8, 3, 7])):
        sc.add_with_window(sid, window, sink)
    batches = [[(0, 4)], [(1, 6)], [(2, 6), (3, 7), (4, 7)]]
    batches += [[(0, 20), (1, 19), (2, 30), (3, 35), (4, 40)]]
    batches += [[(0, 6), (1, 5), (2, 4), (3, 3), (4, 2)]]
    batches += [[(i, 1) for i in range(5)]] * 20
    for batch in batches:
        sc.step(list(batch))


def run_sliding_window_fork(sc):
    """tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:958-1022"""
    for sid, (window, sink) in enumerate(zip([30, 35, 40], [15, 20, 25])):
        sc.add_with_window(sid, window, sink)
    sc.step([(0, 12), (1, 18), (2, 28)])
    sc.step([((3, 0, 10), 8), ((4, 1, -1), 20), ((5, 2, 18), 18)])
    sc.step([(0, 9), (1, 15), (2, 4), (3, 10), (4, 3), (5, 7)])
    sc.fork_with_window(3, 6, 18, 25, 24)
    sc.step([(3, 10), (6, 12)])


def run_sliding_window_page_reuse(sc):
    """Four sequences with a 40-token window and 4 sink tokens, six steps of 17 tokens each: from the
    third step on every sequence slides its window while the step's slots are reserved, the pages it
    frees go to the next sequence of the same batch, and that sequence's new tokens land on slots the
    step's page table of the first one still attends to.  Only a cache that writes the new rows after
    attention (src/runtime/vm/paged_kv_cache.cc:1396-1401) computes this batch correctly."""
    for sid in range(4):
        sc.add_with_window(sid, 40, 4)
    for _ in range(6):
        sc.step([(sid, 17) for sid in range(4)])


def run_tree_attn(sc):
    """test_paged_attention_kv_cache_tree_attn
    (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:1053-1134)."""
    from tests.util import REFERENCE_TREES
    prefill = [(0, 10), (1, 20), (2, 30), (3, 40)]
    tree_step = [(0, 7), (1, 15), (2, 10), (3, 14)]
    decode = [(0, 1), (1, 1), (2, 1), (3, 1)]
    # trees, one of them a chain; commit; plain decode
    sc.step(list(prefill))
    sc.step(list(tree_step), trees=[list(t) for t in REFERENCE_TREES], accepted=[6, 11, 6, 13])
    for _ in range(5):
        sc.step(list(decode))
    # every tree is a chain
    sc.cache.clear()
    sc.cached_k.clear()
    sc.cached_v.clear()
    sc.step(list(prefill))
    sc.step(list(tree_step), trees=[list(range(-1, n - 1)) for n in (7, 15, 10, 14)], accepted=[2, 6, -1, 4])
    for _ in range(5):
        sc.step(list(decode))
    # trees grown level by level over five steps against the cached tokens, committed at the end
    sc.cache.clear()
    sc.cached_k.clear()
    sc.cached_v.clear()
    sc.step(list(prefill))
    for i in range(5):
        leaves = 2 ** i
        parents = [(k - 1) // 2 for k in range(2 * leaves - 1)]
        sc.step([(sid, leaves) for sid in range(4)], trees=[list(parents) for _ in range(4)],
                accepted=None if i != 4 else [2, 6, -1, 4])
