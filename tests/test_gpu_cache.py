"""GPU parity of the whole cache object: the reference's scenario batches through the
HIP-backed cache, checked (a) against the numpy closed form the reference's own test uses,
(b) against the CPU oracle cache on identical seeded inputs, with page tables / append
indices / pool state compared bit for bit."""
import numpy as np
import pytest
import torch

import tvm_amd
from oracle.paged_kv_cache import OraclePagedKVCache
from tests import scenario as S
from tests.gpu_util import DEV, GpuCache, dev, host
from tests.test_host_cache_parity import GLOBAL, PER_DEPTH
from tests.util import assert_close
from tvm_amd import get_global_func as gf

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("d,rope_mode", [(128, S.ROPE_NORMAL), (64, S.ROPE_NORMAL), (128, S.ROPE_NONE), (256, S.ROPE_NORMAL)])
@pytest.mark.parametrize("runner", [S.run_prefill_and_decode, S.run_remove_sequence, S.run_fork_sequence,
                                    S.run_unlimited_depth, S.run_popn])
def test_reference_scenarios_on_the_gpu(runner, d, rope_mode):
    """tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:706-909 of the
    reference with its geometry (32 query / 4 kv heads, page 16, capacity 2048)."""
    layers, hq, hkv = 2, 32, 4
    cache = GpuCache([32, 2048, 512, 16, 0], layers, hq, hkv, d, d, rope_mode=rope_mode)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=rope_mode, seed=5, tol=4e-3)
    runner(sc)


class Mirror:
    """Feeds the oracle cache and the GPU cache the same calls and the same tensors."""

    def __init__(self, cache_config, layers, hq, hkv, d, rope_mode=1, dtype=np.float16, **rope):
        self.o = OraclePagedKVCache(cache_config, layers, hq, hkv, d, d, rope_mode=rope_mode, dtype=dtype, **rope)
        self.g = GpuCache(cache_config, layers, hq, hkv, d, d, rope_mode=rope_mode, dtype=dtype, **rope)
        self.layers, self.hq, self.hkv, self.d = layers, hq, hkv, d
        self.dtype = dtype
        # float32 storage: what is left is the order of the float32 sums and the device's exp2 / sin / cos
        self.tol = dict(atol=2e-4, rtol=2e-4) if dtype == np.float32 else {}
        self.rng = np.random.default_rng(21)
        self.lengths = {}

    def compare_bookkeeping(self):
        aux = self.o.host.aux
        c = self.g.cache
        flags = c.flags()
        assert flags["num_depths"] == aux["num_depths"]
        assert bool(flags["append_before_attn"]) == aux["append_before_attn"]
        for dd in range(aux["num_depths"]):
            for name in PER_DEPTH:
                assert c.aux(name, dd) == aux[name][dd], f"{name}[{dd}]"
        for name in GLOBAL:
            assert c.aux(name) == aux[name], name
        so, sg = self.o.host.state(), c.state()
        assert sg["free_page_ids"] == so["free_page_ids"] and sg["free_block_idx"] == so["free_block_idx"]
        assert [tuple(b) for b in sg["blocks"]] == [tuple(b) for b in so["blocks"]] and sg["seqs"] == so["seqs"]
        assert c.copy_log() == self.o.host.copies

    def step(self, batch):
        ids, lens = [], []
        for item, n in batch:
            if isinstance(item, tuple):
                sid, parent, pos = item
                self.o.fork_sequence(parent, sid, pos)
                self.g.fork_sequence(parent, sid, pos)
                self.lengths[sid] = self.lengths[parent] if pos == -1 else pos
            else:
                sid = item
                if sid not in self.lengths:
                    self.o.add_sequence(sid)
                    self.g.add_sequence(sid)
                    self.lengths[sid] = 0
            ids.append(sid)
            lens.append(n)
        self.o.begin_forward(ids, lens)
        self.g.begin_forward(ids, lens)
        self.compare_bookkeeping()
        total = sum(lens)
        for layer in range(self.layers):
            qkv = self.rng.standard_normal((total, self.hq + 2 * self.hkv, self.d)).astype(self.dtype)
            eo = np.zeros((total, self.hq, self.d), self.dtype)
            go = np.zeros_like(eo)
            self.o.attention_with_fused_qkv(layer, self.d ** -0.5, qkv, eo)
            self.g.attention_with_fused_qkv(layer, self.d ** -0.5, qkv, go)
            assert_close(go, eo, what=f"layer {layer} output vs oracle cache", **self.tol)
        self.o.end_forward()
        self.g.end_forward()
        for sid, n in zip(ids, lens):
            self.lengths[sid] += n
            L = self.lengths[sid]
            ek = np.zeros((self.layers, L, self.hkv, self.d), self.dtype)
            ev, gk, gv = np.zeros_like(ek), np.zeros_like(ek), np.zeros_like(ek)
            self.o.debug_get_kv(sid, 0, L, ek, ev)
            self.g.debug_get_kv(sid, 0, L, gk, gv)
            assert np.array_equal(gv, ev), f"cached V of seq {sid}"
            assert_close(gk, ek, atol=1e-3, rtol=2e-3, what=f"cached K of seq {sid}")


@pytest.mark.parametrize("page_size,hq,hkv,d", [(16, 32, 8, 128), (32, 32, 8, 128), (64, 32, 8, 128), (16, 8, 2, 96),
                                                (32, 12, 4, 80), (16, 4, 4, 112)])
def test_identical_inputs_through_oracle_and_gpu_caches(page_size, hq, hkv, d):
    m = Mirror([16, 4096, 1024, page_size, 0], 2, hq, hkv, d)
    m.step([(0, 60), (1, 88), (2, 17), (3, 4)])
    m.step([((4, 3, -1), 35)])
    m.step([((5, 0, 33), 20)])            # fork inside a page -> page copy on the device
    m.step([(0, 1), (1, 1), (2, 1), (4, 1), (5, 1)])
    m.step([((6, 5, -1), 40), (2, 3)])
    m.step([(6, 1), (5, 1), (0, 1)])      # two block depths + merge_state
    m.o.popn(6, 30)
    m.g.popn(6, 30)
    m.lengths[6] -= 30
    m.step([(6, 1), (1, 200)])
    m.step([(i, 1) for i in (0, 1, 2, 4, 5, 6)])


@pytest.mark.parametrize("dtype,page_size,hq,hkv,d", [(np.float32, 16, 8, 2, 128), (np.float32, 16, 32, 4, 64),
                                                      (np.float16, 24, 8, 2, 128), (np.float16, 5, 8, 2, 64),
                                                      (np.float32, 12, 6, 2, 72), (np.float16, 16, 8, 2, 72),
                                                      (np.float16, 48, 20, 1, 128)])
def test_float32_storage_other_page_sizes_and_head_dims_through_both_caches(dtype, page_size, hq, hkv, d):
    """What the reference's kernel factories accept beside the tuned shapes (its tests run float32 storage,
    test_runtime_builtin_paged_attention_kv_cache_cpu.py:269-276; page size and head dim are free parameters of
    every factory): the cache runs these on the generic matrix-core kernels.  Same calls and tensors through the
    oracle cache (the oracle's float32 build for float32 storage), page tables and pool state bit for bit."""
    m = Mirror([16, 2048, 512, page_size, 0], 2, hq, hkv, d, dtype=dtype)
    m.step([(0, 60), (1, 88), (2, 17), (3, 4)])
    m.step([((4, 3, -1), 35)])
    m.step([((5, 0, 33), 20)])            # fork inside a page -> page copy on the device
    m.step([(0, 1), (1, 1), (2, 1), (4, 1), (5, 1)])
    m.step([((6, 5, -1), 40), (2, 3)])
    m.step([(6, 1), (5, 1), (0, 1)])      # two block depths + merge_state
    m.o.popn(6, 30)
    m.g.popn(6, 30)
    m.lengths[6] -= 30
    m.step([(6, 1), (1, 200)])
    m.step([(i, 1) for i in (0, 1, 2, 4, 5, 6)])


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("runner", [S.run_prefill_and_decode, S.run_remove_sequence, S.run_fork_sequence,
                                    S.run_unlimited_depth, S.run_popn])
def test_reference_scenarios_float32_storage(runner, d):
    """The float32 rows of the reference's fixture (head dims 64 and 128, RopeMode.NORMAL,
    test_runtime_builtin_paged_attention_kv_cache_cpu.py:269-276) with its geometry, against the numpy closed form."""
    layers, hq, hkv = 2, 32, 4
    cache = GpuCache([32, 2048, 512, 16, 0], layers, hq, hkv, d, d, rope_mode=S.ROPE_NORMAL, dtype=np.float32)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=S.ROPE_NORMAL, seed=5, tol=1e-3, dtype=np.float32)
    runner(sc)


def test_storage_type_of_the_tensors_is_checked():
    cache = GpuCache([4, 64, 32, 16, 0], 1, 8, 2, 128, 128, dtype=np.float32)
    cache.add_sequence(0)
    cache.begin_forward([0], [2])
    qkv = torch.zeros((2, 12, 128), dtype=torch.float16, device=DEV)
    out = torch.zeros((2, 8, 128), dtype=torch.float16, device=DEV)
    with pytest.raises(tvm_amd.KVError, match="stores float32"):
        gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")(cache.cache, 0, 1.0, qkv, out)


@pytest.mark.parametrize("dtype,page_size,d,tol", [(np.float16, 16, 96, 4e-3), (np.float32, 16, 128, 1e-3),
                                                   (np.float16, 24, 128, 4e-3), (np.float32, 12, 72, 1e-3)])
@pytest.mark.parametrize("runner", [S.run_sliding_window, S.run_sliding_window_fork, S.run_sliding_window_page_reuse])
def test_sliding_window_scenarios_on_the_generic_kernels(runner, dtype, page_size, d, tol):
    """The reference's sliding-window scenarios (attention sinks, window trimming, forks inside the sink, page reuse;
    test_runtime_builtin_paged_attention_kv_cache_cpu.py:912-1022) on caches that the tuned extended kernels do not
    serve: head dim 96, float32 storage, pages of 24 and 12 tokens.  Such a cache rotates inside the attention
    kernels and hands them the (3, batch) length_info."""
    layers, hq, hkv = 2, 8, 2
    cache = GpuCache([32, 2048, 512, page_size, 1], layers, hq, hkv, d, d, rope_mode=S.ROPE_INLINE, dtype=dtype)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=S.ROPE_INLINE, seed=4, tol=tol, dtype=dtype)
    runner(sc)


@pytest.mark.parametrize("dtype,page_size,d", [(np.float16, 16, 80), (np.float32, 16, 64), (np.float16, 40, 128)])
@pytest.mark.parametrize("sliding", [0, 1])
def test_inline_rope_and_forks_on_the_generic_kernels(dtype, page_size, d, sliding):
    """Caches that rotate inside the attention kernels (rope mode 2, with and without sliding-window support) at a
    head dim, a storage type and a page size of the generic kernels, with a frequency variant: prefill (ragged +
    paged + merge), decode, a fork with two block depths, against the oracle cache."""
    rope = dict(rope_theta=5e5, rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                              "high_freq_factor": 4.0, "original_max_position_embeddings": 64})
    m = Mirror([8, 2048, 512, page_size, sliding], 2, 8, 2, d, rope_mode=2, dtype=dtype, **rope)
    m.step([(0, 60), (1, 88), (2, 17)])
    m.step([(0, 1), (1, 1), (2, 1)])
    m.step([((3, 1, 40), 25), (0, 2)])
    m.step([(3, 1), (1, 1)])


def test_short_chunk_against_a_long_cached_sequence():
    """A chunk of a few tokens against thousands of cached ones is one or two row tiles per kv head: the
    launch splits their keys over several workgroups and merges the states.  Through the cache's one-pass
    chunked prefill and its mixed prefill / decode batches, against the oracle cache."""
    m = Mirror([4, 8192, 2048, 16, 0], 2, 8, 2, 64)
    m.step([(0, 2000), (1, 40)])
    m.step([(0, 1500)])
    m.step([(0, 20), (1, 3)])       # 3520 cached tokens, 20 new ones
    m.step([(0, 1), (1, 2)])        # not a pure decode batch: the prefill kernels again
    m.step([((2, 0, 3000), 7)])     # a fork deep inside the long sequence


@pytest.mark.parametrize("rope", [
    dict(rope_theta=5e5, rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                       "original_max_position_embeddings": 8192}),
    dict(rope_scaling={"rope_type": "yarn", "factor": 40.0, "beta_fast": 32, "beta_slow": 1,
                       "original_max_position_embeddings": 4096}),
    dict(rope_scaling={"rope_type": "default", "rotary_dim": 32}),
    dict(rope_scaling={"rope_type": "gptj", "rotary_dim": 64}),
    dict(rope_scaling={"rope_type": "longrope", "max_position_embeddings": 131072, "original_max_position_embeddings": 64},
         rope_ext_factors=np.concatenate([np.linspace(1.0, 8.0, 64), np.linspace(1.0, 1.3, 64)]).astype(np.float32)),
])
def test_rope_frequency_variants_through_the_cache(rope):
    """The model's RoPE variant (what the reference compiles into the split-rotary kernel it hands to the
    cache): prefill, decode and a fork, cached K compared with the oracle cache that rotates the same way.
    The longrope steps have fewer and more rows than original_max_position_embeddings (short / long factors)."""
    m = Mirror([8, 2048, 512, 16, 0], 1, 32, 8, 128, **rope)
    m.step([(0, 60), (1, 88), (2, 17)])   # 165 rows
    m.step([(0, 1), (1, 1), (2, 1)])      # 3 rows
    m.step([((3, 1, 40), 25), (0, 2)])


@pytest.mark.parametrize("rope", [
    dict(rope_theta=5e5, rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                       "original_max_position_embeddings": 8192}),
    dict(rope_scaling={"rope_type": "yarn", "factor": 40.0, "beta_fast": 32, "beta_slow": 1,
                       "original_max_position_embeddings": 4096}),
    dict(rope_scaling={"rope_type": "longrope", "max_position_embeddings": 131072, "original_max_position_embeddings": 4096}),
    dict(rope_scaling={"rope_type": "llama4", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                       "original_max_position_embeddings": 8192}),
], ids=lambda r: r["rope_scaling"]["rope_type"])
@pytest.mark.parametrize("sliding", [0, 1])
def test_rope_frequency_variants_in_a_cache_that_rotates_inside_the_attention_kernels(rope, sliding):
    """Inline-RoPE caches (rope mode 2; a sliding-window cache is always one): K is stored unrotated, and every
    attention kernel rotates q and k itself with the model's frequency variant -- prefill (ragged + paged +
    merge), decode and a fork with two block depths, against the oracle cache with the same variant in force."""
    m = Mirror([8, 2048, 512, 16, sliding], 1, 8, 2, 128, rope_mode=2, **rope)
    m.step([(0, 60), (1, 88), (2, 17)])
    m.step([(0, 1), (1, 1), (2, 1)])
    m.step([((3, 1, 40), 25), (0, 2)])
    m.step([(3, 1), (1, 1)])


def test_cfg1_decode_through_the_cache_verbs():
    """BASELINE configs[0] end to end: 1024-page pool, contexts 512/1024/1500/2048 prefilled through
    the real verbs, then one decode step; page table as derived by hand from the reference."""
    m = Mirror([32, 16368, 8192, 16, 0], 1, 32, 8, 128)
    m.step([(0, 512), (1, 1024), (2, 1500), (3, 2048)])
    m.step([(0, 1), (1, 1), (2, 1), (3, 1)])
    c = m.g.cache
    assert c.aux("page_indptr") == [0, 33, 98, 192, 321]
    assert c.aux("append_position_map") == [5088, 5104, 3036, 5120]
    assert c.aux("last_page_len") == [1, 1, 13, 1]
    assert c.aux("q_rope_position_map") == [512, 1024, 1500, 2048]
    assert gf("vm.builtin.attention_kv_cache_get_num_available_pages")(c) == 703


def test_error_paths_on_the_device_cache():
    cache = GpuCache([4, 64, 32, 16, 0], 1, 8, 2, 128, 128)
    c = cache.cache
    cache.add_sequence(0)
    qkv = torch.zeros((4, 12, 128), dtype=torch.float16, device=DEV)
    out = torch.zeros((4, 8, 128), dtype=torch.float16, device=DEV)
    attn = gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")
    with pytest.raises(tvm_amd.KVError, match="begin_forward has not been called"):
        attn(c, 0, 1.0, qkv, out)
    cache.begin_forward([0], [8])
    with pytest.raises(tvm_amd.KVError, match="fewer than the batch appends"):
        attn(c, 0, 1.0, qkv, out)
    with pytest.raises(tvm_amd.KVError, match="out of range"):
        attn(c, 3, 1.0, torch.zeros((8, 12, 128), dtype=torch.float16, device=DEV),
             torch.zeros((8, 8, 128), dtype=torch.float16, device=DEV))
    cache.add_sequence(1)
    with pytest.raises(tvm_amd.KVError, match="The KV cache is full"):
        cache.begin_forward([1], [80])
    # a kernel's refusal surfaces through the cache call: head_dim 68 is not built (the generic kernels take
    # multiples of 8)
    c2 = GpuCache([4, 64, 32, 16, 0], 1, 8, 2, 68, 68, rope_mode=0)
    c2.add_sequence(0)
    qkv96 = torch.zeros((1, 12, 68), dtype=torch.float16, device=DEV)
    out96 = torch.zeros((1, 8, 68), dtype=torch.float16, device=DEV)
    c2.begin_forward([0], [1])
    with pytest.raises(tvm_amd.KVError, match="is not built"):
        attn(c2.cache, 0, 1.0, qkv96, out96)


@pytest.mark.parametrize("runner", [S.run_sliding_window, S.run_sliding_window_fork, S.run_sliding_window_page_reuse])
def test_sliding_window_scenarios_on_the_gpu(runner):
    """The reference's sliding-window tests (attention sinks, window trimming after every step,
    forks inside the sink; tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:912-1022)
    on the HIP cache: inline RoPE, length_info (3, B), prefill and decode kernels."""
    layers, hq, hkv, d = 2, 8, 2, 128
    cache = GpuCache([32, 2048, 512, 16, 1], layers, hq, hkv, d, d, rope_mode=S.ROPE_INLINE)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=S.ROPE_INLINE, seed=4)
    runner(sc)


@pytest.mark.parametrize("d,rope_mode", [(128, S.ROPE_NORMAL), (64, S.ROPE_NORMAL), (128, S.ROPE_NONE)])
def test_token_tree_scenario_on_the_gpu(d, rope_mode):
    """test_paged_attention_kv_cache_tree_attn of the reference
    (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:1053-1134): tree attention
    over new tokens and over appended tree nodes, commit with the compaction copy, decode after it."""
    layers, hq, hkv = 2, 32, 4
    cache = GpuCache([32, 2048, 512, 16, 0], layers, hq, hkv, d, d, rope_mode=rope_mode)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=rope_mode, seed=8, tol=4e-3)
    S.run_tree_attn(sc)


def test_padded_qkv_rows_are_ignored():
    """qkv / out may carry more rows than the batch appends (src/runtime/vm/paged_kv_cache.cc:1330-1354)."""
    layers, hq, hkv, d = 1, 8, 2, 128
    a = GpuCache([4, 256, 64, 16, 0], layers, hq, hkv, d, d)
    b = GpuCache([4, 256, 64, 16, 0], layers, hq, hkv, d, d)
    rng = np.random.default_rng(3)
    qkv = rng.standard_normal((10, hq + 2 * hkv, d)).astype(np.float16)
    for cache in (a, b):
        cache.add_sequence(0)
        cache.begin_forward([0], [10])
    o_exact = np.zeros((10, hq, d), np.float16)
    a.attention_with_fused_qkv(0, d ** -0.5, qkv, o_exact)
    padded = np.concatenate([qkv, np.full((6, hq + 2 * hkv, d), np.nan, np.float16)])
    o_pad = np.full((16, hq, d), 3.0, np.float16)
    b.attention_with_fused_qkv(0, d ** -0.5, padded, o_pad)
    assert np.array_equal(o_pad[:10], o_exact)


def test_attention_with_shared_kv_reads_the_source_layer():
    """vm.builtin.attention_kv_cache_attention_with_shared_kv (src/runtime/vm/kv_state.cc:97-105,
    paged_kv_cache.cc:1487-1525): a second set of queries attends to the K/V that layer 0 caches plus
    the step's own rows, nothing is appended.  Prefill (self + cross), a second chunk, then decode;
    checked against the oracle cache and against the closed form over layer 0's K/V."""
    from oracle import closed_form as cf
    layers, hq, hkv, d = 2, 8, 2, 128
    cfg = [4, 512, 128, 16, 0]
    gpu = GpuCache(cfg, layers, hq, hkv, d, d, rope_mode=S.ROPE_NONE)
    cpu = OraclePagedKVCache(cfg, layers, hq, hkv, d, d, rope_mode=S.ROPE_NONE)
    rng = np.random.default_rng(17)
    cached_k = {0: np.zeros((0, hkv, d), np.float16), 1: np.zeros((0, hkv, d), np.float16)}
    cached_v = {0: np.zeros((0, hkv, d), np.float16), 1: np.zeros((0, hkv, d), np.float16)}
    for cache in (gpu, cpu):
        cache.add_sequence(0)
        cache.add_sequence(1)
    for lens in ([40, 23], [9, 30], [1, 1], [1, 1]):
        total = sum(lens)
        qkv = rng.standard_normal((total, hq + 2 * hkv, d)).astype(np.float16)
        q2 = rng.standard_normal((total, hq, d)).astype(np.float16)
        k_cur = np.ascontiguousarray(qkv[:, hq:hq + hkv])
        v_cur = np.ascontiguousarray(qkv[:, hq + hkv:])
        outs = []
        for cache in (gpu, cpu):
            cache.begin_forward([0, 1], lens)
            o1 = np.zeros((total, hq, d), np.float16)
            cache.attention_with_fused_qkv(0, d ** -0.5, qkv, o1)
            o2 = np.zeros((total, hq, d), np.float16)
            cache.attention_with_shared_kv(0, d ** -0.5, q2, k_cur, v_cur, o2)
            cache.end_forward()
            outs.append(o2)
        assert_close(outs[0], outs[1], what=f"shared-kv attention vs oracle cache, step {lens}")
        cursor = 0
        for sid, n in enumerate(lens):
            cached_k[sid] = np.concatenate([cached_k[sid], k_cur[cursor:cursor + n]])
            cached_v[sid] = np.concatenate([cached_v[sid], v_cur[cursor:cursor + n]])
            expected, _ = cf.attention(q2[cursor:cursor + n], cached_k[sid], cached_v[sid], d ** -0.5, causal=True)
            assert_close(outs[0][cursor:cursor + n], expected, atol=4e-3, rtol=4e-3,
                         what=f"shared-kv attention vs closed form, seq {sid}")
            cursor += n
    # layer 1 never received anything
    with pytest.raises(tvm_amd.KVError, match="rows"):
        gf("vm.builtin.attention_kv_cache_attention_with_shared_kv")(
            gpu.cache, 0, 1.0, torch.zeros((5, hq, d), dtype=torch.float16, device=DEV),
            torch.zeros((5, hkv, d), dtype=torch.float16, device=DEV),
            torch.zeros((5, hkv, d), dtype=torch.float16, device=DEV),
            torch.zeros((5, hq, d), dtype=torch.float16, device=DEV))


@pytest.mark.parametrize("runner,rope_mode,sliding", [(S.run_fork_sequence, S.ROPE_NORMAL, 0), (S.run_tree_attn, S.ROPE_NORMAL, 0),
                                                      (S.run_sliding_window_fork, S.ROPE_INLINE, 1),
                                                      (S.run_sliding_window_page_reuse, S.ROPE_INLINE, 1)])
def test_reference_scenarios_with_pages_of_32_tokens(runner, rope_mode, sliding):
    """The reference's scenarios on a cache whose pages hold 32 tokens (the kernels walk such pages as
    two runs of 16): forks inside a page, token trees with their commit, sliding windows."""
    layers, hq, hkv, d = 2, 8, 2, 128
    cache = GpuCache([32, 2048, 512, 32, sliding], layers, hq, hkv, d, d, rope_mode=rope_mode)
    sc = S.Scenario(cache, layers, hq, hkv, d, rope_mode=rope_mode, seed=9, tol=4e-3)
    runner(sc)
