"""Helpers of the GPU parity tests: tensors to the device and back, and an adapter that gives
the HIP-backed cache the method names the scenario driver and the oracle cache use."""
import numpy as np
import torch

import tvm_amd
from tvm_amd import get_global_func as gf

DEV = "cuda:0"


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def i32(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), dtype=torch.int32, device=DEV)


def host(t):
    return t.detach().cpu().numpy()


class GpuCache:
    """The library's cache behind the interface of oracle.paged_kv_cache.OraclePagedKVCache."""

    def __init__(self, cache_config, num_layers, hq, hkv, dqk, dv, attn_kinds=None, rope_mode=1, rope_scale=1.0,
                 rope_theta=1e4, rope_scaling=None, rope_ext_factors=None, dtype=np.float16):
        attn_kinds = list(attn_kinds) if attn_kinds is not None else [0] * num_layers
        ext = None if rope_ext_factors is None else dev(np.asarray(rope_ext_factors, dtype=np.float32))
        self.cache = gf("vm.builtin.paged_attention_kv_cache_create")(
            list(cache_config), [0, num_layers], hq, hkv, dqk, dv, attn_kinds, False, rope_mode, rope_scale,
            rope_theta, ext, torch.empty((), dtype=self._torch(dtype), device=DEV), rope_scaling=rope_scaling)
        self.num_layers, self.hq, self.hkv, self.dqk, self.dv = num_layers, hq, hkv, dqk, dv
        self.dtype = self._torch(dtype)

    @staticmethod
    def _torch(dtype):
        return torch.float32 if np.dtype(dtype) == np.float32 else torch.float16

    def clear(self):
        gf("vm.builtin.kv_state_clear")(self.cache)

    def add_sequence(self, sid):
        gf("vm.builtin.kv_state_add_sequence")(self.cache, sid)

    def remove_sequence(self, sid):
        gf("vm.builtin.kv_state_remove_sequence")(self.cache, sid)

    def fork_sequence(self, parent, child, pos=-1):
        gf("vm.builtin.kv_state_fork_sequence")(self.cache, parent, child, pos)

    def enable_sliding_window_for_seq(self, sid, window, sink):
        gf("vm.builtin.attention_kv_cache_enable_sliding_window_for_seq")(self.cache, sid, window, sink)

    def popn(self, sid, n):
        gf("vm.builtin.kv_state_popn")(self.cache, sid, n)

    def begin_forward(self, ids, lens, tree=None):
        gf("vm.builtin.kv_state_begin_forward")(self.cache, ids, lens, tree)

    def end_forward(self):
        gf("vm.builtin.kv_state_end_forward")(self.cache)

    def commit_accepted_token_tree_nodes(self, ids, leaf_indices):
        gf("vm.builtin.attention_kv_cache_commit_accepted_token_tree_nodes")(self.cache, ids, leaf_indices)

    def empty(self):
        return gf("vm.builtin.attention_kv_cache_empty")(self.cache)

    def attention_with_fused_qkv(self, layer, sm_scale, qkv, out):
        o = torch.zeros(out.shape, dtype=self.dtype, device=DEV)
        gf("vm.builtin.attention_kv_cache_attention_with_fused_qkv")(self.cache, layer, sm_scale, dev(qkv), o)
        out[...] = host(o)

    def attention_with_shared_kv(self, source_layer, sm_scale, q, current_k, current_v, out):
        o = torch.zeros(out.shape, dtype=self.dtype, device=DEV)
        gf("vm.builtin.attention_kv_cache_attention_with_shared_kv")(self.cache, source_layer, sm_scale, dev(q),
                                                                     dev(current_k), dev(current_v), o)
        out[...] = host(o)

    def self_attention(self, layer, sm_scale, q, k, v, out, lse):
        o = torch.zeros(out.shape, dtype=self.dtype, device=DEV)
        s = torch.zeros(lse.shape, dtype=torch.float32, device=DEV)
        gf("vm.builtin.attention_kv_cache_self_attention")(self.cache, layer, sm_scale, dev(q), dev(k), dev(v), o, s)
        out[...] = host(o)
        lse[...] = host(s)

    def cross_attention(self, layer, sm_scale, q, out, lse):
        o = torch.zeros(out.shape, dtype=self.dtype, device=DEV)
        s = torch.zeros(lse.shape, dtype=torch.float32, device=DEV)
        gf("vm.builtin.attention_kv_cache_cross_attention")(self.cache, layer, sm_scale, dev(q), o, s)
        out[...] = host(o)
        lse[...] = host(s)

    def append_mla_kv(self, layer, kv):
        gf("vm.builtin.attention_kv_cache_append_mla_kv")(self.cache, layer, dev(kv))

    def merge_attn_output_inplace(self, o_self, lse_self, o_cross, lse_cross):
        a, b = dev(o_self), dev(lse_self)
        gf("vm.builtin.attention_kv_cache_merge_attn_output_inplace")(self.cache, a, b, dev(o_cross), dev(lse_cross))
        o_self[...] = host(a)
        lse_self[...] = host(b)
        return o_self, lse_self

    def debug_get_kv(self, sid, start, end, k, v):
        kd = torch.zeros(k.shape, dtype=self.dtype, device=DEV)
        vd = torch.zeros(v.shape, dtype=self.dtype, device=DEV)
        gf("vm.builtin.attention_kv_cache_debug_get_kv")(self.cache, sid, start, end, kd, vd)
        k[...] = host(kd)
        v[...] = host(vd)

    def debug_get_kv_mla(self, sid, start, end, kv):
        kd = torch.zeros(kv.shape, dtype=self.dtype, device=DEV)
        gf("vm.builtin.attention_kv_cache_debug_get_kv_mla")(self.cache, sid, start, end, kd)
        kv[...] = host(kd)
