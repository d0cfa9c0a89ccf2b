"""CPU stand-in for the reference's whole cache object: host bookkeeping + llvm-target kernels.

TEST INFRASTRUCTURE ONLY.  ``OraclePagedKVCache`` wires ``oracle.host_cache.HostCache`` (the
integer state machine) to ``oracle.kernels`` (the C restatement of the CPU kernels) in the
order the reference's cache object calls them:

  attention_with_fused_qkv   src/runtime/vm/paged_kv_cache.cc:1303-1402
  self_attention             src/runtime/vm/paged_kv_cache.cc:1404-1445
  cross_attention            src/runtime/vm/paged_kv_cache.cc:1447-1485
  attention_with_shared_kv   src/runtime/vm/paged_kv_cache.cc:1487-1525
  append_mla_kv              src/runtime/vm/paged_kv_cache.cc:1527-1551
  merge_attn_output_inplace  src/runtime/vm/paged_kv_cache.cc:1553-1559
  debug_get_kv(_mla)         src/runtime/vm/paged_kv_cache.cc:1669-1766
  AttentionInternal / MHASelfAttnInternal / MHACrossAttnInternal / MLACrossAttnInternal
                             src/runtime/vm/paged_kv_cache.cc:2161-2335
  fork page copy             src/runtime/vm/paged_kv_cache.cc:721-734
  commit of token-tree nodes src/runtime/vm/paged_kv_cache.cc:1566-1659, :736-770

Arrays are numpy (fp16 data, int32 indices, fp32 lse).  Parity tests run the same seeded call
sequence through this object and through the HIP-backed cache and compare outputs, cached
K/V and every auxiliary array.
"""
import numpy as np

from . import host_cache as hc
from . import kernels as ok


class OraclePagedKVCache:
    def __init__(self, cache_config, num_layers, num_qo_heads, num_kv_heads, qk_head_dim, v_head_dim,
                 attn_kinds=None, rope_mode=hc.ROPE_NORMAL, rope_scale=1.0, rope_theta=1e4,
                 dtype=np.float16, rope_scaling=None, rope_ext_factors=None):
        attn_kinds = list(attn_kinds) if attn_kinds is not None else [hc.ATTN_MHA] * num_layers
        self.host = hc.HostCache(cache_config, attn_kinds, rope_mode)
        self.num_layers = num_layers
        self.hq, self.hkv = num_qo_heads, num_kv_heads
        self.dqk, self.dv = qk_head_dim, v_head_dim
        self.attn_kinds = attn_kinds
        self.rope_mode = self.host.rope_mode
        self.rope_scale, self.rope_theta = rope_scale, rope_theta
        # the frequency variant the reference bakes into its split-rotary kernel (position_embedding.py:258-299)
        self.rope_scaling, self.rope_ext_factors = rope_scaling, rope_ext_factors
        self.dtype = dtype
        ps, npages = self.host.page_size, self.host.num_total_pages
        self.pages = []
        for kind in attn_kinds:
            if kind in (hc.ATTN_MHA, hc.ATTN_MHA_SLIDING):
                self.pages.append(np.zeros((npages, 2, num_kv_heads, ps, qk_head_dim), dtype))
            elif kind == hc.ATTN_MLA:
                self.pages.append(np.zeros((npages, ps, qk_head_dim), dtype))
            else:
                raise hc.CacheError("unsupported attention kind")
        self._copies_done = 0

    # ---- state verbs -------------------------------------------------------------
    def clear(self):
        self.host.clear()
        self._copies_done = 0

    def add_sequence(self, seq_id):
        self.host.add_sequence(seq_id)

    def remove_sequence(self, seq_id):
        self.host.remove_sequence(seq_id)

    def _flush_copies(self):
        for src, tgt, n in self.host.copies[self._copies_done:]:
            for layer, kind in enumerate(self.attn_kinds):
                if kind == hc.ATTN_MLA:
                    ok.copy_single_page_mla(self.pages[layer], src, tgt, n)
                else:
                    ok.copy_single_page(self.pages[layer], src, tgt, n)
        self._copies_done = len(self.host.copies)

    def fork_sequence(self, parent, child, fork_pos=-1):
        self.host.fork_sequence(parent, child, fork_pos)
        self._flush_copies()

    def popn(self, seq_id, n):
        self.host.popn(seq_id, n)
        self._flush_copies()

    def commit_accepted_token_tree_nodes(self, seq_ids, leaf_indices):
        """CommitAcceptedTokenTreeNodes + CompactKVCopy (paged_kv_cache.cc:1566-1659, :736-770)."""
        batch = len(self.host.cur_seq_ids)
        copies = self.host.commit_accepted_token_tree_nodes(seq_ids, leaf_indices)
        if copies is not None and copies[0][-1] > 0:
            indptr, src, dst = copies
            for layer in range(self.num_layers):
                ok.compact_kv_copy(self.pages[layer], indptr, np.array([src, dst], np.int32), batch)
        self._flush_copies()

    def enable_sliding_window_for_seq(self, seq_id, window, sink):
        self.host.enable_sliding_window_for_seq(seq_id, window, sink)

    def begin_forward(self, seq_ids, append_lengths, token_tree_parent_ptr=None):
        return self.host.begin_forward(seq_ids, append_lengths, token_tree_parent_ptr)

    def end_forward(self):
        self.host.end_forward()

    def empty(self):
        return self.host.empty()

    def get_num_available_pages(self):
        return self.host.get_num_available_pages()

    def get_total_sequence_length(self):
        return self.host.get_total_sequence_length()

    def get_query_positions(self):
        return np.array(self.host.aux["q_rope_position_map"], np.int32)

    # ---- attention ---------------------------------------------------------------
    def _i32(self, x):
        return np.ascontiguousarray(x, dtype=np.int32)

    def _length_info(self, d):
        aux = self.host.aux
        if not self.host.support_sliding_window:
            return self._i32(aux["last_page_len"][d])
        return self._i32([aux["last_page_len"][d], aux["sliding_window_offset"][d], aux["sink_size"][d]])

    def _self_attn(self, q, k, v, out, lse, sm_scale, rope_mode):
        aux = self.host.aux
        indptr = self._i32(aux["cur_append_lengths_indptr"])
        if not self.host.is_chain_on_depths[0]:
            # the batch forms token trees (paged_kv_cache.cc:2192-2202)
            mask = self._i32(aux["tree_attn_mask"][0]).reshape(-1, 2)
            ok.tree_attn_ragged(q, indptr, k, v, indptr, self._i32(aux["q_rope_position_map"]),
                                self._i32(aux["tree_attn_mn_indptr"][0]), mask, out, lse,
                                int(rope_mode == hc.ROPE_INLINE), self.rope_scale, self.rope_theta, sm_scale)
            return
        ok.prefill_ragged(q, indptr, k, v, indptr, self._i32(aux["q_rope_position_map"]),
                          self._i32(aux["k_ragged_rope_pos_offset"]), out, lse, 1,
                          int(rope_mode == hc.ROPE_INLINE), self.rope_scale, self.rope_theta, sm_scale)

    def _mha_cross_attn(self, layer, q, out, lse, sm_scale, is_first_kernel, causal):
        aux, host = self.host.aux, self.host
        sliding_layer = self.attn_kinds[layer] == hc.ATTN_MHA_SLIDING
        computed = False
        total = q.shape[0]
        temp_out = np.zeros((total, self.hq, self.dv), self.dtype)
        temp_lse = np.zeros((total, self.hq), np.float32)
        for d in range(host.num_depths):
            if len(aux["page_indices"][d]) == 0:
                continue
            o, s = (out, lse) if is_first_kernel else (temp_out, temp_lse)
            if sliding_layer:
                page_indptr = aux["page_indptr_sliding_window"][d]
                page_indices = aux["page_indices_sliding_window"][d]
                length_info = self._i32([aux["last_page_len"][d], aux["sliding_window_offset"][d], aux["sink_size"][d]])
                k_rope_pos = aux["k_rope_pos_offset_sliding_window"][d]
                theta, scale = 10000.0, 1.0
            else:
                page_indptr, page_indices = aux["page_indptr"][d], aux["page_indices"][d]
                length_info = self._length_info(d)
                k_rope_pos = aux["k_rope_pos_offset"][d]
                theta, scale = self.rope_theta, self.rope_scale
            rotary = int(self.rope_mode == hc.ROPE_INLINE)
            if host.append_before_attn and not host.is_chain_on_depths[d]:
                # paged_kv_cache.cc:2266-2272
                mask = self._i32(aux["tree_attn_mask"][d]).reshape(-1, 2)
                ok.tree_attn_paged(q, aux["qo_indptr"][d], self.pages[layer], page_indptr, page_indices,
                                   length_info, k_rope_pos, aux["q_rope_position_map"], o, s, rotary, scale,
                                   theta, sm_scale, aux["tree_attn_mn_indptr"][d], mask)
            elif host.use_decode_kernel[d]:
                ok.decode(q, self.pages[layer], page_indptr, page_indices, length_info, k_rope_pos,
                          aux["q_rope_position_map"], o, s, rotary, scale, theta, sm_scale)
            else:
                ok.prefill_paged(q, aux["qo_indptr"][d], self.pages[layer], page_indptr, page_indices,
                                 length_info, k_rope_pos, aux["q_rope_position_map"], o, s, int(causal),
                                 rotary, scale, theta, sm_scale,
                                 sliding_window_size=host.layer_sliding_window_size)
            if not is_first_kernel:
                ok.merge_state_inplace(out, lse, temp_out, temp_lse)
            else:
                is_first_kernel = False
            computed = True
        return computed

    def _attention_internal(self, layer, q, k, v, out, sm_scale):
        host = self.host
        total = q.shape[0]
        merged_lse = np.zeros((total, self.hq), np.float32)
        is_first_kernel = True
        if not host.append_before_attn:
            is_first_kernel = False
            self._self_attn(q, k, v, out, merged_lse, sm_scale, self.rope_mode)
        self_done = not is_first_kernel
        causal = (not host.append_before_attn) and self.attn_kinds[layer] == hc.ATTN_MHA_SLIDING
        cross_done = self._mha_cross_attn(layer, q, out, merged_lse, sm_scale, is_first_kernel, causal)
        if not (self_done or cross_done):
            raise hc.CacheError("Both self-attention and cross-attention are not computed.")

    def attention_with_fused_qkv(self, layer_id, sm_scale, qkv, out):
        host = self.host
        if self.attn_kinds[layer_id] not in (hc.ATTN_MHA, hc.ATTN_MHA_SLIDING):
            raise hc.CacheError("layer is not MHA")
        total = sum(host.cur_append_lengths)
        if total > qkv.shape[0]:
            raise hc.CacheError("qkv has fewer rows than the batch appends")
        aux = host.aux
        qkv_view = np.ascontiguousarray(qkv[:total])
        q = np.zeros((total, self.hq, self.dqk), self.dtype)
        k = np.zeros((total, self.hkv, self.dqk), self.dtype)
        v = np.zeros((total, self.hkv, self.dqk), self.dtype)
        if self.rope_scaling:
            # the longrope kernel has no apply_rope argument and always rotates (position_embedding.py:582-667)
            apply = 1 if self.rope_ext_factors is not None else int(self.rope_mode == hc.ROPE_NORMAL)
            ok.fused_rope_scaled(qkv_view, aux["q_rope_position_map"], q, k, v, apply, self.rope_scaling,
                                 theta=self.rope_theta, scale=self.rope_scale, ext_factors=self.rope_ext_factors)
        else:
            ok.fused_rope(qkv_view, aux["q_rope_position_map"], q, k, v, int(self.rope_mode == hc.ROPE_NORMAL),
                          theta=self.rope_theta, scale=self.rope_scale)
        if host.append_before_attn:
            ok.transpose_append(self.pages[layer_id], k, v, aux["append_position_map"])
        o_view = np.zeros((total, self.hq, self.dqk), self.dtype)
        with self._inline_rope():
            self._attention_internal(layer_id, q, k, v, o_view, sm_scale)
        out[:total] = o_view
        if not host.append_before_attn:
            ok.transpose_append(self.pages[layer_id], k, v, aux["append_position_map"])

    def attention_with_shared_kv(self, source_layer_id, sm_scale, q, current_k, current_v, out):
        if self.attn_kinds[source_layer_id] not in (hc.ATTN_MHA, hc.ATTN_MHA_SLIDING):
            raise hc.CacheError("Querying K/V from another logical layer is only supported for MHA caches.")
        total = sum(self.host.cur_append_lengths)
        if not (q.shape[0] == current_k.shape[0] == current_v.shape[0] == out.shape[0] == total):
            raise hc.CacheError("attention_with_shared_kv: row counts do not match the batch")
        with self._inline_rope():
            self._attention_internal(source_layer_id, q, current_k, current_v, out, sm_scale)

    def _inline_rope(self):
        """The frequency variant the reference bakes into its attention kernels (kv_cache.py:494-497, :680-682):
        in force while a cache that rotates inside the attention kernels runs them."""
        return ok.inline_rope_scaling(self.rope_scaling if self.rope_mode == hc.ROPE_INLINE else None)

    def self_attention(self, layer_id, sm_scale, q, k, v, out, lse):
        with self._inline_rope():
            if self.attn_kinds[layer_id] == hc.ATTN_MHA:
                self._self_attn(q, k, v, out, lse, sm_scale, self.rope_mode)
            else:
                self._self_attn(q, k, v, out, lse, sm_scale, hc.ROPE_NONE)

    def cross_attention(self, layer_id, sm_scale, q, out, lse):
        host, aux = self.host, self.host.aux
        if self.attn_kinds[layer_id] == hc.ATTN_MHA:
            with self._inline_rope():
                self._mha_cross_attn(layer_id, q, out, lse, sm_scale, True, False)
            return
        total = q.shape[0]
        temp_out = np.zeros((total, self.hq, self.dv), self.dtype)
        temp_lse = np.zeros((total, self.hq), np.float32)
        is_first_kernel = True
        for d in range(host.num_depths):
            if len(aux["page_indices"][d]) == 0:
                continue
            o, s = (out, lse) if is_first_kernel else (temp_out, temp_lse)
            ok.prefill_paged_mla(q, aux["qo_indptr"][d], self.pages[layer_id], aux["page_indptr"][d],
                                 aux["page_indices"][d], self._length_info(d), o, s, 0, sm_scale,
                                 d_latent=self.dv)
            if not is_first_kernel:
                ok.merge_state_inplace(out, lse, temp_out, temp_lse)
            else:
                is_first_kernel = False

    def append_mla_kv(self, layer_id, kv):
        if self.attn_kinds[layer_id] != hc.ATTN_MLA:
            raise hc.CacheError("layer is not MLA")
        ok.transpose_append_mla(self.pages[layer_id], kv, self.host.aux["append_position_map"])

    def merge_attn_output_inplace(self, o_self, lse_self, o_cross, lse_cross):
        ok.merge_state_inplace(o_self, lse_self, o_cross, lse_cross)
        return o_self, lse_self

    # ---- debug -------------------------------------------------------------------
    def debug_get_kv(self, seq_id, start_pos, end_pos, k_data, v_data):
        pm = self.host.position_map_of(seq_id)[start_pos:end_pos]
        for layer in range(self.num_layers):
            ok.debug_get_kv(self.pages[layer], pm, k_data, v_data, layer)

    def debug_get_kv_mla(self, seq_id, start_pos, end_pos, kv_data):
        pm = self.host.position_map_of(seq_id)[start_pos:end_pos]
        for layer in range(self.num_layers):
            ok.debug_get_kv_mla(self.pages[layer], pm, kv_data, layer)
