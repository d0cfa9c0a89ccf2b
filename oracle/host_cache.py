"""Pure-Python restatement of the host-side state machine of the reference's paged KV cache.

TEST INFRASTRUCTURE ONLY -- the checker for the C++ host cache shipped in ``tvm_amd/csrc``.
It holds no tensors and launches nothing: it reproduces the integer bookkeeping (page pool,
block tree, sequences) and the auxiliary arrays that ``BeginForward`` hands to the kernels,
so that page tables, append indices and pool state can be compared bit for bit.

Follows, method by method:
  Block / Sequence             src/runtime/vm/attn_utils.h:101-230
  get_block_ids_on_depth       src/runtime/vm/attn_utils.h:243-279
  get_chunked_block_ids        src/runtime/vm/attn_utils.h:293-332
  clear / add / remove         src/runtime/vm/paged_kv_cache.cc:561-604
  fork_sequence                src/runtime/vm/paged_kv_cache.cc:606-719
  enable_sliding_window_for_seq src/runtime/vm/paged_kv_cache.cc:772-801
  popn                         src/runtime/vm/paged_kv_cache.cc:803-862
  begin_forward                src/runtime/vm/paged_kv_cache.cc:884-1212
  commit_accepted_token_tree_nodes src/runtime/vm/paged_kv_cache.cc:1566-1659
  construct_token_tree_mask    src/runtime/vm/paged_kv_cache.cc:1800-1928
  slide_window_for_sequence    src/runtime/vm/paged_kv_cache.cc:1935-1992
  reserve_append_length_in_seq src/runtime/vm/paged_kv_cache.cc:2004-2044
  num_total_pages              src/runtime/vm/paged_kv_cache.cc:2606-2619

Pinned by tests/test_host_cache_oracle.py: the hand-derived examples (fork inside a page, at a
page-aligned end, at an interior page boundary, popn, the cfg-1 decode step), the closed form
for fork-free runs (pages are handed out 0,1,2,... in BeginForward order) and structural
invariants (every page in exactly one place, block lengths sum to the sequence length,
reference counts equal children + ending sequences, Empty() after removing everything).
PARITY UNPINNED for what those leave open: no run of the real runtime library is possible in
this build (its FFI dependency is not vendored), so BeginForward's per-depth arrays under
forks deeper than two levels and PopN into shared prefixes are pinned by invariants and
K/V round trips only.
"""
import math

MAX_BLOCK_DEPTH = 2  # kPagedKVCacheMaxBlockDepth, attn_utils.h:50
TREE_MAX_SIZE = 256  # kTreeAttnMaxTreeSize, attn_utils.h:52
TEMP_PAGE_ID = -1  # kPagedKVCacheTempPageId, attn_utils.h:58

ATTN_MHA, ATTN_MLA, ATTN_LINEAR, ATTN_MHA_SLIDING = 0, 1, 2, 3
ROPE_NONE, ROPE_NORMAL, ROPE_INLINE = 0, 1, 2


class CacheError(RuntimeError):
    """Stands in for the reference's ffi::Error raised by a failed ICHECK."""


def _check(cond, msg):
    if not cond:
        raise CacheError(msg)


class Block:
    def __init__(self, index):
        self.index = index
        self.reset()

    def reset(self):
        self.page_ids = []
        self.seq_length = 0
        self.start_pos = 0
        self.sink_length = 0
        self.sliding_window_offset = 0
        self.parent_idx = -1
        self.external_ref_cnt = 0

    def as_tuple(self):
        return (list(self.page_ids), self.seq_length, self.start_pos, self.sink_length,
                self.sliding_window_offset, self.parent_idx, self.external_ref_cnt)


class Sequence:
    def __init__(self, pool, last_block_idx):
        pool[last_block_idx].external_ref_cnt += 1
        self.last_block_idx = last_block_idx
        self.seq_length = 0
        self.sliding_window_size = -1
        self.last_block_attn_sink_size = 0
        self.is_chain = True
        self.token_tree_parent_ptr = []
        self.token_tree_node_depths = []
        self.accepted_indices_committed = True
        ptr = last_block_idx
        while True:
            self.seq_length += pool[ptr].seq_length
            if pool[ptr].parent_idx == -1:
                break
            ptr = pool[ptr].parent_idx

    def copy(self):
        other = object.__new__(Sequence)
        other.__dict__.update(self.__dict__)
        other.token_tree_parent_ptr = list(self.token_tree_parent_ptr)
        other.token_tree_node_depths = list(self.token_tree_node_depths)
        return other

    def block_trace(self, pool):
        trace = []
        ptr = self.last_block_idx
        while ptr != -1:
            trace.append(ptr)
            ptr = pool[ptr].parent_idx
        return trace[::-1]


def get_block_ids_on_depth(sequences, pool):
    num_depths = 0
    seq_traces, trailing = [], []
    for seq in sequences:
        trace = seq.block_trace(pool)
        if len(trace) <= MAX_BLOCK_DEPTH:
            seq_traces.append(trace)
            trailing.append([])
            num_depths = max(num_depths, len(trace))
        else:
            seq_traces.append(trace[:MAX_BLOCK_DEPTH])
            trailing.append(trace[MAX_BLOCK_DEPTH:])
            num_depths = max(num_depths, MAX_BLOCK_DEPTH)
    on_depths = [[t[d] if d < len(t) else -1 for t in seq_traces] for d in range(num_depths)]
    return on_depths, trailing


def get_chunked_block_ids(block_ids, enable_coalesce, append_lengths, pool, is_decode_request):
    uncoalesced, coalesced = [], []
    cur_block_id = block_ids[0]
    chunk_append_length = append_lengths[0]
    page_counter_coalesced = 0
    page_counter_uncoalesced = len(pool[block_ids[0]].page_ids) if block_ids[0] != -1 else 0
    for i in range(1, len(block_ids)):
        if block_ids[i] != -1:
            page_counter_uncoalesced += len(pool[block_ids[i]].page_ids)
        uncoalesced.append((block_ids[i - 1], append_lengths[i - 1]))
        if block_ids[i] == cur_block_id:
            chunk_append_length += append_lengths[i]
        else:
            coalesced.append((cur_block_id, chunk_append_length))
            if cur_block_id != -1:
                page_counter_coalesced += len(pool[cur_block_id].page_ids)
            cur_block_id = block_ids[i]
            chunk_append_length = append_lengths[i]
    uncoalesced.append((block_ids[-1], append_lengths[-1]))
    coalesced.append((cur_block_id, chunk_append_length))
    if cur_block_id != -1:
        page_counter_coalesced += len(pool[cur_block_id].page_ids)
    ratio = page_counter_uncoalesced / page_counter_coalesced if page_counter_coalesced > 0 else 0.0
    use_decode_kernel = is_decode_request and ratio < 32
    return (uncoalesced if (use_decode_kernel or not enable_coalesce) else coalesced), use_decode_kernel


class HostCache:
    """cache_config = [reserved_num_seqs, total_token_capacity, prefill_chunk_size, page_size,
    support_sliding_window(, layer_sliding_window_size)] as in the reference's create call."""

    def __init__(self, cache_config, attn_kinds=(ATTN_MHA,), rope_mode=ROPE_NORMAL):
        _check(len(cache_config) in (5, 6), "KV cache config must contain five or six fields")
        self.reserved_num_seqs, capacity, self.prefill_chunk_size, self.page_size = cache_config[:4]
        support_sliding_window = bool(cache_config[4])
        self.layer_sliding_window_size = cache_config[5] if len(cache_config) == 6 else 1024
        self.num_total_pages = (capacity + self.page_size - 1) // self.page_size + 1
        if support_sliding_window:
            self.num_total_pages += self.reserved_num_seqs * 2
        self.attn_kinds = list(attn_kinds)
        has_layer_sliding = ATTN_MHA_SLIDING in self.attn_kinds
        self.support_sliding_window = False if has_layer_sliding else support_sliding_window
        self.support_layer_sliding_window = has_layer_sliding
        self.rope_mode = ROPE_INLINE if (support_sliding_window and rope_mode != ROPE_NONE) else rope_mode
        _check(self.layer_sliding_window_size > 0, "Per-layer sliding window size must be positive.")
        self.is_chain_on_depths = [True] * MAX_BLOCK_DEPTH
        self.clear()
        self.aux = {}

    # ------------------------------------------------------------------ pool
    def clear(self):
        self.seq_map = {}
        self.free_page_ids = list(range(self.num_total_pages - 1, -1, -1))
        self.pool = []
        self.free_block_idx = []
        self.dirty = False
        self.copies = []  # (src_page, tgt_page, copy_length) issued by fork, in order

    def _get_free_page(self):
        _check(self.free_page_ids, "The KV cache is full. No page can be allocated.")
        return self.free_page_ids.pop()

    def _get_free_block(self):
        if self.free_block_idx:
            idx = self.free_block_idx.pop()
            self.pool[idx].reset()
            return idx
        idx = len(self.pool)
        self.pool.append(Block(idx))
        return idx

    # ------------------------------------------------------------------ verbs
    def add_sequence(self, seq_id):
        _check(seq_id not in self.seq_map, f'The sequence "{seq_id}" is already in the KV cache.')
        block_idx = self._get_free_block()
        self.seq_map[seq_id] = Sequence(self.pool, block_idx)
        self.dirty = True

    def remove_sequence(self, seq_id):
        _check(seq_id in self.seq_map, f'The sequence "{seq_id}" cannot be found in KV cache.')
        block_idx = self.seq_map[seq_id].last_block_idx
        _check(self.pool[block_idx].external_ref_cnt >= 1, "ref count")
        while block_idx != -1 and self.pool[block_idx].external_ref_cnt == 1:
            self.free_page_ids.extend(self.pool[block_idx].page_ids)
            self.free_block_idx.append(block_idx)
            block_idx = self.pool[block_idx].parent_idx
        if block_idx != -1:
            _check(self.pool[block_idx].external_ref_cnt > 1, "ref count")
            self.pool[block_idx].external_ref_cnt -= 1
        del self.seq_map[seq_id]
        self.dirty = True

    def fork_sequence(self, parent_seq_id, child_seq_id, fork_pos=-1):
        _check(parent_seq_id in self.seq_map,
               f'The parent sequence "{parent_seq_id}" cannot be found in KV cache.')
        _check(child_seq_id not in self.seq_map,
               f'The child sequence "{child_seq_id}" is already in the KV cache.')
        parent = self.seq_map[parent_seq_id]
        _check(fork_pos >= -1, "The forked position should be non-negative, or -1 for last position as default.")
        _check(fork_pos <= parent.seq_length,
               "The forked position should not exceed the total length of parent sequence.")
        _check(parent.accepted_indices_committed, "token tree of the parent not committed")
        pool, ps = self.pool, self.page_size
        if fork_pos == -1:
            fork_pos = parent.seq_length
        if parent.sliding_window_size != -1:
            sink_size = parent.seq_length - pool[parent.last_block_idx].seq_length + parent.last_block_attn_sink_size
            _check(fork_pos <= sink_size, "sliding-window sequence can only be forked within the sink")
        if fork_pos == parent.seq_length and fork_pos % ps == 0 and pool[parent.last_block_idx].seq_length > 0:
            new_idx = self._get_free_block()
            pool[new_idx].start_pos = parent.seq_length
            pool[new_idx].parent_idx = parent.last_block_idx
            pool[new_idx].external_ref_cnt = 1
            parent.last_block_idx = new_idx
        child_idx = self._get_free_block()
        trace = parent.block_trace(pool)
        in_block_offset = fork_pos
        for forked in trace:
            if forked != trace[-1]:
                _check(pool[forked].seq_length > 0, "empty interior block")
                _check(pool[forked].seq_length % ps == 0, "interior block not page aligned")
                if pool[forked].seq_length <= in_block_offset:
                    in_block_offset -= pool[forked].seq_length
                    continue
            in_page_offset = in_block_offset % ps
            moved_offset = in_block_offset - in_page_offset
            moved_pages = moved_offset // ps
            if moved_pages == 0:
                parent_block_idx = pool[forked].parent_idx
                if parent_block_idx != -1:
                    pool[parent_block_idx].external_ref_cnt += 1
                pool[child_idx].parent_idx = parent_block_idx
            else:
                parent_block_idx = self._get_free_block()
                pool[parent_block_idx].parent_idx = pool[forked].parent_idx
                pool[forked].parent_idx = parent_block_idx
                pool[child_idx].parent_idx = parent_block_idx
                pool[parent_block_idx].external_ref_cnt = 2
                pool[parent_block_idx].page_ids = pool[forked].page_ids[:moved_pages]
                pool[forked].page_ids = pool[forked].page_ids[moved_pages:]
                pool[parent_block_idx].start_pos = pool[forked].start_pos
                pool[forked].start_pos += moved_offset
                pool[parent_block_idx].seq_length = moved_offset
                pool[forked].seq_length -= moved_offset
                if parent.sliding_window_size != -1 and forked == parent.last_block_idx:
                    _check(moved_offset <= parent.last_block_attn_sink_size, "sink")
                    parent.last_block_attn_sink_size -= moved_offset
            pool[child_idx].start_pos = fork_pos - in_page_offset
            pool[child_idx].seq_length = in_page_offset
            if in_page_offset > 0:
                src_page_id = pool[forked].page_ids[0]
                tgt_page_id = self._get_free_page()
                pool[child_idx].page_ids.append(tgt_page_id)
                self.copies.append((src_page_id, tgt_page_id, in_page_offset))
            break
        self.seq_map[child_seq_id] = Sequence(pool, child_idx)
        self.dirty = True

    def enable_sliding_window_for_seq(self, seq_id, sliding_window_size, attn_sink_size):
        _check(self.support_sliding_window or self.support_layer_sliding_window,
               "The KV cache does not support sliding window.")
        _check(seq_id in self.seq_map, f'The sequence "{seq_id}" cannot be found in KV cache.')
        _check(attn_sink_size >= 0, "attn sink size must be non negative")
        _check(sliding_window_size > 0, "sliding window size should be positive")
        _check(attn_sink_size < sliding_window_size, "The attn sink size should be less than the sliding window size.")
        seq = self.seq_map[seq_id]
        _check(seq.sliding_window_size == -1, "A sequence cannot be enabled twice for sliding window.")
        prefix_length = seq.seq_length - self.pool[seq.last_block_idx].seq_length
        _check(prefix_length >= 0, "prefix length")
        seq.last_block_attn_sink_size = max(attn_sink_size - prefix_length, 0)
        seq.sliding_window_size = sliding_window_size

    def popn(self, seq_id, n):
        _check(seq_id in self.seq_map, f'The sequence "{seq_id}" cannot be found in KV cache.')
        seq = self.seq_map[seq_id]
        _check(n >= 0, f"The length of popping {n} cannot be negative.")
        _check(n <= seq.seq_length, "pop length exceeds the whole sequence length")
        if n == 0:
            return
        pool, ps = self.pool, self.page_size
        block_idx = seq.last_block_idx
        _check(pool[block_idx].external_ref_cnt >= 1, "ref count")
        while block_idx != -1 and pool[block_idx].external_ref_cnt == 1:
            if n > pool[block_idx].seq_length:
                n -= pool[block_idx].seq_length
                seq.seq_length -= pool[block_idx].seq_length
                self.free_page_ids.extend(pool[block_idx].page_ids)
                self.free_block_idx.append(block_idx)
                block_idx = pool[block_idx].parent_idx
                seq.last_block_idx = block_idx
                continue
            cur_npage = len(pool[block_idx].page_ids)
            tgt_npage = (pool[block_idx].seq_length - n + ps - 1) // ps
            while cur_npage > tgt_npage:
                self.free_page_ids.append(pool[block_idx].page_ids.pop())
                cur_npage -= 1
            seq.seq_length -= n
            pool[block_idx].seq_length -= n
            n = 0
            break
        if n:
            temp_seq_id = -1 - seq_id
            _check(temp_seq_id not in self.seq_map, "temp id in use")
            self.fork_sequence(seq_id, temp_seq_id, seq.seq_length - n)
            self.remove_sequence(seq_id)
            self.seq_map[seq_id] = self.seq_map[temp_seq_id].copy()
            del self.seq_map[temp_seq_id]
        self.dirty = True

    # ------------------------------------------------------------------ queries
    def empty(self):
        return (not self.seq_map and len(self.free_block_idx) == len(self.pool)
                and len(self.free_page_ids) == self.num_total_pages)

    def get_num_available_pages(self):
        return len(self.free_page_ids)

    def get_total_sequence_length(self):
        return sum(s.seq_length for s in self.seq_map.values())

    # ------------------------------------------------------------------ sliding window helpers
    def _layer_sw_offset(self, seq_length):
        if seq_length <= self.layer_sliding_window_size:
            return 0
        return (seq_length - self.layer_sliding_window_size) % self.page_size

    def _layer_sw_num_pages(self, seq_length):
        if seq_length == 0:
            return 0
        window_length = min(seq_length, self.layer_sliding_window_size)
        return (self._layer_sw_offset(seq_length) + window_length + self.page_size - 1) // self.page_size

    def _slide_window_for_sequence(self, seq):
        if seq.sliding_window_size == -1 or not self.support_sliding_window:
            return
        if seq.seq_length <= seq.sliding_window_size:
            return
        ps = self.page_size
        length_to_slide = seq.seq_length - seq.sliding_window_size
        block = self.pool[seq.last_block_idx]
        if seq.last_block_attn_sink_size > 0 and block.sink_length == 0:
            _check(block.sliding_window_offset == 0, "offset")
            block.sink_length = seq.last_block_attn_sink_size
            block.sliding_window_offset = seq.last_block_attn_sink_size
        # the reference erases pages without looking (:1966-1972): undefined behaviour when a shared
        # prefix alone is longer than the window; an error here and in the library
        _check(length_to_slide <= block.seq_length - block.sink_length,
               f"The sliding window has to drop {length_to_slide} tokens, but the last block of the sequence holds only "
               f"{block.seq_length - block.sink_length} behind its attention sink.")
        num_sink_pages = (block.sink_length + ps - 1) // ps
        page_idx_after = (block.sliding_window_offset + length_to_slide) // ps
        page_start_offset_after = (block.sliding_window_offset + length_to_slide) % ps
        while page_idx_after > num_sink_pages:
            if block.page_ids[num_sink_pages] != TEMP_PAGE_ID:
                self.free_page_ids.append(block.page_ids[num_sink_pages])
            del block.page_ids[num_sink_pages]
            page_idx_after -= 1
        _check(page_idx_after in (num_sink_pages - 1, num_sink_pages), "slide")
        seq.seq_length = seq.sliding_window_size
        block.seq_length -= length_to_slide
        block.sliding_window_offset = page_idx_after * ps + page_start_offset_after
        _check(block.seq_length >= block.sink_length, "slide")
        _check(block.sliding_window_offset >= block.sink_length, "slide")
        _check((block.sliding_window_offset + (block.seq_length - block.sink_length) + ps - 1) // ps
               == len(block.page_ids), "slide page count")

    def _reserve_append_length_in_seq(self, seq, append_length):
        block = self.pool[seq.last_block_idx]
        _check(append_length > 0, "Append with length 0 is not allowed.")
        _check(block.external_ref_cnt == 1,
               f"The block is {block.external_ref_cnt - 1}-time referenced by other blocks, thus cannot accept new KV values.")
        ps = self.page_size
        cur_npage = len(block.page_ids)
        tgt_npage = (block.seq_length - block.sink_length + block.sliding_window_offset + append_length + ps - 1) // ps
        for _ in range(cur_npage, tgt_npage):
            if not self.free_page_ids and seq.sliding_window_size != -1 and self.support_sliding_window:
                block.page_ids.append(TEMP_PAGE_ID)
            else:
                block.page_ids.append(self._get_free_page())
        block.seq_length += append_length
        self._slide_window_for_sequence(seq)
        if self.support_sliding_window:
            for i, pid in enumerate(block.page_ids):
                if pid == TEMP_PAGE_ID:
                    block.page_ids[i] = self._get_free_page()
        self.dirty = True

    # ------------------------------------------------------------------ token tree
    def _construct_token_tree_mask(self, sequences, token_tree_parent_ptr, block_ids_on_depths,
                                   trailing_blocks, append_lengths, num_depths, aux):
        def check_for_sequence(seq_i, depth):
            if not self.append_before_attn:
                return True
            if (block_ids_on_depths[depth][seq_i] == sequences[seq_i].last_block_idx
                    or (depth + 1 == MAX_BLOCK_DEPTH and trailing_blocks[seq_i])):
                return True
            return False

        aux["tree_attn_mn_indptr"] = [[] for _ in range(MAX_BLOCK_DEPTH)]
        aux["tree_attn_mask"] = [[] for _ in range(MAX_BLOCK_DEPTH)]
        batch = len(sequences)
        for d in range(num_depths):
            mn_indptr, mask_out = [0], []
            in_depth = [False] * batch
            self.is_chain_on_depths = [True] * MAX_BLOCK_DEPTH
            is_chain = True
            offset = 0
            for i in range(batch):
                append_length = append_lengths[i]
                in_depth[i] = check_for_sequence(i, d)
                if not in_depth[i]:
                    mn_indptr.append(mn_indptr[-1])
                    offset += append_length
                    continue
                _check(len(sequences[i].token_tree_parent_ptr)
                       <= self.pool[sequences[i].last_block_idx].seq_length,
                       "The token tree size is larger than the sequence length of the last block.")
                sequences[i].token_tree_parent_ptr.extend(token_tree_parent_ptr[offset:offset + append_length])
                offset += append_length
                _check(len(sequences[i].token_tree_parent_ptr) <= TREE_MAX_SIZE, "tree too large")
                mn_indptr.append(mn_indptr[-1] + len(sequences[i].token_tree_parent_ptr))
            _check(len(token_tree_parent_ptr) == offset, "Invalid token tree size.")
            for i in range(batch):
                if not in_depth[i]:
                    continue
                seq = sequences[i]
                tree_size = len(seq.token_tree_parent_ptr)
                depth = []
                seq.is_chain = True
                seq.accepted_indices_committed = False
                children = {}
                roots = []
                for n in range(tree_size):
                    parent = seq.token_tree_parent_ptr[n]
                    _check(parent < n, "Invalid token tree: parent not smaller than node")
                    _check(parent >= -1, "Invalid token tree")
                    if parent != n - 1:
                        seq.is_chain = False
                        is_chain = False
                    children.setdefault(parent, []).append(n)
                    if parent != -1:
                        depth.append(depth[parent] + 1)
                    else:
                        depth.append(0)
                        roots.append(n)
                tree_order = [[0, 0] for _ in range(tree_size)]
                order = [0]

                def dfs(node):
                    tree_order[node][0] = order[0]
                    order[0] += 1
                    upper = tree_order[node][0] + 1
                    for child in children.get(node, []):
                        upper = max(upper, dfs(child))
                    tree_order[node][1] = upper
                    return upper

                for root in roots:
                    dfs(root)
                for n in range(tree_size):
                    mask_out.extend(tree_order[n])
                seq.token_tree_node_depths = depth
            self.is_chain_on_depths[d] = is_chain
            aux["tree_attn_mn_indptr"][d] = mn_indptr
            aux["tree_attn_mask"][d] = mask_out
            if not self.append_before_attn:
                break

    # ------------------------------------------------------------------ BeginForward
    def begin_forward(self, seq_ids, append_lengths, token_tree_parent_ptr=None):
        _check(len(seq_ids) == len(append_lengths), "seq_ids / append_lengths size mismatch")
        if self.attn_kinds[0] == ATTN_MLA:
            _check(token_tree_parent_ptr is None, "Tree attention is not supported yet for MLA")
        pool, ps = self.pool, self.page_size
        batch = len(seq_ids)
        self.cur_seq_ids = list(seq_ids)
        self.cur_append_lengths = list(append_lengths)
        sequences, last_block_length_before_append = [], []
        self.is_decode_request = True
        k_ragged_rope_pos_offset = []
        for i in range(batch):
            _check(seq_ids[i] in self.seq_map, f'The sequence "{seq_ids[i]}" cannot be found in KV cache.')
            seq = self.seq_map[seq_ids[i]]
            sequences.append(seq)
            last_block_length_before_append.append(pool[seq.last_block_idx].seq_length)
            k_rope_offset = seq.seq_length
            if not seq.accepted_indices_committed:
                k_rope_offset -= len(seq.token_tree_parent_ptr)
            k_ragged_rope_pos_offset.append(k_rope_offset)
            seq.seq_length += append_lengths[i]
            if append_lengths[i] != 1:
                self.is_decode_request = False

        block_ids_on_depths, trailing_blocks = get_block_ids_on_depth(sequences, pool)
        num_depths = min(len(block_ids_on_depths), MAX_BLOCK_DEPTH)
        chunked_arr, self.use_decode_kernel = [], []
        for d in range(num_depths):
            chunked, use_decode = get_chunked_block_ids(block_ids_on_depths[d], d != MAX_BLOCK_DEPTH - 1,
                                                        self.cur_append_lengths, pool, self.is_decode_request)
            chunked_arr.append(chunked)
            self.use_decode_kernel.append(use_decode)
        if num_depths == MAX_BLOCK_DEPTH:
            _check(len(chunked_arr[num_depths - 1]) == batch, "max depth blocks must not coalesce")
        self.append_before_attn = (not self.support_sliding_window) and self.use_decode_kernel[-1]
        if any(not s.accepted_indices_committed for s in sequences):
            self.append_before_attn = True

        aux = {"num_depths": num_depths}
        if token_tree_parent_ptr is not None:
            _check(not self.support_sliding_window, "Tree attention does not support sliding window.")
            _check(self.rope_mode != ROPE_INLINE, "Tree attention does not support inline RoPE mode.")
            self._construct_token_tree_mask(sequences, list(token_tree_parent_ptr), block_ids_on_depths,
                                            trailing_blocks, self.cur_append_lengths, num_depths, aux)
        else:
            for i, seq in enumerate(sequences):
                _check(seq.accepted_indices_committed,
                       f"Please invoke CommitAcceptedTokenTreeNodes for sequence {seq_ids[i]}")
                seq.is_chain = True
                seq.token_tree_parent_ptr = []
                seq.token_tree_node_depths = []
            self.is_chain_on_depths = [True] * MAX_BLOCK_DEPTH

        if self.append_before_attn:
            for i in range(batch):
                self._reserve_append_length_in_seq(sequences[i], append_lengths[i])

        names = ["qo_indptr", "page_indptr", "page_indices", "page_indptr_sliding_window",
                 "page_indices_sliding_window", "last_page_len", "sliding_window_offset", "sink_size",
                 "k_rope_pos_offset", "k_rope_pos_offset_sliding_window"]
        for name in names:
            aux[name] = [[] for _ in range(num_depths)]
        for d in range(num_depths):
            qo_indptr, page_indptr, page_indices = [0], [0], []
            page_indptr_sw, page_indices_sw = [0], []
            last_page_len, sw_offset, sink_size, k_rope, k_rope_sw = [], [], [], [], []
            for i, (block_id, chunk_append_length) in enumerate(chunked_arr[d]):
                qo_indptr.append(qo_indptr[-1] + chunk_append_length)
                if block_id == -1:
                    page_indptr.append(page_indptr[-1])
                    page_indptr_sw.append(page_indptr_sw[-1])
                    last_page_len.append(0)
                    sw_offset.append(0)
                    sink_size.append(0)
                    k_rope.append(0)
                    k_rope_sw.append(0)
                    continue
                block = pool[block_id]
                if d < MAX_BLOCK_DEPTH - 1:
                    page_indptr.append(page_indptr[-1] + len(block.page_ids))
                    page_indices.extend(block.page_ids)
                    n_sw = min(len(block.page_ids), self._layer_sw_num_pages(block.seq_length))
                    page_indptr_sw.append(page_indptr_sw[-1] + n_sw)
                    page_indices_sw.extend(page_indices[len(page_indices) - n_sw:])
                    last_page_len.append(0 if block.seq_length == 0 else
                                         (block.seq_length - block.sink_length + block.sliding_window_offset - 1) % ps + 1)
                    sw_offset.append(self._layer_sw_offset(block.seq_length) if self.support_layer_sliding_window
                                     else block.sliding_window_offset)
                    sink_size.append(block.sink_length)
                    k_rope.append(block.start_pos)
                    if self.support_layer_sliding_window:
                        k_rope_sw.append(max(0, block.start_pos + block.seq_length - self.layer_sliding_window_size))
                else:
                    num_pages = len(block.page_ids)
                    total_seq_length = block.seq_length
                    last_block_id = block_id
                    page_indices.extend(block.page_ids)
                    for tid in trailing_blocks[i]:
                        tb = pool[tid]
                        page_indices.extend(tb.page_ids)
                        num_pages += len(tb.page_ids)
                        total_seq_length += tb.seq_length
                        last_block_id = tid
                    page_indptr.append(page_indptr[-1] + num_pages)
                    n_sw = min(num_pages, self._layer_sw_num_pages(total_seq_length))
                    page_indptr_sw.append(page_indptr_sw[-1] + n_sw)
                    page_indices_sw.extend(page_indices[len(page_indices) - n_sw:])
                    last_block = pool[last_block_id]
                    last_page_len.append(0 if total_seq_length == 0 else
                                         (total_seq_length - last_block.sink_length + last_block.sliding_window_offset - 1) % ps + 1)
                    sw_offset.append(self._layer_sw_offset(total_seq_length) if self.support_layer_sliding_window
                                     else last_block.sliding_window_offset)
                    sink_size.append(last_block.sink_length)
                    k_rope.append(block.start_pos)
                    if self.support_layer_sliding_window:
                        k_rope_sw.append(max(0, block.start_pos + total_seq_length - self.layer_sliding_window_size))
            aux["qo_indptr"][d] = qo_indptr
            aux["page_indptr"][d] = page_indptr
            aux["page_indices"][d] = page_indices
            aux["page_indptr_sliding_window"][d] = page_indptr_sw
            aux["page_indices_sliding_window"][d] = page_indices_sw
            aux["last_page_len"][d] = last_page_len
            aux["sliding_window_offset"][d] = sw_offset
            aux["sink_size"][d] = sink_size
            aux["k_rope_pos_offset"][d] = k_rope
            aux["k_rope_pos_offset_sliding_window"][d] = k_rope_sw

        if not self.append_before_attn:
            for i in range(batch):
                self._reserve_append_length_in_seq(sequences[i], append_lengths[i])

        q_rope_position_map, append_position_map = [], []
        for i in range(batch):
            append_length = append_lengths[i]
            block = pool[sequences[i].last_block_idx]
            for pos in range(append_length):
                if not sequences[i].token_tree_node_depths:
                    q_rope_position_map.append(k_ragged_rope_pos_offset[i] + pos)
                else:
                    offset_in_tree = len(sequences[i].token_tree_parent_ptr) - append_length
                    _check(offset_in_tree >= 0, "tree offset")
                    q_rope_position_map.append(k_ragged_rope_pos_offset[i]
                                               + sequences[i].token_tree_node_depths[offset_in_tree + pos])
                pos_in_block = block.seq_length - append_length + pos
                if last_block_length_before_append[i] + pos < block.sink_length:
                    off = last_block_length_before_append[i] + pos
                    append_position_map.append(block.page_ids[off // ps] * ps + off % ps)
                elif pos_in_block < block.sink_length:
                    append_position_map.append(-1)
                else:
                    off = pos_in_block - block.sink_length + block.sliding_window_offset
                    append_position_map.append(block.page_ids[off // ps] * ps + off % ps)
        indptr = [0]
        for n in append_lengths:
            indptr.append(indptr[-1] + n)
        aux["q_rope_position_map"] = q_rope_position_map
        aux["append_position_map"] = append_position_map
        aux["cur_append_lengths_indptr"] = indptr
        aux["k_ragged_rope_pos_offset"] = k_ragged_rope_pos_offset
        aux["append_before_attn"] = self.append_before_attn
        aux["use_decode_kernel"] = list(self.use_decode_kernel)
        aux["is_chain_on_depths"] = list(self.is_chain_on_depths)
        self.aux = aux
        self.num_depths = num_depths
        return aux

    def end_forward(self):
        pass

    def commit_accepted_token_tree_nodes(self, seq_ids, leaf_indices):
        """Returns the (copy_length_indptr, src_pos, dst_pos) handed to the compact-copy kernel, or
        None when every tree is a chain."""
        _check(len(seq_ids) == len(leaf_indices), "size mismatch")
        sequences = []
        is_chain = True
        for i, sid in enumerate(seq_ids):
            _check(sid in self.seq_map, f'The sequence "{sid}" cannot be found in KV cache.')
            seq = self.seq_map[sid]
            sequences.append(seq)
            is_chain = seq.is_chain
            _check(leaf_indices[i] == -1 or not seq.accepted_indices_committed, "already committed")
            _check(leaf_indices[i] >= -1, "invalid tree index")
            _check(leaf_indices[i] < len(seq.token_tree_parent_ptr), "invalid tree index")
        result = None
        if not is_chain:
            indptr, src, dst = [0], [], []
            apm = self.aux["append_position_map"]
            cur_indptr = self.aux["cur_append_lengths_indptr"]
            for i, seq in enumerate(sequences):
                if leaf_indices[i] == -1:
                    indptr.append(indptr[-1])
                    continue
                path = []
                node = leaf_indices[i]
                while node != -1:
                    path.append(node)
                    node = seq.token_tree_parent_ptr[node]
                _check(len(path) == seq.token_tree_node_depths[leaf_indices[i]] + 1, "path length")
                dst_pos = list(range(len(path)))[::-1]
                while path and path[-1] == dst_pos[-1]:
                    path.pop()
                    dst_pos.pop()
                path.reverse()
                dst_pos.reverse()
                for p in range(len(path)):
                    src.append(apm[cur_indptr[i] + path[p]])
                    dst.append(apm[cur_indptr[i] + dst_pos[p]])
                indptr.append(indptr[-1] + len(path))
            result = (indptr, src, dst)
        for i, seq in enumerate(sequences):
            length_to_pop = self.cur_append_lengths[i] - (
                seq.token_tree_node_depths[leaf_indices[i]] + 1 if leaf_indices[i] != -1 else 0)
            self.popn(self.cur_seq_ids[i], length_to_pop)
            seq.accepted_indices_committed = True
            seq.token_tree_parent_ptr = []
            seq.token_tree_node_depths = []
        return result

    # ------------------------------------------------------------------ introspection
    def position_map_of(self, seq_id):
        """Global slot ids of every cached token of a sequence (DebugGetKV,
        src/runtime/vm/paged_kv_cache.cc:1698-1710)."""
        seq = self.seq_map[seq_id]
        out = []
        for block_id in seq.block_trace(self.pool):
            block = self.pool[block_id]
            for i in range(block.seq_length):
                off = i if i < block.sink_length else i - block.sink_length + block.sliding_window_offset
                out.append(block.page_ids[off // self.page_size] * self.page_size + off % self.page_size)
        return out

    def state(self):
        """Canonical snapshot of the pool, comparable with the C++ cache's dump."""
        return {
            "free_page_ids": list(self.free_page_ids),
            "free_block_idx": list(self.free_block_idx),
            "blocks": [b.as_tuple() for b in self.pool],
            "seqs": {sid: (s.last_block_idx, s.seq_length, s.sliding_window_size, s.last_block_attn_sink_size)
                     for sid, s in self.seq_map.items()},
        }
