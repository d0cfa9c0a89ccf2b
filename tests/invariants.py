"""Structural invariants of the paged-KV pool, checked on a ``state()`` snapshot
(``{"free_page_ids", "free_block_idx", "blocks", "seqs"}``) of either implementation."""


def check_pool_invariants(state, num_total_pages, page_size):
    blocks = state["blocks"]
    free_blocks = set(state["free_block_idx"])
    assert len(free_blocks) == len(state["free_block_idx"]), "duplicate free block index"
    live = [i for i in range(len(blocks)) if i not in free_blocks]
    # every page id is in exactly one of {free list, one live block}
    seen = list(state["free_page_ids"])
    for i in live:
        seen.extend(blocks[i][0])
    assert sorted(seen) == list(range(num_total_pages)), "page ids are not a partition of the pool"
    children = {i: 0 for i in live}
    for i in live:
        page_ids, seq_length, start_pos, sink, sw_off, parent, ref = blocks[i]
        if parent != -1:
            assert parent in children, f"block {i} has a freed parent {parent}"
            children[parent] += 1
            pp = blocks[parent]
            assert pp[2] + pp[1] == start_pos, f"block {i} does not start where its parent ends"
            assert pp[1] % page_size == 0 and pp[1] > 0, "interior block must be full pages"
        if sink == 0 and sw_off == 0:
            assert len(page_ids) == (seq_length + page_size - 1) // page_size, f"block {i} page count"
    ending = {i: 0 for i in live}
    for sid, (last_block, seq_length, _, _) in state["seqs"].items():
        assert last_block in ending, f"sequence {sid} ends in a freed block"
        ending[last_block] += 1
        total, ptr = 0, last_block
        while ptr != -1:
            total += blocks[ptr][1]
            ptr = blocks[ptr][5]
        assert total == seq_length, f"sequence {sid}: block lengths sum to {total}, not {seq_length}"
    for i in live:
        assert blocks[i][6] == children[i] + ending[i], (
            f"block {i}: external_ref_cnt {blocks[i][6]} != children {children[i]} + sequences {ending[i]}")
