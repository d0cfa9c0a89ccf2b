"""Host-side checks of the split-KV chunk-slot arithmetic (the kernels repeat it on the device from
page_indptr alone) and of the library's tuning options, on page tables chosen to break it: empty
sequences, page counts that are not multiples of the chunk, more than 64 sequences, one very long
sequence among short ones."""
import numpy as np
import pytest

import tvm_amd


def enumerate_chunks(page_counts, cp):
    """Direct statement of what the grid must cover: ceil(n / cp) chunks per sequence, in order."""
    return [(b, c) for b, n in enumerate(page_counts) for c in range(-(-n // cp))]


CASES = {
    "single": [37],
    "empty_first_last": [0, 5, 0, 0, 130, 0],
    "all_empty": [0, 0, 0],
    "multiples_of_8": [8, 16, 64, 128],
    "one_short_of_a_chunk": [7, 15, 63, 127, 1],
    "one_past_a_chunk": [9, 17, 65, 129],
    "long_among_short": [1] * 20 + [8192] + [2] * 20,
    "more_than_64_sequences": list(np.random.default_rng(0).integers(0, 90, size=150)),
    "cfg2_like": list(np.random.default_rng(1).integers(64, 513, size=64)),
    "cfg4_like": list(np.random.default_rng(3).integers(2048, 8193, size=8)),
}


@pytest.mark.parametrize("h_kv", [1, 8])
@pytest.mark.parametrize("forced_cp", [0, 8, 64])
@pytest.mark.parametrize("name", sorted(CASES))
def test_every_chunk_has_exactly_one_slot(name, forced_cp, h_kv):
    counts = [int(n) for n in CASES[name]]
    indptr = np.concatenate([[0], np.cumsum(counts)])
    nnz = int(indptr[-1])
    prev = tvm_amd.set_option("decode_chunk_pages", forced_cp)
    try:
        cp, slot_seq, slot_chunk = tvm_amd.decode_split_plan(indptr, nnz, h_kv)
    finally:
        tvm_amd.set_option("decode_chunk_pages", prev)
    assert cp % 8 == 0 and 8 <= cp <= 128
    if forced_cp:
        assert cp == forced_cp
    assert len(slot_seq) == nnz // cp + len(counts)  # the grid is sized from shapes alone
    used = [(b, c) for b, c in zip(slot_seq, slot_chunk) if b >= 0]
    assert used == enumerate_chunks(counts, cp)       # every chunk once, in order; the rest are spare
    assert all(c == -1 for b, c in zip(slot_seq, slot_chunk) if b < 0)


def test_chunk_size_follows_the_work():
    # 768 work items for small launches up to ~2300 for large ones; chunks of 16 to 128 pages
    assert tvm_amd.decode_split_plan([0, 4], 4, 8)[0] == 24             # small launches: 24 pages at least
    cfg2 = [288 * i for i in range(65)]
    assert tvm_amd.decode_split_plan(cfg2, 18432, 8)[0] == 48            # configs[1]: 64 pages by the item count, its neighbour that does not camp
    assert tvm_amd.decode_split_plan(cfg2, 18432, 4)[0] == 64            # four kv heads: no camping seen
    assert tvm_amd.decode_split_plan([0, 18432], 18432, 8)[0] == 128     # as one sequence: fewer states to merge
    short = [80 * i for i in range(257)]
    assert tvm_amd.decode_split_plan(short, 80 * 256, 8)[0] == 128       # 256 short sequences: no split at all
    assert tvm_amd.decode_split_plan([0, 1 << 20], 1 << 20, 8)[0] == 128
    assert tvm_amd.decode_split_plan([0, 18432], 18432, 1)[0] == 32      # one kv head: 768 items
    assert tvm_amd.decode_split_plan([0, 8192], 8192, 8)[0] == 128       # one sequence of 131072 tokens: 64 states, not 128
    assert tvm_amd.decode_split_plan([0, 4096, 8192], 8192, 8)[0] == 128  # two of 65536
    assert tvm_amd.decode_split_plan([0, 2048, 4096, 6144, 8192], 8192, 8)[0] == 104  # four of 32768: the grid fits 768 workgroups (96 would camp)
    long8 = [5000 * i for i in range(9)]
    assert tvm_amd.decode_split_plan(long8, 40000, 8)[0] == 112          # eight long sequences: 128 by the states, its neighbour
    assert tvm_amd.decode_split_plan([0, 100, 250, 400, 457], 457, 8)[0] == 24          # (457 / 24 + 4) * 8 = 184 items


def test_options_round_trip_and_reject_unknown_names():
    assert tvm_amd.set_option("mla_chunk_tokens", 256) == 0
    assert tvm_amd.set_option("mla_chunk_tokens", 0) == 256
    with pytest.raises(tvm_amd.KVError, match="unknown option"):
        tvm_amd.set_option("no_such_option", 1)
