"""Shared helpers of the test-suite: page-table builders and tolerance checks."""
import numpy as np

ATOL = RTOL = 1e-2  # fp16 outputs, fp32 accumulate: the tolerance the path is specified to


def assert_close(actual, expected, atol=ATOL, rtol=RTOL, what=""):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    for name, a in (("actual", actual), ("expected", expected)):  # NaN would compare as "not greater than the tolerance"
        if not np.isfinite(a).all():
            idx = tuple(np.argwhere(~np.isfinite(a))[0])
            raise AssertionError(f"{what}: {name} holds {a[idx]!r} at {idx} ({(~np.isfinite(a)).sum()} non-finite elements)")
    err = np.abs(actual - expected)
    tol = atol + rtol * np.abs(expected)
    bad = err > tol
    if bad.any():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} / {bad.size} elements out of tolerance; worst at {idx}: "
            f"actual {actual[idx]!r} expected {expected[idx]!r}")


def rows_without_keys(q_lens, causal, window):
    """Boolean mask over the query rows of a paged prefill call: under the per-layer window mask row r of
    a sequence sees the last max(window - r - 1, 0) keys (python/tvm/relax/frontend/nn/llm/
    _kernel_common.py:138-144), so rows from window - 1 on see none.  For such a row the reference's CPU
    kernel divides 0 by 0 (its running maximum is the previous row's, _prefill_kernels.py:192-201, and
    the oracle restates that) and its GPU kernel averages V over the masked keys; the library returns
    what a sequence without keys returns, out = 0 and lse = -5e4, and the tests pin that."""
    if not (causal and window > 0):
        return np.zeros(sum(q_lens), bool)
    return np.concatenate([np.arange(n) >= window - 1 for n in q_lens])


def assert_close_where_keys(actual_out, actual_lse, expected_out, expected_lse, no_keys, lse_atol, what):
    """assert_close on the rows that see keys; out = 0 and lse = -5e4 on the others."""
    assert not np.asarray(actual_out)[no_keys].any(), f"{what}: rows without keys must be 0"
    assert np.all(np.asarray(actual_lse)[no_keys] == np.float32(-5e4)), f"{what}: lse of rows without keys must be -5e4"
    assert_close(np.asarray(actual_out)[~no_keys], np.asarray(expected_out)[~no_keys], what=f"{what} out")
    assert_close(np.asarray(actual_lse)[~no_keys], np.asarray(expected_lse)[~no_keys], atol=lse_atol, rtol=1e-4,
                 what=f"{what} lse")


def build_paged_kv(rng, kv_lens, num_pages, hkv, page_size, d, permute=True, scale=1.0,
                   dtype=np.float16):
    """Random K/V for each sequence scattered into a page pool.

    Returns (pages, page_indptr, page_values, last_page_len, ks, vs) where ks[i]/vs[i] are the
    dense (len, hkv, d) arrays of sequence i.
    """
    pages = np.zeros((num_pages, 2, hkv, page_size, d), dtype=dtype)
    order = rng.permutation(num_pages) if permute else np.arange(num_pages)
    indptr = [0]
    values = []
    last = []
    ks, vs = [], []
    cursor = 0
    for n in kv_lens:
        npage = (n + page_size - 1) // page_size
        ids = order[cursor:cursor + npage]
        cursor += npage
        assert cursor <= num_pages
        k = (rng.standard_normal((n, hkv, d)) * scale).astype(dtype)
        v = (rng.standard_normal((n, hkv, d)) * scale).astype(dtype)
        for t in range(n):
            pages[ids[t // page_size], 0, :, t % page_size, :] = k[t]
            pages[ids[t // page_size], 1, :, t % page_size, :] = v[t]
        values.extend(int(x) for x in ids)
        indptr.append(len(values))
        last.append(0 if n == 0 else (n - 1) % page_size + 1)
        ks.append(k)
        vs.append(v)
    return (pages, np.array(indptr, np.int32), np.array(values, np.int32),
            np.array(last, np.int32), ks, vs)


# Token trees of the reference's speculative-decoding test
# (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:1076-1081)
REFERENCE_TREES = [
    [-1, 0, 0, 1, 1, 2, 2],  # complete binary tree of height 3
    [-1, 0, 0, 1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6],  # complete binary tree of height 4
    [-1, 0, 1, 2, 3, 4, 5, 6, 7, 8],  # chain of length 10
    [-1, 0, 0, 1, 1, 2, 2, -1, 7, 7, 8, 8, 9, 9],  # two complete binary trees of height 3
]


def random_forest(rng, n, p_root=0.15):
    """Parent pointers of a random forest: parent[i] < i, -1 for roots."""
    return [-1 if (i == 0 or rng.random() < p_root) else int(rng.integers(0, i)) for i in range(n)]


def tree_order(parent_ptr):
    """(n, 2) int32 labels a cache hands to the tree-attention kernels: the pre-order number of
    each node (roots and children in index order) and the end of the range its subtree covers."""
    n = len(parent_ptr)
    children = {}
    for node, parent in enumerate(parent_ptr):
        children.setdefault(parent, []).append(node)
    labels = np.zeros((n, 2), np.int32)
    counter = 0
    for root in children.get(-1, []):
        stack = [(root, False)]
        while stack:
            node, done = stack.pop()
            if done:
                labels[node, 1] = counter
                continue
            labels[node, 0] = counter
            counter += 1
            stack.append((node, True))
            for child in reversed(children.get(node, [])):
                stack.append((child, False))
    return labels
