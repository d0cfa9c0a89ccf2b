"""Shared helpers of the test-suite: page-table builders and tolerance checks."""
import numpy as np

ATOL = RTOL = 1e-2  # fp16 outputs, fp32 accumulate: the tolerance the path is specified to


def assert_close(actual, expected, atol=ATOL, rtol=RTOL, what=""):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    err = np.abs(actual - expected)
    tol = atol + rtol * np.abs(expected)
    bad = err > tol
    if bad.any():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} / {bad.size} elements out of tolerance; worst at {idx}: "
            f"actual {actual[idx]!r} expected {expected[idx]!r}")


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
