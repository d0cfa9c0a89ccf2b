"""The decode entry point that allocates nothing (tvmkv_batch_decode_paged_kv_noalloc): its scratch
memory is an array built into the library, addressed through hipGetSymbolAddress.  Called through
the C ABI twice in a row, the second time with a smaller input (the array keeps the first call's
contents), and compared bit for bit with the allocating entry point, which runs the same kernels;
both against the CPU oracle."""
import numpy as np
import pytest
import torch

import tvm_amd
from oracle import kernels as ok
from tests.gpu_util import DEV, dev, host, i32
from tests.util import assert_close, build_paged_kv
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
F16 = np.float16


def _run(rng, kv_lens, hq, hkv, d, npages, noalloc):
    pages, indptr, values, last, _, _ = build_paged_kv(rng, kv_lens, npages, hkv, 16, d)
    b = len(kv_lens)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    z = np.zeros(b, np.int32)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    ok.decode(q, pages, indptr, values, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    outs = []
    args = (dev(q), dev(pages), i32(indptr), i32(values), i32(last), i32(z), i32(z))
    for flag in noalloc:
        go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_decode_paged_kv(*args, go, gl, 0, 1.0, 1e4, d ** -0.5, noalloc=flag)
        outs.append((host(go), host(gl)))
    return outs, eo, el


def test_noalloc_decode_matches_the_allocating_entry_point_twice_in_a_row():
    rng = np.random.default_rng(31)
    # first call: many chunks per sequence (multi-chunk merge through the arrival counters)
    big = [9000, 5, 4100, 0, 777, 2049, 16, 1]
    (na1, al1), eo, el = _run(rng, big, 32, 8, 128, npages=1100, noalloc=[True, False])
    assert np.array_equal(na1[0], al1[0]) and np.array_equal(na1[1], al1[1]), "first call differs"
    assert_close(na1[0], eo, what="noalloc decode out (first call)")
    assert_close(na1[1], el, atol=1e-3, rtol=1e-4, what="noalloc decode lse (first call)")
    # second call, smaller: fewer sequences, fewer chunks, other head shape; stale partial states and
    # counters of the first call are still in the array
    small = [300, 0, 129]
    (na2, al2), eo, el = _run(rng, small, 16, 2, 128, npages=40, noalloc=[True, False])
    assert np.array_equal(na2[0], al2[0]) and np.array_equal(na2[1], al2[1]), "second call differs"
    assert_close(na2[0], eo, what="noalloc decode out (second call)")
    assert_close(na2[1], el, atol=1e-3, rtol=1e-4, what="noalloc decode lse (second call)")
    # and again the large one: counters left by both calls must read as zero in a new epoch
    (na3, al3), eo, el = _run(np.random.default_rng(31), big, 32, 8, 128, npages=1100, noalloc=[True, False])
    assert np.array_equal(na3[0], na1[0]) and np.array_equal(na3[1], na1[1]), "third call differs from the first"


def test_noalloc_decode_head_dim_64_uses_the_same_array():
    rng = np.random.default_rng(32)
    (na, al), eo, el = _run(rng, [700, 33, 0, 64], 8, 4, 64, npages=60, noalloc=[True, False])
    assert np.array_equal(na[0], al[0]) and np.array_equal(na[1], al[1])
    assert_close(na[0], eo, what="noalloc decode out (head_dim 64)")


def test_noalloc_decode_refuses_what_does_not_fit():
    """24 MiB built in: a shape whose partial states need more is rejected before any launch."""
    b, hq, hkv, d = 1024, 128, 8, 128
    nnz = 8
    t = lambda *shape, dt=torch.float16: torch.zeros(shape, dtype=dt, device=DEV)
    q, pages = t(b, hq, d), t(16, 2, hkv, 16, d)
    indptr = torch.zeros(b + 1, dtype=torch.int32, device=DEV)
    indptr[1:] = nnz
    vals = torch.arange(nnz, dtype=torch.int32, device=DEV)
    z = torch.zeros(b, dtype=torch.int32, device=DEV)
    last = torch.ones(b, dtype=torch.int32, device=DEV)
    with pytest.raises(tvm_amd.KVError, match="bytes of scratch memory"):
        K.batch_decode_paged_kv(q, pages, indptr, vals, last, z, z, t(b, hq, d), t(b, hq, dt=torch.float32), 0, 1.0,
                                1e4, d ** -0.5, noalloc=True)


def test_noalloc_decode_in_a_graph_that_is_replayed():
    """Callers under HIP graph capture are what the entry point is for: a captured launch keeps its
    arguments, the epoch of the arrival counters included, so every replay must find the counters as a
    first launch does.  Replayed with new q, new K/V data and new sequence ends between the replays
    (eager work and synchronisations in between), each replay compared bit for bit with an eager call
    of the allocating entry point and, first and last, with the oracle."""
    rng = np.random.default_rng(33)
    kv_lens = [9000, 5, 4100, 0, 777, 2049, 16, 1]
    hq, hkv, d = 32, 8, 128
    pages, indptr, values, last, _, _ = build_paged_kv(rng, kv_lens, 1100, hkv, 16, d)
    b = len(kv_lens)
    z = i32(np.zeros(b, np.int32))
    tq = dev(rng.standard_normal((b, hq, d)).astype(F16))
    tpages, tind, tval, tlast = dev(pages), i32(indptr), i32(values), i32(last)
    go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
    eo_t, el_t = torch.empty_like(go), torch.empty_like(gl)
    call = lambda o, l, noalloc: K.batch_decode_paged_kv(tq, tpages, tind, tval, tlast, z, z, o, l, 0, 1.0, 1e4, d ** -0.5,
                                                         noalloc=noalloc)
    call(go, gl, True)  # the first call on a device looks up the array's address: not a thing to capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(go, gl, True)
    for rep in range(4):
        q = rng.standard_normal((b, hq, d)).astype(F16)
        new_last = np.where(np.asarray(last) > 0, rng.integers(1, 17, size=b), 0).astype(np.int32)
        tq.copy_(dev(q))
        tlast.copy_(i32(new_last))
        tpages.mul_(-1.0 if rep % 2 else 0.5)
        go.fill_(7.0)
        gl.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        call(eo_t, el_t, False)
        assert torch.equal(go, eo_t) and torch.equal(gl, el_t), f"replay {rep} differs from the eager call"
        if rep in (0, 3):
            eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
            ok.decode(q, host(tpages), indptr, values, new_last, np.zeros(b, np.int32), np.zeros(b, np.int32), eo, el, 0, 1.0,
                      1e4, d ** -0.5)
            assert_close(host(go), eo, what=f"replay {rep} out")
            assert_close(host(gl), el, atol=1e-3, rtol=1e-4, what=f"replay {rep} lse")


def test_allocating_entry_point_says_so_under_capture():
    """The allocating entry point under capture, on a stream it has no scratch memory for yet: refused
    with a message that names the way out, before any HIP call that would spoil the capture."""
    rng = np.random.default_rng(34)
    hq, hkv, d = 32, 8, 128
    pages, indptr, values, last, _, _ = build_paged_kv(rng, [5000, 3000], 520, hkv, 16, d)
    z = i32(np.zeros(2, np.int32))
    args = (dev(rng.standard_normal((2, hq, d)).astype(F16)), dev(pages), i32(indptr), i32(values), i32(last), z, z)
    go = torch.zeros((2, hq, d), dtype=torch.float16, device=DEV)
    gl = torch.zeros((2, hq), dtype=torch.float32, device=DEV)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        with pytest.raises(tvm_amd.KVError, match="captured into a graph"):
            K.batch_decode_paged_kv(*args, go, gl, 0, 1.0, 1e4, d ** -0.5)
        K.batch_decode_paged_kv(*args, go, gl, 0, 1.0, 1e4, d ** -0.5, noalloc=True)  # the capture is still good
    graph.replay()
    torch.cuda.synchronize()
    eo, el = torch.empty_like(go), torch.empty_like(gl)
    K.batch_decode_paged_kv(*args, eo, el, 0, 1.0, 1e4, d ** -0.5)
    assert torch.equal(go, eo) and torch.equal(gl, el)
