"""The HIP path against the committed golden fixtures (tests/golden/): split + rotary embedding,
and the 4-sequence decode configuration (contexts 512/1024/1500/2048, 32 query / 8 kv heads,
head_dim 128, page 16, 1024-page pool) driven through the cache verbs: page table and append
indices bit-exact, attention output within atol = rtol = 1e-2."""
import os

import numpy as np
import pytest
import torch

from tests.golden import make_fixtures as mf
from tests.gpu_util import DEV, GpuCache, dev, host, i32
from tests.util import assert_close
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
GOLD = os.path.dirname(os.path.abspath(mf.__file__))


def test_fused_rope_matches_fixture():
    g = np.load(os.path.join(GOLD, "rope_vectors.npz"))
    q = torch.zeros(g["q"].shape, dtype=torch.float16, device=DEV)
    k = torch.zeros(g["k"].shape, dtype=torch.float16, device=DEV)
    v = torch.zeros(g["v"].shape, dtype=torch.float16, device=DEV)
    K.fused_rope(dev(g["qkv"]), i32(g["pos"]), q, k, v, 1, 1.0, 1e4)
    # device sin/cos differ from libm in the last ulp: allow one fp16 ulp
    assert_close(host(q), g["q"], atol=2e-3, rtol=1e-3, what="rope q")
    assert_close(host(k), g["k"], atol=2e-3, rtol=1e-3, what="rope k")
    assert np.array_equal(host(v), g["v"])
    assert np.array_equal(host(q)[0], g["q"][0]), "position 0 must be the identity, exactly"


def test_cfg1_decode_matches_fixture():
    g = np.load(os.path.join(GOLD, "cfg1_decode.npz"))
    c = mf.CFG1
    cache = GpuCache(mf.cfg1_cache_config(), 1, c["hq"], c["hkv"], c["d"], c["d"], rope_mode=1)
    seen = {}

    def grab():
        for name in mf.PER_DEPTH:
            seen[name] = cache.cache.aux(name, 0)
        for name in mf.GLOBAL:
            seen[name] = cache.cache.aux(name)

    qkv, out = mf.cfg1_drive(cache, grab)
    assert np.array_equal(qkv, g["qkv"])
    for name in mf.PER_DEPTH + mf.GLOBAL:
        assert seen[name] == list(g[name]), name
    assert_close(out, g["out"], what="cfg1 decode output")
