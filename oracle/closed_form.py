"""Closed forms that pin the oracle (numpy, float32/float64).

TEST INFRASTRUCTURE ONLY.  These are the mathematical definitions the reference's own
tests check its kernels against, written down independently of ``kv_kernels.c`` so that a
dropped term, a wrong sign or a transposed index in the C restatement fails a comparison:

* ``apply_rotary`` -- rotate-half RoPE with ``inv_freq = scale / theta**(arange(0,D,2)/D)``
  (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:305-324).
* ``attention`` -- ``softmax(q k^T * sm_scale + causal mask) v`` with GQA head repeat and the
  query block aligned to the *end* of the keys (same file, :499-535 and :596-607); also
  returns the base-2 log-sum-exp the kernels expose
  (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:176).
* ``tree_ancestor_mask`` -- the token-tree mask of speculative decoding from the parent
  pointers (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:614-627).
* ``merge`` -- two-way log-sum-exp merge of partial attention states
  (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:441-450).
* ``mla_expand`` -- MLA by its definition: expand the latent with ``w_kv`` and run plain MHA
  (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_mla_tir.py:351-398).
"""
import numpy as np


def apply_rotary(x, positions, scale=1.0, theta=1e4):
    """x: (N, H, D) any float dtype; positions: (N,) ints.  Returns float32."""
    x = np.asarray(x, dtype=np.float32)
    nfeat = x.shape[-1]
    half = nfeat // 2
    y = np.concatenate([-x[:, :, half:], x[:, :, :half]], axis=-1)
    inv_freq = scale / (theta ** (np.arange(0, nfeat, 2).astype("float32") / nfeat))
    t = np.asarray(positions, dtype=inv_freq.dtype)
    freqs = np.einsum("i,j->ij", t, inv_freq)
    emb = np.concatenate((freqs, freqs), axis=-1)
    return np.einsum("ij,ikj->ikj", np.cos(emb), x) + np.einsum("ij,ikj->ikj", np.sin(emb), y)


def tree_ancestor_mask(parent_ptr):
    """(n, n) bool: node i sees node j iff j is i or an ancestor of i.

    Built the way the reference's test builds it: a node inherits its parent's row and adds
    itself (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:614-627).
    """
    n = len(parent_ptr)
    mask = np.zeros((n, n), dtype=bool)
    for i, parent in enumerate(parent_ptr):
        if parent != -1:
            mask[i] = mask[parent]
        mask[i, i] = True
    return mask


def attention(q, k, v, sm_scale, causal=True, window=None, mask=None):
    """q: (Lq, Hq, Dqk), k: (Lk, Hkv, Dqk), v: (Lk, Hkv, Dv).

    ``mask`` (Lq, Lk) bool, if given, replaces the causal / window masks.

    Query i sits at absolute position Lk - Lq + i.  Returns (out float64 (Lq, Hq, Dv),
    lse_base2 float64 (Lq, Hq)).  An all-masked row gives out 0 and lse -inf.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    lq, hq, _ = q.shape
    lk, hkv, _ = k.shape
    group = hq // hkv
    k = np.repeat(k, group, axis=1)
    v = np.repeat(v, group, axis=1)
    scores = np.einsum("qhd,khd->hqk", q, k) * sm_scale
    qpos = lk - lq + np.arange(lq)
    kpos = np.arange(lk)
    if mask is None:
        mask = np.ones((lq, lk), dtype=bool)
        if causal:
            mask &= kpos[None, :] <= qpos[:, None]
        if window is not None:
            mask &= kpos[None, :] > qpos[:, None] - window
    mask = np.asarray(mask, dtype=bool)
    scores = np.where(mask[None], scores, -np.inf)
    with np.errstate(invalid="ignore", divide="ignore"):
        m = scores.max(axis=-1, keepdims=True)
        m = np.where(np.isfinite(m), m, 0.0)
        e = np.exp(scores - m)
        denom = e.sum(axis=-1, keepdims=True)
        p = np.where(denom > 0, e / np.where(denom > 0, denom, 1.0), 0.0)
        lse = (m[..., 0] + np.log(denom[..., 0])) / np.log(2.0)
    out = np.einsum("hqk,khd->qhd", p, v)
    return out, lse.T


def merge(o1, lse1, o2, lse2):
    """Merge two partial softmax states (base-2 lse).  float64 in, float64 out."""
    o1 = np.asarray(o1, dtype=np.float64)
    o2 = np.asarray(o2, dtype=np.float64)
    lse1 = np.asarray(lse1, dtype=np.float64)
    lse2 = np.asarray(lse2, dtype=np.float64)
    lse = np.logaddexp2(lse1, lse2)
    w1 = np.exp2(lse1 - lse)[..., None]
    w2 = np.exp2(lse2 - lse)[..., None]
    return o1 * w1 + o2 * w2, lse


def mla_expand(latent_kpe, w_kv, n_heads, d_nope, d_v):
    """latent_kpe: (L, d_latent + d_rope); w_kv: (d_latent, H*(d_nope+d_v)).

    Returns k (L, H, d_nope + d_rope), v (L, H, d_v) in float64, the un-absorbed form.
    """
    latent_kpe = np.asarray(latent_kpe, dtype=np.float64)
    d_latent = w_kv.shape[0]
    latent, k_pe = latent_kpe[:, :d_latent], latent_kpe[:, d_latent:]
    kv = (latent @ np.asarray(w_kv, dtype=np.float64)).reshape(latent.shape[0], n_heads, d_nope + d_v)
    k_nope, v = kv[..., :d_nope], kv[..., d_nope:]
    k = np.concatenate([k_nope, np.broadcast_to(k_pe[:, None, :], (latent.shape[0], n_heads, k_pe.shape[1]))], axis=-1)
    return k, v
