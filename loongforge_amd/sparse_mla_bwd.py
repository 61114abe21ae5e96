"""``sparse_mla_bwd_interface`` with the reference's signature
(loongforge/models/common/experimental_attention_variant/sparse_mla_bwd.py:405-498), backed by the
deterministic gfx950 backward kernels."""
import torch

from . import ops


def sparse_mla_bwd_interface(q, kv, o, do, indices, lse, offsets, chunk_offset, sm_scale=None, is_casual=True,
                             return_kernel=False, delta=None):
    """dQ and dKV of sparse MLA attention.

    q ``[S, H, 576]``, kv ``[S_kv, 1, 576]``, o / do ``[S, H, 512]``, indices ``[S, 1, topk]`` int32,
    lse ``[S, H]`` natural log, offsets ``[0, S]`` (a single sequence, as the reference's caller
    passes), chunk_offset = global position of query 0.  ``delta`` is recomputed from ``o`` and
    ``do`` inside the kernel and ignored when given.  Returns ``(dq [S,H,576], dkv [S_kv,1,576])``.
    """
    assert is_casual, "non-casual is not supported now"
    assert not return_kernel, "there is no JIT kernel object to return in this build"
    assert q.is_contiguous()
    assert kv.is_contiguous()
    assert indices.is_contiguous()
    assert lse.is_contiguous()
    S, H, dim_plus_tail_dim = q.shape
    S_kv, kv_group, _ = kv.shape
    assert kv.shape[-1] == dim_plus_tail_dim
    assert kv_group == 1, "one shared latent KV head"
    topk = indices.shape[-1]
    assert indices.shape == (S, kv_group, topk)
    assert lse.shape == (S, H)
    if offsets is not None:
        assert offsets.numel() == 2, "packed batches go through chunk_offset and global ids, not offsets"
    if sm_scale is None:
        sm_scale = dim_plus_tail_dim ** (-0.5)
    dq, dkv = ops.sparse_mla_bwd(q, kv.reshape(S_kv, dim_plus_tail_dim), o, do, indices.reshape(S, topk), lse,
                                 int(chunk_offset), float(sm_scale), 512)
    return dq, dkv.reshape(S_kv, 1, dim_plus_tail_dim)
