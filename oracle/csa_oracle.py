"""CPU restatement of the compressed-sparse-attention (CSA) index rules.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the
product (loongforge_amd/) never does.

The reference is loongforge/models/foundation/deepseek_v4/deepseek_v4_csa.py (cited per function);
it was read, not run (it imports Megatron, DeepGEMM and flashinfer, all absent here).  Everything
below is integer index arithmetic written as explicit loops over (query, slot).

Parity status
-------------
window_ids, compress_ids (+ packed variants)
        pinned by the rule they encode, checked in the tests from an independent statement of it:
        a query at position p of its segment sees the last `window` raw positions <= p, and the
        compressed key c (which summarises raw positions [c*ratio, (c+1)*ratio)) once its last
        position (c+1)*ratio - 1 <= p.
csa_indexer_window, csa_indexer_forward
        pinned: windows by the same rule (ke - ks == number of visible compressed keys; the
        single-sequence form keeps at least one key, deepseek_v4_csa.py:1460-1461); selection by
        torch.topk on the dense oracle logits (dsa_oracle.indexer_logits, itself pinned).
        unpinned: order of the selected slots (the reference asks flashinfer for unsorted output).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import dsa_oracle as O


def _segments(cu) -> list:
    cu = [int(v) for v in cu]
    return [(cu[b], cu[b + 1]) for b in range(len(cu) - 1)]


def window_ids(window: int, seqlen: int) -> torch.Tensor:
    """[seqlen, window]: the last `window` positions up to and including the query's, ascending,
    left-aligned, -1 after them (deepseek_v4_csa.py:221-231)."""
    out = torch.full((seqlen, window), -1, dtype=torch.int64)
    for i in range(seqlen):
        first = max(0, i - window + 1)
        for c, p in enumerate(range(first, i + 1)):
            out[i, c] = p
    return out


def compress_ids(ratio: int, seqlen: int, offset: int) -> torch.Tensor:
    """[seqlen, seqlen // ratio]: compressed keys visible to each query, shifted by `offset`
    (deepseek_v4_csa.py:244-256)."""
    n = seqlen // ratio
    out = torch.full((seqlen, n), -1, dtype=torch.int64)
    for i in range(seqlen):
        for c in range(n):
            if (c + 1) * ratio - 1 <= i:
                out[i, c] = c + offset
    return out


def window_ids_thd(window: int, cu_seqlens_q, total_q: int) -> torch.Tensor:
    """Packed form: positions are counted inside the query's own segment; rows past the last
    segment are all -1 (deepseek_v4_csa.py:722-756)."""
    out = torch.full((total_q, window), -1, dtype=torch.int32)
    for s, e in _segments(cu_seqlens_q):
        for t in range(s, min(e, total_q)):
            p = t - s
            first = max(0, p - window + 1)
            for c, v in enumerate(range(first, p + 1)):
                out[t, c] = v
    return out


def compress_ids_thd(ratio: int, cu_seqlens_q, cu_seqlens_kv, cu_seqlens_compressed, total_q: int,
                     max_n_compressed: int) -> torch.Tensor:
    """Packed form: column c of a query at segment position p is `len_kv(segment) + c` while the
    compressed key c exists in the segment and is complete at p (deepseek_v4_csa.py:759-824)."""
    out = torch.full((total_q, max_n_compressed), -1, dtype=torch.int32)
    seg_q, seg_kv, seg_c = _segments(cu_seqlens_q), _segments(cu_seqlens_kv), _segments(cu_seqlens_compressed)
    for (s, e), (ks, ke), (cs, ce) in zip(seg_q, seg_kv, seg_c):
        for t in range(s, min(e, total_q)):
            p = t - s
            for c in range(min(max_n_compressed, ce - cs)):
                if (c + 1) * ratio - 1 <= p:
                    out[t, c] = (ke - ks) + c
    return out


def csa_indexer_window(sq: int, ratio: int, sk: int, sq_offset: int = 0, cu_seqlens_q=None,
                       cu_seqlens_kv=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rows [ks, ke) of the compressed indexer keys each query scores
    (deepseek_v4_csa.py:1456-1461 single sequence; :1398-1425 packed)."""
    ks = torch.zeros(sq, dtype=torch.int32)
    ke = torch.zeros(sq, dtype=torch.int32)
    if cu_seqlens_q is None:
        for i in range(sq):
            ke[i] = min(max((i + sq_offset + 1) // ratio, 1), sk)
        return ks, ke
    for (s, e), (a, b) in zip(_segments(cu_seqlens_q), _segments(cu_seqlens_kv)):
        for t in range(s, min(e, sq)):
            ks[t] = a
            ke[t] = a + min((t - s + 1) // ratio, b - a)
    return ks, ke


def csa_indexer_forward(index_q, index_k, weights, index_topk: int, ratio: int, sq_offset: int = 0,
                        cu_seqlens_q=None, cu_seqlens_kv=None, max_seqlen_kv: Optional[int] = None):
    """Quantise -> window over compressed keys -> logits -> top-k (deepseek_v4_csa.py:1342-1484).
    index_q [sq, h, d], index_k [sk, d], weights [sq, h].  Packed: ids are relative to the first
    compressed key of the query's segment and -1 where fewer keys are visible (:1437-1446)."""
    d = index_q.shape[-1]
    sk = index_k.shape[0]
    q8, q_scale = O.quant_rowwise_e4m3(index_q)
    k8, k_scale = O.quant_rowwise_e4m3(index_k)
    ks, ke = csa_indexer_window(index_q.shape[0], ratio, sk, sq_offset, cu_seqlens_q, cu_seqlens_kv)
    weight_scaled = weights.float() * q_scale * (d ** -0.5)
    logits = O.indexer_logits(q8, weight_scaled, k8, k_scale, ks, ke)
    k_eff = min(index_topk, sk if cu_seqlens_q is None else int(max_seqlen_kv))
    scores, idx = O.topk_select(logits, k_eff)
    global_idx = idx
    if cu_seqlens_q is not None:
        idx = torch.where(idx >= 0, idx - ks[:, None], idx)
    return scores, idx, dict(q8=q8, k8=k8, q_scale=q_scale, k_scale=k_scale, weight_scaled=weight_scaled,
                             ks=ks, ke=ke, logits=logits, global_idx=global_idx)
