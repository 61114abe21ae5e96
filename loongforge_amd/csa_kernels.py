"""Compressed-sparse-attention (CSA) callers of the indexer and sparse-attention kernels.

Mirrors the pieces of loongforge/models/foundation/deepseek_v4/deepseek_v4_csa.py that sit directly
on the kernels: the fp8 indexer over *compressed* keys (`CSAIndexerKernel`, reference :1319-1561) and
the index helpers that encode its causal rule in id space (:221-268, :722-824).  A compressed key c
summarises the raw positions [c * ratio, (c + 1) * ratio) and becomes visible to a query at position
p once it is complete: c < (p + 1) // ratio.  The attention call itself is
`DSADotProductAttention` with `chunk_offset = kv.size(0)` (reference :2806-2816): the ids already
encode causality, so the kernel's own position test is switched off that way.
"""
from functools import lru_cache
from typing import Optional

import torch
from torch import Tensor

from . import ops
from .dsa_fused_kernels import _pad_to, _unscale_indexer_grad
from .megatron_compat import PackedSeqParams


# ---------------------------------------------------------------------------------------------------
# index helpers
# ---------------------------------------------------------------------------------------------------
def _segment_of_row(cu_seqlens: Tensor, rows: int) -> Tensor:
    """Segment index of each packed row; rows at or past cu_seqlens[-1] map to the last segment."""
    r = torch.arange(rows, device=cu_seqlens.device, dtype=cu_seqlens.dtype)
    seg = torch.searchsorted(cu_seqlens[1:].contiguous(), r, right=True)
    return seg.clamp(max=max(cu_seqlens.numel() - 2, 0))


@lru_cache(maxsize=8)
def _window_ids(window_size: int, seqlen: int, device_str: str) -> Tensor:
    pos = torch.arange(seqlen, device=device_str).unsqueeze(1)
    first = (pos - (window_size - 1)).clamp(min=0)
    ids = first + torch.arange(window_size, device=device_str)
    return torch.where(ids <= pos, ids, torch.full_like(ids, -1))


def get_window_topk_idxs(window_size: int, batch_size: int, seqlen: int, device) -> Tensor:
    """[batch, seqlen, window_size]: the last `window_size` positions up to the query's own,
    ascending from column 0, -1 after them (reference :221-241)."""
    return _window_ids(int(window_size), int(seqlen), str(device)).unsqueeze(0).expand(batch_size, -1, -1)


@lru_cache(maxsize=8)
def _compress_ids(ratio: int, seqlen: int, offset: int, device_str: str) -> Tensor:
    n = seqlen // ratio
    col = torch.arange(n, device=device_str).unsqueeze(0)
    visible = torch.div(torch.arange(1, seqlen + 1, device=device_str), ratio, rounding_mode="floor").unsqueeze(1)
    return torch.where(col < visible, col + offset, -1)


def get_compress_topk_idxs(ratio: int, batch_size: int, seqlen: int, offset: int, device) -> Tensor:
    """[batch, seqlen, seqlen // ratio]: every compressed key visible to the query, shifted by
    `offset` (the row of compressed key 0 in the concatenated key tensor); -1 for keys not yet
    complete (reference :244-268)."""
    return _compress_ids(int(ratio), int(seqlen), int(offset), str(device)).unsqueeze(0).expand(batch_size, -1, -1)


def get_window_topk_idxs_thd(window_size: int, cu_seqlens_q: Tensor, total_q: Optional[int] = None) -> Tensor:
    """Packed layout: `(total_q, window_size)` int32 ids local to the query's segment; rows past the
    last segment are all -1 (reference :722-756)."""
    if total_q is None:
        total_q = int(cu_seqlens_q[-1].item())
    seg = _segment_of_row(cu_seqlens_q, total_q)
    row = torch.arange(total_q, device=cu_seqlens_q.device, dtype=cu_seqlens_q.dtype)
    live = row < cu_seqlens_q[-1]
    pos = torch.where(live, row - cu_seqlens_q[seg], torch.zeros_like(row)).unsqueeze(1)
    ids = (pos - (window_size - 1)).clamp(min=0) + torch.arange(window_size, device=row.device, dtype=row.dtype)
    ids = torch.where((ids <= pos) & live.unsqueeze(1), ids, torch.full_like(ids, -1))
    return ids.int()


def get_compress_topk_idxs_thd(ratio: int, cu_seqlens_q: Tensor, cu_seqlens_kv: Tensor, cu_seqlens_compressed: Tensor,
                               total_q: Optional[int] = None, max_n_compressed: Optional[int] = None) -> Tensor:
    """Packed layout: `(total_q, max_n_compressed)` int32; column c of a query at segment position p
    holds `len_kv(segment) + c` while c < min((p + 1) // ratio, compressed keys of the segment), else
    -1: the ids address the segment's keys followed by its compressed keys (reference :759-824)."""
    if total_q is None:
        total_q = int(cu_seqlens_q[-1].item())
    device = cu_seqlens_q.device
    len_kv = cu_seqlens_kv[1:] - cu_seqlens_kv[:-1]
    len_c = cu_seqlens_compressed[1:] - cu_seqlens_compressed[:-1]
    if max_n_compressed is None:
        max_n_compressed = int(len_c.max().item()) if len_c.numel() else 0
    if max_n_compressed == 0:
        return torch.empty((total_q, 0), dtype=torch.int32, device=device)
    seg = _segment_of_row(cu_seqlens_q, total_q)
    row = torch.arange(total_q, device=device, dtype=cu_seqlens_q.dtype)
    live = row < cu_seqlens_q[-1]
    pos = torch.where(live, row - cu_seqlens_q[seg], torch.zeros_like(row))
    n_vis = torch.minimum(torch.div(pos + 1, ratio, rounding_mode="floor"), len_c[seg])
    n_vis = torch.where(live, n_vis, torch.zeros_like(n_vis)).unsqueeze(1)
    col = torch.arange(max_n_compressed, device=device, dtype=cu_seqlens_q.dtype).unsqueeze(0)
    ids = torch.where(col < n_vis, col + len_kv[seg].unsqueeze(1), -1)
    return ids.int()


# ---------------------------------------------------------------------------------------------------
# fp8 indexer over compressed keys
# ---------------------------------------------------------------------------------------------------
class CSAIndexerKernelFunction(torch.autograd.Function):
    """quantise -> windowed logits over the compressed keys -> top-k, with the sparse backward
    (reference :1319-1522).  `index_q [sq, 1, h, d]`, `index_k [sk, 1, d]`, `weights [sq, 1, h]`.

    Single sequence: query i (global position i + sq_offset) scores compressed keys
    [0, max((i + sq_offset + 1) // ratio, 1)); ids are rows of `index_k`.  Packed: the window is
    [cu_kv[seg], cu_kv[seg] + min((pos_in_seg + 1) // ratio, len_kv[seg])) and the returned ids are
    relative to cu_kv[seg].  In both forms slots without a visible key hold score -inf and id -1
    (the reference leaves arbitrary masked positions there in the single-sequence form), and the
    logits never leave the kernels' workspace.
    """

    @staticmethod
    def forward(ctx, index_q: Tensor, index_k: Tensor, weights: Tensor, index_topk: int, compress_ratio: int,
                sq_offset: int = 0, packed_seq_params: Optional[PackedSeqParams] = None):
        sq, bsz, head, dim = index_q.size()
        sk = index_k.size(0)
        assert bsz == 1, "CSAIndexerKernel only supports batch_size=1"
        assert dim == 128, "Only support dim=128"
        assert head <= 64, "the indexer kernel supports at most 64 heads"
        device = index_q.device
        softmax_scale = dim ** -0.5
        head_p = 32 if head <= 32 else 64

        q = _pad_to(index_q.squeeze(1).to(torch.bfloat16), head_p, 1).contiguous()
        k = index_k.squeeze(1).to(torch.bfloat16).contiguous()
        w = _pad_to(weights.squeeze(1).float(), head_p, 1)
        q_fp8, q_scale, weight_scaled = ops.quant_rowwise_e4m3_weights(q, w, softmax_scale)
        k_fp8, k_scale = ops.quant_rowwise_e4m3(k)

        row = torch.arange(sq, dtype=torch.int, device=device)
        if packed_seq_params is not None:
            cu_q = packed_seq_params.cu_seqlens_q_padded
            if cu_q is None:
                cu_q = packed_seq_params.cu_seqlens_q
            cu_kv = packed_seq_params.cu_seqlens_kv_padded
            if cu_kv is None:
                cu_kv = packed_seq_params.cu_seqlens_kv
            cu_q, cu_kv = cu_q.to(device).int(), cu_kv.to(device).int()
            seg = _segment_of_row(cu_q, sq)
            k_start = cu_kv[seg]
            visible = torch.div(row - cu_q[seg] + 1, compress_ratio, rounding_mode="floor")
            visible = torch.minimum(visible, (cu_kv[1:] - cu_kv[:-1])[seg])
            visible = torch.where(row < cu_q[-1], visible, torch.zeros_like(visible))
            k_end = k_start + visible
            effective_topk = min(index_topk, int(packed_seq_params.max_seqlen_kv))
        else:
            k_start = torch.zeros(sq, dtype=torch.int, device=device)
            k_end = torch.div(row + (sq_offset + 1), compress_ratio, rounding_mode="floor").clamp(min=1, max=sk)
            effective_topk = min(index_topk, sk)

        # the reference asks for unsorted output, i.e. any slot order will do: the descending-score path of the
        # top-k kernel is its fast one
        index_score_topk, global_ids = ops.indexer_topk(q_fp8, weight_scaled, k_fp8, k_scale, k_start.int(),
                                                        k_end.int(), effective_topk, True)
        if packed_seq_params is not None:
            topk_indices = torch.where(global_ids >= 0, global_ids - k_start.unsqueeze(1), global_ids)
        else:
            topk_indices = global_ids
        ctx.softmax_scale = softmax_scale
        ctx.head = head
        ctx.in_dtypes = (index_q.dtype, index_k.dtype, weights.dtype)
        ctx.save_for_backward(q_fp8, k_fp8, q_scale, k_scale, weight_scaled, global_ids)
        ctx.mark_non_differentiable(topk_indices)
        return index_score_topk, topk_indices

    @staticmethod
    def backward(ctx, grad_score, grad_topk):
        q_fp8, k_fp8, q_scale, k_scale, weight_scaled, global_ids = ctx.saved_tensors
        # padding slots are constants of the forward: their upstream gradient (often NaN) is dropped
        grad_score = torch.where(global_ids >= 0, grad_score.float(), torch.zeros_like(grad_score, dtype=torch.float32))
        d_q, d_k, d_weights = ops.indexer_bwd(grad_score.contiguous(), q_fp8, k_fp8, k_scale, weight_scaled, global_ids)
        d_weights = d_weights * q_scale * ctx.softmax_scale
        d_q = _unscale_indexer_grad(d_q, q_scale)
        d_k = _unscale_indexer_grad(d_k, k_scale)
        dq_t, dk_t, dw_t = ctx.in_dtypes
        return (d_q[:, :ctx.head].to(dq_t).unsqueeze(1), d_k.to(dk_t).unsqueeze(1),
                d_weights[:, :ctx.head].to(dw_t).unsqueeze(1), None, None, None, None)


class CSAIndexerKernel(torch.nn.Module):
    """`forward(index_q, index_k, weights, index_topk, sq_offset=0, packed_seq_params=None)` ->
    `(index_score_topk [sq, topk] fp32, topk_indices [sq, topk] int32)`; reference :1544-1561."""

    def __init__(self, compress_ratio: int):
        super().__init__()
        self.compress_ratio = compress_ratio

    def forward(self, index_q, index_k, weights, index_topk, sq_offset=0, packed_seq_params=None):
        return CSAIndexerKernelFunction.apply(index_q, index_k, weights, index_topk, self.compress_ratio, sq_offset,
                                              packed_seq_params)
