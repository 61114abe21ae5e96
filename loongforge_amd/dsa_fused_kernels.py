"""Kernel wrappers of the fused DSA path, with the reference's names and call signatures.

Drop-in counterparts of loongforge/models/common/experimental_attention_variant/dsa_fused_kernels.py
(``triton_attn_dist`` :1898, ``padded_flashinfer_topk`` :1958, ``DSADotProductAttentionFunction``
:2001, ``DSADotProductAttention`` :2115, ``DSAIndexerKernelFunction`` :2287, ``DSAIndexerKernel``
:2445), backed by the gfx950 HIP kernels instead of DeepGEMM / FlashInfer / FlashMLA / Triton.
"""
import os
from dataclasses import dataclass
from typing import Optional

import torch
from torch import Tensor

from . import ops
from .megatron_compat import AttnMaskType, MegatronModule, PackedSeqParams

_LOG2E = 1.44269504


def triton_attn_dist(p_out: torch.Tensor, sm_scale) -> torch.Tensor:
    """``output[s, :] = mean_h softmax(p_out[s, h, :] * sm_scale)``.

    Same contract as the reference function of this name (dsa_fused_kernels.py:1898-1955): input
    ``(s_q, h_q, topk)``, output ``(s_q, topk)`` in ``p_out.dtype``, softmax in fp32.  The slot count
    does not have to be a power of two here.
    """
    if p_out.ndim != 3:
        raise ValueError("p_out must be (s_q, h_q, topk)")
    return ops.attn_dist(p_out, float(sm_scale)).to(p_out.dtype)


def padded_flashinfer_topk(logits, topk, sk, *, sorted=True):
    """Top-k values and indices of the last dimension, padded when ``topk`` exceeds it.

    Reference: dsa_fused_kernels.py:1958-1998.  Values come back descending when ``sorted``; when
    ``topk > d`` the tail is filled with ``-inf`` / ``sk``.  Rows with fewer than ``topk`` finite
    entries return id ``-1`` for the ``-inf`` slots (the reference leaves arbitrary masked ids there,
    which its attention kernel rejects later; ``-1`` is rejected the same way).
    """
    d = logits.size(-1)
    topk = int(topk)
    lead = logits.shape[:-1]
    flat = logits.reshape(-1, d).float()
    k_eff = min(topk, d)
    vals, idx = ops.topk(flat, k_eff, sorted=sorted)
    if topk > d:
        pad = topk - d
        vals = torch.cat([vals, vals.new_full((vals.shape[0], pad), float("-inf"))], dim=-1)
        idx = torch.cat([idx, idx.new_full((idx.shape[0], pad), sk)], dim=-1)
    return vals.reshape(*lead, topk), idx.reshape(*lead, topk)


class DSADotProductAttentionFunction(torch.autograd.Function):
    """Sparse MLA attention over the selected latent rows (forward and backward on the HIP kernels).

    Same argument list as the reference (dsa_fused_kernels.py:2006-2021).  ``attn_sink`` ([h_q] or a
    divisor of it, expanded as at :2040-2046) adds a per-head sink term to the softmax denominator;
    ``topk_length`` ([s_q] int32) keeps only the first ``topk_length[i]`` slots of query ``i``.  No
    gradient is returned for ``attn_sink`` (the reference returns none either, :2112).
    ``window_size`` (DeepSeek-V4: the leading slots hold the sliding-window keys) leaves those slots
    out of ``p_out``, which is then [sq, n, topk - window_size]
    (loongforge/models/foundation/deepseek_v4/deepseek_v4_csa.py:2341-2346); attention runs over every
    slot.  As in the reference it is only accepted together with ``return_p_out`` (:2971-2974).
    ``dist_heads`` > 0 (not in the reference) returns, instead of the logits, what the training path
    makes of them: the head-averaged attention distribution over the slots, mean over the first
    ``dist_heads`` heads (dsa_fused.py:915-929): reduced from the logits when those are a small passing
    allocation (at most DSA_P_OUT_BUDGET_GIB, default 6, GiB), recomputed from q, kv and lse otherwise, so
    that no large [sq, n, topk] tensor is ever allocated.
    """

    @staticmethod
    def forward(ctx, q, kv, indices, chunk_offset=0, sm_scale=None, d_v=512, return_p_out=False,
                packed_seq_params=None, topk_length=None, attn_sink=None, window_size=0, fast_mode=False,
                dist_heads=0):
        window_size = int(window_size or 0)
        if dist_heads and (return_p_out or window_size):
            raise ValueError("dist_heads replaces return_p_out and does not take a window_size")
        if window_size and not return_p_out:
            raise ValueError("window_size > 0 needs return_p_out=True")
        if window_size % 32:
            raise NotImplementedError("window_size must be a multiple of 32, got %d" % window_size)
        # q [sq, n, d]; kv [skv, 1, d]; indices [sq, 1, topk]
        sq = q.size(0)
        kv2 = kv.reshape(kv.shape[0], kv.shape[-1])
        ids = indices.reshape(sq, indices.shape[-1])
        if topk_length is not None:
            slot = torch.arange(ids.shape[-1], device=ids.device)
            ids = torch.where(slot[None, :] < topk_length.reshape(sq, 1).to(ids.device), ids, torch.full_like(ids, -1))
        if attn_sink is not None:
            h_q = q.size(1)
            if attn_sink.numel() != h_q:
                attn_sink = attn_sink.flatten().repeat_interleave(h_q // attn_sink.numel())
            attn_sink = attn_sink.contiguous().view(h_q).float()
        # the head-averaged distribution comes from the forward's raw logits, which are a passing buffer of at most
        # DSA_P_OUT_BUDGET_GIB (default 6) GiB: all queries at once when they fit (forward + 0.9 ms, reduction 0.8 ms at
        # 8k tokens x 128 heads x 2048 slots: 4.3 GB), else a block of queries at a time (17 GB of logits at 32k tokens
        # never exist; recomputing the distribution from q, kv and lse instead costs 2.6 ms per 8k tokens)
        budget = float(os.environ.get("DSA_P_OUT_BUDGET_GIB", "6")) * 2 ** 30
        per_query = q.size(1) * ids.shape[-1] * 2
        dist = None
        if dist_heads and not return_p_out and sq * per_query > budget and budget >= 64 * per_query:
            out, lse, dist = ops.sparse_mla_fwd_dist(q, kv2, ids, chunk_offset, sm_scale, d_v, int(dist_heads),
                                                     int(budget // per_query) // 64 * 64, attn_sink)
            p_out = None
        else:
            dist_from_logits = bool(dist_heads) and sq * per_query <= budget
            out, lse, p_out = ops.sparse_mla_fwd(q, kv2, ids, chunk_offset, sm_scale, d_v, return_p_out or dist_from_logits,
                                                 attn_sink=attn_sink, p_out_skip=window_size)
        ctx.save_for_backward(q, kv, ids, out, lse)
        ctx.sm_scale = sm_scale
        ctx.chunk_offset = chunk_offset
        ctx.d_v = d_v
        out = out.unsqueeze(0)
        if return_p_out:
            ctx.mark_non_differentiable(p_out)
            return out, p_out
        if dist_heads:
            if dist is not None:
                pass
            elif dist_from_logits:
                dist = ops.attn_dist(p_out[:, :int(dist_heads)], sm_scale)
                del p_out
            else:
                dist = ops.attn_dist_qk(q, kv2, ids, lse, chunk_offset, sm_scale, int(dist_heads), attn_sink)
            ctx.mark_non_differentiable(dist)
            return out, dist
        return out

    @staticmethod
    def backward(ctx, grad_out, grad_p_out=None):
        q, kv, ids, out, lse = ctx.saved_tensors
        grad_out = grad_out.squeeze(0).contiguous()
        kv2 = kv.reshape(kv.shape[0], kv.shape[-1])
        grad_q, grad_kv = ops.sparse_mla_bwd(q, kv2, out, grad_out, ids, lse, ctx.chunk_offset, ctx.sm_scale, ctx.d_v)
        return (grad_q, grad_kv.reshape(kv.shape), None, None, None, None, None, None, None, None, None, None, None)


class DSADotProductAttention(MegatronModule):
    """Layout-normalising wrapper around the sparse attention kernel (dsa_fused_kernels.py:2115-2284)."""

    def __init__(self, config, softmax_scale: Optional[float] = None):
        super().__init__(config=config)
        self.config = config
        self.qkv_format: str = "sbhd"
        self.softmax_scale = softmax_scale

    def forward(self, query: Tensor, kv: Tensor, indices: Tensor, chunk_offset: int,
                attn_mask_type: AttnMaskType = None, attention_bias: Tensor = None,
                packed_seq_params: PackedSeqParams = None, return_p_out: bool = False, window_size: int = 0,
                topk_length: Optional[Tensor] = None, attn_sink: Optional[Tensor] = None,
                return_attn_dist: int = 0):
        # return_attn_dist = n > 0 (not in the reference's signature): also return the attention
        # distribution averaged over the first n heads, [sq, topk] fp32, without materialising p_out
        if attn_mask_type is None:
            attn_mask_type = AttnMaskType.causal
        assert attn_mask_type in (AttnMaskType.causal, AttnMaskType.padding_causal), (
            "DSADotProductAttention only support causal attention."
            "Please use TEDotProductAttention instead."
        )
        assert attention_bias is None, "Attention bias is not supported for DSADotProductAttention."
        assert self.config.qk_pos_emb_head_dim == 64, (
            f"DSADotProductAttention only support qk_pos_emb_head_dim 64, but got {self.config.qk_pos_emb_head_dim}."
        )
        qkv_format = self.qkv_format
        if getattr(self.config, "apply_rope_fusion", False):
            qkv_format = "bshd"
        if packed_seq_params is not None and getattr(packed_seq_params, "qkv_format", None):
            qkv_format = packed_seq_params.qkv_format

        if qkv_format == "bshd" and getattr(self.config, "apply_rope_fusion", False):
            query = query.transpose(0, 1).contiguous()
            kv = kv.unsqueeze(2).transpose(0, 1).contiguous()
        elif qkv_format == "thd":
            kv = kv.unsqueeze(1)
        else:  # sbhd: query [sq, b, n, d], kv [skv, b, d]
            query = query.transpose(0, 1).contiguous()
            kv = kv.unsqueeze(2).transpose(0, 1).contiguous()

        assert indices is not None, "DSADotProductAttention need topk_indices."
        indices = indices.unsqueeze(1) if qkv_format == "thd" else indices.unsqueeze(2)
        # the kernels take one sequence (or one packed batch) at a time
        if query.ndim == 4:
            assert query.size(0) == 1, "DSADotProductAttention does not support batched input"
            query = query.squeeze(0)
        if kv.ndim == 4:
            kv = kv.squeeze(0)
        # callers in thd mode hand [1, total_q, topk]; it is memory-identical to [total_q, 1, topk]
        indices = indices.reshape(-1, 1, indices.shape[-1])

        topk = indices.size(-1)
        topk_aligned = ((topk + 63) // 64) * 64
        if topk_aligned != topk:
            indices = torch.nn.functional.pad(indices, (0, topk_aligned - topk), value=-1)

        d_qk = query.size(-1)
        d_v = self.config.v_head_dim if d_qk == self.config.v_head_dim else self.config.kv_lora_rank

        res = DSADotProductAttentionFunction.apply(query, kv, indices, chunk_offset, self.softmax_scale, d_v,
                                                   return_p_out, packed_seq_params, topk_length, attn_sink,
                                                   window_size, True, int(return_attn_dist))
        core_attn_out, p_out = (res if (return_p_out or return_attn_dist) else (res, None))
        if qkv_format == "thd":
            core_attn_out = core_attn_out.squeeze(0).contiguous()
        else:
            core_attn_out = core_attn_out.contiguous()
        if return_p_out:
            return core_attn_out, p_out
        if return_attn_dist:
            return core_attn_out, p_out[:, :topk]
        return core_attn_out


def _unscale_indexer_grad(grad, scale_inv):
    """``grad / scale_inv`` with rows sitting on the quantiser's epsilon floor forced to zero
    (loongforge/models/foundation/deepseek_v4/deepseek_v4_csa.py:1525-1541)."""
    epsilon_scale_floor = 2.0 ** -48 * 1.5
    scale_inv = scale_inv.unsqueeze(-1)
    usable = torch.isfinite(scale_inv) & (scale_inv > epsilon_scale_floor)
    safe = torch.where(usable, scale_inv, torch.ones_like(scale_inv))
    return (grad / safe).masked_fill(~usable.expand_as(grad), 0.0)


_H128 = {}


def _hadamard128(device) -> Tensor:
    """Sylvester Hadamard matrix of order 128 in fp32 (cached per device)."""
    key = str(device)
    if key not in _H128:
        h = torch.ones(1, 1, dtype=torch.float32, device=device)
        while h.shape[0] < 128:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        _H128[key] = h
    return _H128[key]


def _pad_to(x: Tensor, size: int, dim: int) -> Tensor:
    if x.shape[dim] == size:
        return x
    pad = [0, 0] * (x.ndim - 1 - dim % x.ndim) + [0, size - x.shape[dim]]
    return torch.nn.functional.pad(x, pad)


class DSAIndexerKernelFunction(torch.autograd.Function):
    """fp8 lightning indexer: quantise -> windowed logits -> top-k, with the sparse backward.

    Reference: dsa_fused_kernels.py:2287-2442.  Differences that do not change results: the logits
    never leave the kernels' workspace, ids of rows with fewer than ``index_topk`` visible keys are
    ``-1`` instead of arbitrary masked positions, and head counts / head dims below the kernel's
    tile sizes are zero-padded (exact: padded heads carry zero weight, padded dims zero products).
    """

    sorted_output = True

    @staticmethod
    def forward(ctx, index_q: Tensor, index_k: Tensor, weights: Tensor, index_topk: int, chunk_offset: int,
                packed_seq_params: Optional[PackedSeqParams], rotate: bool = False, front: Optional["IndexerFrontEnd"] = None,
                k_norm_weight: Optional[Tensor] = None, k_norm_bias: Optional[Tensor] = None):
        assert index_q.ndim == 3 and index_k.ndim == 2 and weights.ndim == 2
        seq_q, head, dim = index_q.size()
        seq_k, _dim = index_k.size()
        assert dim == _dim, "Query and Key have diff dim."
        assert dim <= 128, "Only support dim with size 128."
        device = index_q.device
        softmax_scale = dim ** -0.5

        head_p = 32 if head <= 32 else 64
        assert head <= 64, "the indexer kernel supports at most 64 heads"
        q_p = _pad_to(_pad_to(index_q.to(torch.bfloat16), 128, 2), head_p, 1).contiguous()
        k_p = _pad_to(index_k.to(torch.bfloat16), 128, 1).contiguous()
        # rotate: the Hadamard rotation of the indexer front end is applied here, fused with the
        # quantiser (a zero-padded head dimension cannot be rotated after padding: 128 only)
        assert not rotate or dim == 128, "the fused rotation needs head dim 128"
        if front is None:
            quant = ops.rotate_quant_e4m3 if rotate else ops.quant_rowwise_e4m3
            # weight_scaled = weights * q_scale * softmax_scale comes out of the query's quantiser kernel
            q_fp8, q_scale, weight_scaled = ops.quant_rowwise_e4m3_weights(q_p, _pad_to(weights.float(), head_p, 1),
                                                                           softmax_scale, rotate)
            k_fp8, k_scale = quant(k_p)
        else:
            # index_q / index_k are the projections' outputs: key LayerNorm, rotary embedding and rotation
            # happen inside the quantiser kernel (a zero-padded head stays zero through all of them)
            assert dim == 128, "the fused front end needs head dim 128"
            q_fp8, q_scale, _, weight_scaled = ops.indexer_front_e4m3(
                q_p, head_p, None, None, 0.0, front.cos, front.sin, front.pairing, front.positions_q, front.batch, rotate,
                _pad_to(weights.float(), head_p, 1), softmax_scale)
            k_fp8, k_scale, _, _ = ops.indexer_front_e4m3(
                k_p, 1, k_norm_weight, k_norm_bias, front.k_norm_eps, front.cos, front.sin, front.pairing,
                front.positions_k, front.batch, rotate)

        if packed_seq_params is None:
            k_start = torch.zeros(seq_q, dtype=torch.int, device=device)
        else:
            cu = packed_seq_params.cu_seqlens_kv_padded
            if cu is None:
                cu = packed_seq_params.cu_seqlens_kv
            cu = cu.to(device)
            seqlens = cu[1:] - cu[:-1]
            full_seq_ids = torch.repeat_interleave(torch.arange(len(seqlens), device=device, dtype=torch.int), seqlens)
            local_seq_ids = full_seq_ids[chunk_offset:chunk_offset + seq_q]
            k_start = cu[local_seq_ids.long()].int()
        k_end = torch.arange(seq_q, dtype=torch.int, device=device) + chunk_offset + 1

        index_score_topk, topk_indices = ops.indexer_topk(q_fp8, weight_scaled, k_fp8, k_scale, k_start, k_end,
                                                          index_topk, DSAIndexerKernelFunction.sorted_output)
        ctx.softmax_scale = softmax_scale
        ctx.rotate = rotate
        ctx.index_topk = index_topk
        ctx.shape = (head, dim)
        ctx.in_dtypes = (index_q.dtype, index_k.dtype, weights.dtype)
        ctx.front = front
        if front is not None:
            ctx.front_saved = (k_p, k_norm_weight, k_norm_bias)
        ctx.save_for_backward(q_fp8, k_fp8, q_scale, k_scale, weight_scaled, topk_indices)
        ctx.mark_non_differentiable(topk_indices)
        return index_score_topk, topk_indices

    @staticmethod
    def backward(ctx, grad_score, grad_topk):
        q_fp8, k_fp8, q_scale, k_scale, weight_scaled, topk_indices = ctx.saved_tensors
        head, dim = ctx.shape
        grad_score = torch.where(topk_indices >= 0, grad_score.float(), torch.zeros_like(grad_score, dtype=torch.float32))
        d_q, d_k, d_weights = ops.indexer_bwd(grad_score.contiguous(), q_fp8, k_fp8, k_scale, weight_scaled,
                                              topk_indices.int())
        d_weights = d_weights * q_scale * ctx.softmax_scale
        d_q = _unscale_indexer_grad(d_q, q_scale)
        d_k = _unscale_indexer_grad(d_k, k_scale)
        if ctx.rotate:      # the rotation is symmetric and orthogonal up to its scale: its transpose is itself
            h = _hadamard128(d_q.device)
            d_q = (d_q @ h) * 128 ** -0.5
            d_k = (d_k @ h) * 128 ** -0.5
        dq_t, dk_t, dw_t = ctx.in_dtypes
        d_ln_w = d_ln_b = None
        front = ctx.front
        if front is not None:
            # back through the rotary embedding (its transpose, on bf16 gradients as the separate kernel's
            # backward sees them) and, on the key side, through the LayerNorm
            d_q, d_k = d_q.to(torch.bfloat16).contiguous(), d_k.to(torch.bfloat16).contiguous()
            _rope_q_rows(d_q, front.cos, front.sin, 0, 64, front.pairing, front.positions_q, front.batch, True)
            _rope_q_rows(d_k.unsqueeze(1), front.cos, front.sin, 0, 64, front.pairing, front.positions_k, front.batch, True)
            k_in, ln_w, ln_b = ctx.front_saved
            d_k, d_ln_w, d_ln_b = _layer_norm_backward(d_k.float(), k_in.float(), ln_w.float(), front.k_norm_eps)
            d_ln_w, d_ln_b = d_ln_w.to(ln_w.dtype), d_ln_b.to(ln_b.dtype)
        return (d_q[:, :head, :dim].to(dq_t), d_k[:, :dim].to(dk_t), d_weights[:, :head].to(dw_t), None, None, None,
                None, None, d_ln_w, d_ln_b)


def _layer_norm_backward(dy: Tensor, x: Tensor, weight: Tensor, eps: float):
    """Gradients of ``y = (x - mean) * rstd * weight + bias`` over the last dimension (fp32)."""
    mean = x.mean(-1, keepdim=True)
    xc = x - mean
    rstd = torch.rsqrt(xc.square().mean(-1, keepdim=True) + eps)
    xhat = xc * rstd
    d_w, d_b = (dy * xhat).sum(0), dy.sum(0)
    dxhat = dy * weight
    dx = rstd * (dxhat - dxhat.mean(-1, keepdim=True) - xhat * (dxhat * xhat).mean(-1, keepdim=True))
    return dx, d_w, d_b


@dataclass
class IndexerFrontEnd:
    """What ``DSAIndexerKernel(..., front=...)`` needs to run the indexer front end inside its quantiser kernels
    (dsa_fused.py:568-606 of the reference): the rotary tables ``[positions, 64]``, where a rotation pair sits
    (``ops.ROPE_ADJACENT`` / ``ops.ROPE_SPLIT``), the position of every query / key token (``None``: token //
    batch) and the key LayerNorm's epsilon (its weight and bias are passed as tensors so that they get gradients)."""

    cos: Tensor
    sin: Tensor
    pairing: int
    positions_q: Optional[Tensor] = None
    positions_k: Optional[Tensor] = None
    batch: int = 1
    k_norm_eps: float = 1e-5


class DSAIndexerKernel(torch.nn.Module):
    """``forward(index_q, index_k, weights, index_topk, chunk_offset, packed_seq_params)`` ->
    ``(index_score_topk [sq, topk] fp32, topk_indices [sq, topk] int32)``; reference
    dsa_fused_kernels.py:2445-2474.  ``rotate=True`` (an extension) applies the front end's Hadamard
    rotation to ``index_q`` / ``index_k`` inside the quantiser kernel instead of before the call."""

    supports_fused_rotate = True
    supports_fused_front_end = True

    def forward(self, index_q, index_k, weights, index_topk, chunk_offset, packed_seq_params, rotate=False,
                front=None, k_norm_weight=None, k_norm_bias=None):
        """``front`` (an extension, :class:`IndexerFrontEnd`): ``index_q`` / ``index_k`` are the outputs of the
        projections and the key LayerNorm (``k_norm_weight``, ``k_norm_bias``), the rotary embedding and the rotation
        run inside the quantiser kernels."""
        return DSAIndexerKernelFunction.apply(index_q, index_k, weights, index_topk, chunk_offset, packed_seq_params,
                                              rotate, front, k_norm_weight, k_norm_bias)


# ---------------------------------------------------------------------------------------------------
# MLA rotary embedding fused with permute / concatenate (reference: Triton kernels at
# dsa_fused_kernels.py:54-1841; here one HIP kernel parameterised by where a rotation pair sits)
# ---------------------------------------------------------------------------------------------------
def _token_positions(cu_seqlens, tokens, cp_rank, cp_size, offset=0):
    """None for sbhd (position = row // batch); for thd the position of each packed token in its own
    sequence (what megatron's ``_get_thd_token_idx`` returns for context-parallel size 1)."""
    if cu_seqlens is None:
        return None
    if cp_size not in (None, 1):
        raise NotImplementedError("context parallelism is not supported by this single-GPU build")
    return ops.thd_positions(cu_seqlens, tokens, offset)


def _rope_q_rows(t3, cos, sin, emb_offset, emb_dim, pairing, positions, batch, inverse):
    pe = t3[:, :, emb_offset: emb_offset + emb_dim]
    ops.rope_rows(pe, pe, cos, sin, pairing, pairing, inverse, positions, batch)


def _rope_q_forward(ctx, pairing, q, cos, sin, qk_head_dim, emb_dim, cu_seqlens_q, cp_rank, cp_size, emb_offset, sp_offset):
    if emb_offset is None:
        emb_offset = qk_head_dim
    if cu_seqlens_q is None:       # sbhd
        batch, nheads, headdim = q.shape[1], q.shape[2], q.shape[3]
        q3 = q.view(-1, nheads, headdim)
    else:                          # thd
        batch, headdim = 1, q.shape[2]
        q3 = q
    assert q3.stride(-1) == 1
    assert cos.is_contiguous() and sin.is_contiguous()
    assert headdim == qk_head_dim + emb_dim
    assert emb_dim % 4 == 0
    positions = _token_positions(cu_seqlens_q, q3.shape[0], cp_rank, cp_size, sp_offset)
    _rope_q_rows(q3, cos, sin, emb_offset, emb_dim, pairing, positions, batch, False)
    ctx.mark_dirty(q)
    ctx.save_for_backward(cos, sin)
    ctx.args = (emb_offset, emb_dim, positions, batch)
    return q


def _rope_q_backward(ctx, pairing, grad):
    cos, sin = ctx.saved_tensors
    emb_offset, emb_dim, positions, batch = ctx.args
    grad = grad.contiguous()
    _rope_q_rows(grad.view(-1, grad.shape[-2], grad.shape[-1]), cos, sin, emb_offset, emb_dim, pairing, positions, batch, True)
    return grad, None, None, None, None, None, None, None, None, None


class ApplyMLARotaryEmbQInterleaved(torch.autograd.Function):
    """Interleaved rotary embedding of MLA's query, in place (reference: dsa_fused_kernels.py:230-349):
    pairs are (x[2i], x[2i+1]) and stay where they are."""

    @staticmethod
    def forward(ctx, q, cos, sin, qk_head_dim, emb_dim, cu_seqlens_q, cp_rank, cp_size, emb_offset=None, sp_offset=0):
        return _rope_q_forward(ctx, ops.ROPE_ADJACENT, q, cos, sin, qk_head_dim, emb_dim, cu_seqlens_q, cp_rank, cp_size,
                               emb_offset, sp_offset)

    @staticmethod
    def backward(ctx, grad):
        return _rope_q_backward(ctx, ops.ROPE_ADJACENT, grad)


class ApplyMLARotaryEmbQNonInterleavedWithOffset(torch.autograd.Function):
    """Rotary embedding of MLA's query with pairs (x[i], x[i + emb_dim/2]), in place
    (reference: dsa_fused_kernels.py:501-603)."""

    @staticmethod
    def forward(ctx, q, cos, sin, qk_head_dim, emb_dim, cu_seqlens_q, cp_rank, cp_size, emb_offset=None, sp_offset=0):
        return _rope_q_forward(ctx, ops.ROPE_SPLIT, q, cos, sin, qk_head_dim, emb_dim, cu_seqlens_q, cp_rank, cp_size,
                               emb_offset, sp_offset)

    @staticmethod
    def backward(ctx, grad):
        return _rope_q_backward(ctx, ops.ROPE_SPLIT, grad)


def fused_apply_mla_rope(t, cos, sin, qk_head_dim: int, emb_dim: int, cu_seqlens_q=None, cp_rank: int = 0,
                         cp_size: int = 1, rotary_interleaved: bool = False, pe_first: bool = False, sp_offset: int = 0):
    """Rotary embedding of MLA's query, modifying ``t`` in place (reference: dsa_fused_kernels.py:1168-1212).

    ``t``: [seq, batch, heads, qk_head_dim + emb_dim] or packed [tokens, heads, ...]; cos / sin
    [max_seq_len, 1, 1, emb_dim]; ``pe_first`` puts the rotary columns at the front of a head.
    """
    emb_offset = 0 if pe_first else qk_head_dim
    fn = ApplyMLARotaryEmbQInterleaved if rotary_interleaved else ApplyMLARotaryEmbQNonInterleavedWithOffset
    return fn.apply(t, cos, sin, qk_head_dim, emb_dim, cu_seqlens_q, cp_rank, cp_size, emb_offset, sp_offset)


class FusedRopePermuteCat(torch.autograd.Function):
    """``query[s, b, h, :] = cat(q_content[h, s*b, :], rope(q_pos_emb[s, b, h, :]))`` in one pass
    (reference: dsa_fused_kernels.py:1010-1131).  The rotary input pairs are adjacent elements; the
    output keeps them adjacent (interleaved) or splits them into halves (non-interleaved)."""

    @staticmethod
    def forward(ctx, q_content, q_pos_emb, cos, sin, cu_seqlens_q, cp_rank, cp_size, rotary_interleaved=False):
        if q_pos_emb.ndim == 4:
            s, b, nheads, emb_dim = q_pos_emb.shape
            S = s * b
        else:
            S, nheads, emb_dim = q_pos_emb.shape
            s, b = S, 1
        d_out = q_content.shape[-1]
        qc = q_content.reshape(nheads, S, d_out)
        pe = q_pos_emb.reshape(S, nheads, emb_dim)
        out = q_content.new_empty(S, nheads, d_out + emb_dim)
        positions = _token_positions(cu_seqlens_q, S, cp_rank, cp_size)
        out_pairing = ops.ROPE_ADJACENT if rotary_interleaved else ops.ROPE_SPLIT
        ops.rope_rows(pe, out[:, :, d_out:], cos, sin, ops.ROPE_ADJACENT, out_pairing, False, positions, b,
                      main_src=qc.transpose(0, 1), main_dst=out[:, :, :d_out])
        ctx.save_for_backward(cos, sin)
        ctx.args = (s, b, nheads, d_out, emb_dim, positions, out_pairing, q_content.shape, q_pos_emb.ndim)
        return out.view(s, b, nheads, d_out + emb_dim) if q_pos_emb.ndim == 4 else out

    @staticmethod
    def backward(ctx, grad_output):
        cos, sin = ctx.saved_tensors
        s, b, nheads, d_out, emb_dim, positions, out_pairing, qc_shape, pe_ndim = ctx.args
        S = s * b
        g = grad_output.reshape(S, nheads, d_out + emb_dim).contiguous()
        grad_qc = g.new_empty(nheads, S, d_out)
        grad_pe = g.new_empty(S, nheads, emb_dim)
        ops.rope_rows(g[:, :, d_out:], grad_pe, cos, sin, out_pairing, ops.ROPE_ADJACENT, True, positions, b,
                      main_src=g[:, :, :d_out], main_dst=grad_qc.transpose(0, 1))
        grad_qc = grad_qc.view(qc_shape)
        if pe_ndim == 4:
            grad_pe = grad_pe.view(s, b, nheads, emb_dim)
        return grad_qc, grad_pe, None, None, None, None, None, None


def fused_rope_permute_cat(q_content, q_pos_emb, cos, sin, cu_seqlens_q=None, cp_rank: int = 0, cp_size: int = 1,
                           rotary_interleaved: bool = False):
    """Permute ``q_content`` (HSD -> SBHD), apply the rotary embedding to ``q_pos_emb`` and concatenate
    (reference: dsa_fused_kernels.py:1134-1165)."""
    return FusedRopePermuteCat.apply(q_content, q_pos_emb, cos, sin, cu_seqlens_q, cp_rank, cp_size, rotary_interleaved)


class ApplyMLARotaryEmbAbsorbKV(torch.autograd.Function):
    """``key[t, h, :] = cat(kv[t, h, :k_dim], rope(k_pos_emb[t, :]))``: the shared rotary part of the
    key is rotated once per token and broadcast to every head (reference: dsa_fused_kernels.py:1610-1793)."""

    @staticmethod
    def forward(ctx, kv, k_pos_emb, cos, sin, emb_dim, k_dim, cu_seqlens_kv, cp_rank, cp_size, rotary_interleaved=False):
        if cu_seqlens_kv is None:
            max_seqlen, batch, nheads, headdim = kv.shape
            kv3 = kv.view(-1, nheads, headdim)
        else:
            max_seqlen, batch = None, 1
            kv3 = kv
            nheads, headdim = kv.shape[1], kv.shape[2]
        T = kv3.shape[0]
        emb2 = k_pos_emb.reshape(T, emb_dim)
        assert headdim == k_dim
        assert kv3.stride(-1) == 1 and emb2.stride(-1) == 1
        assert cos.is_contiguous() and sin.is_contiguous()
        assert emb_dim % 4 == 0
        o_key = kv.new_empty(T, nheads, emb_dim + k_dim)
        positions = _token_positions(cu_seqlens_kv, T, cp_rank, cp_size)
        out_pairing = ops.ROPE_ADJACENT if rotary_interleaved else ops.ROPE_SPLIT
        ops.rope_rows(emb2.unsqueeze(1).expand(T, nheads, emb_dim), o_key[:, :, k_dim:], cos, sin, ops.ROPE_ADJACENT,
                      out_pairing, False, positions, batch, main_src=kv3, main_dst=o_key[:, :, :k_dim])
        ctx.save_for_backward(cos, sin)
        ctx.args = (emb_dim, k_dim, positions, batch, out_pairing, max_seqlen)
        if cu_seqlens_kv is None:
            o_key = o_key.view(max_seqlen, -1, nheads, emb_dim + k_dim)
        return o_key

    @staticmethod
    def backward(ctx, dk):
        cos, sin = ctx.saved_tensors
        emb_dim, k_dim, positions, batch, out_pairing, max_seqlen = ctx.args
        nheads = dk.shape[-2]
        dk3 = dk.contiguous().view(-1, nheads, emb_dim + k_dim)
        T = dk3.shape[0]
        d_kv = dk3.new_empty(T, nheads, k_dim)
        ops.rope_rows(None, None, None, None, 0, 0, main_src=dk3[:, :, :k_dim], main_dst=d_kv)
        d_emb = ops.rope_headsum_inverse(dk3[:, :, k_dim:], cos, sin, out_pairing, positions, batch).view(T, 1, emb_dim)
        if max_seqlen is not None:
            d_kv = d_kv.view(max_seqlen, batch, nheads, k_dim)
            d_emb = d_emb.view(max_seqlen, batch, 1, emb_dim)
        return d_kv, d_emb, None, None, None, None, None, None, None, None


class FusedAbsorbRopeQuery(torch.autograd.Function):
    """The attention query of the absorbed MLA form in one pass over the up-projected query
    ``q_up [s, (b,) h, 128 + 64]``:  ``query[..., :512] = q_up[..., :128] @ W_UK[h]`` (the key up-projection
    absorbed into the query, multi_latent_attention.py:1177-1194 of the reference) and ``query[..., 512:] =
    rope(q_up[..., 128:])`` (its fused_rope_permute_cat, :1196-1204), both written straight into the
    ``[.., h, 576]`` rows the attention kernel reads: no q_content tensor in head-major layout, no permute, no
    concatenation.  ``w_uk_t`` is W_UK as ``[h, 512, 128]``."""

    @staticmethod
    def forward(ctx, q_up, w_uk_t, cos, sin, cu_seqlens_q, cp_rank, cp_size, rotary_interleaved=False):
        lead = q_up.shape[:-2]
        nheads, width = q_up.shape[-2], q_up.shape[-1]
        d_nope, d_out, emb = w_uk_t.shape[2], w_uk_t.shape[1], width - w_uk_t.shape[2]
        batch = q_up.shape[1] if q_up.ndim == 4 else 1
        q3 = q_up.reshape(-1, nheads, width)
        S = q3.shape[0]
        query = q_up.new_empty(S, nheads, d_out + emb)
        positions = _token_positions(cu_seqlens_q, S, cp_rank, cp_size)
        out_pairing = ops.ROPE_ADJACENT if rotary_interleaved else ops.ROPE_SPLIT
        ops.mla_absorb_into(q3[:, :, :d_nope], w_uk_t, query[:, :, :d_out])
        ops.rope_rows(q3[:, :, d_nope:], query[:, :, d_out:], cos, sin, ops.ROPE_ADJACENT, out_pairing, False, positions, batch)
        ctx.save_for_backward(q3, w_uk_t, cos, sin)
        ctx.args = (positions, batch, out_pairing, d_nope, d_out, emb, q_up.shape)
        return query.view(*lead, nheads, d_out + emb)

    @staticmethod
    def backward(ctx, grad):
        q3, w_uk_t, cos, sin = ctx.saved_tensors
        positions, batch, out_pairing, d_nope, d_out, emb, shape = ctx.args
        g3 = grad.reshape(-1, grad.shape[-2], grad.shape[-1])
        d_up = torch.empty_like(q3)
        g_c = g3[:, :, :d_out].transpose(0, 1)                                   # [h, S, 512]
        d_up[:, :, :d_nope] = torch.bmm(g_c, w_uk_t).transpose(0, 1)
        ops.rope_rows(g3[:, :, d_out:], d_up[:, :, d_nope:], cos, sin, out_pairing, ops.ROPE_ADJACENT, True, positions, batch)
        d_w = torch.bmm(g_c.transpose(1, 2), q3[:, :, :d_nope].transpose(0, 1)) if ctx.needs_input_grad[1] else None
        return d_up.view(shape), d_w, None, None, None, None, None, None


def fused_absorb_rope_query(q_up, w_uk_t, cos, sin, cu_seqlens_q=None, cp_rank: int = 0, cp_size: int = 1,
                            rotary_interleaved: bool = False):
    """``[.., h, 192]`` up-projected query -> ``[.., h, 576]`` attention query (see :class:`FusedAbsorbRopeQuery`)."""
    return FusedAbsorbRopeQuery.apply(q_up, w_uk_t, cos, sin, cu_seqlens_q, cp_rank, cp_size, rotary_interleaved)


def absorb_attention_output(core_attn_out, w_uv):
    """``[.., h, 512]`` attention output -> ``[.., h * 128]``: the value up-projection applied per head
    (multi_latent_attention.py:955-975 of the reference: einsum("...hk,hdk->...hd") then flatten), read from
    the attention kernel's own layout and written in the layout the output projection reads."""
    lead, nheads = core_attn_out.shape[:-2], core_attn_out.shape[-2]
    o3 = core_attn_out.reshape(-1, nheads, core_attn_out.shape[-1])
    return ops.mla_absorb(o3, w_uv).reshape(*lead, nheads * w_uv.shape[1])


def fused_apply_mla_rope_for_absorb_kv(kv, k_pos_emb, cos, sin, emb_dim: int, k_dim: int, cu_seqlens_kv=None,
                                       cp_rank: int = 0, cp_size: int = 1, rotary_interleaved: bool = False):
    """Key rows of the absorbed MLA form: copy of ``kv`` plus the rotated, head-shared ``k_pos_emb``
    (reference: dsa_fused_kernels.py:1796-1841)."""
    return ApplyMLARotaryEmbAbsorbKV.apply(kv, k_pos_emb, cos, sin, emb_dim, k_dim, cu_seqlens_kv, cp_rank, cp_size,
                                           rotary_interleaved)
