"""CPU oracle for the fused DeepSeek-Sparse-Attention path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain PyTorch on the CPU, the arithmetic of the reference's fused DSA
path.  It is the checker the HIP kernels are compared against; nothing in the shipped package
imports it, and it must never be used as a fallback for a missing kernel.  Only the test-suite,
the smoke entry and the benchmark's CPU-baseline leg may import it.

Every function cites the reference text it follows (paths relative to the reference tree).
The reference's own implementation of this path cannot be imported here (its arithmetic lives in
closed or absent wheels: deep_gemm, flashinfer, flash_mla_fwd/bwd, lightning_indexer_bwd,
TransformerEngine, tilelang), so each function below is pinned by independent checks in
``tests/test_oracle_*.py`` (library routines such as SDPA / torch.topk / F.kl_div, brute-force
loops, closed forms and invariants).

Parity status per function
--------------------------
quant_rowwise_e4m3      pinned: closed form + constants quoted in the reference docstring
                        (zero row -> 2**-48, amax in (3.5, 7] -> 2**-6) + torch's e4m3 RNE cast.
indexer_logits          pinned: brute-force fp64 loops; exact integer special case; linearity.
topk_select             pinned: torch.sort brute force + set invariants.
                        unpinned detail: tie-breaking / output order of flashinfer.top_k
                        (closed wheel); order inside a row is not part of the contract.
sparse_mla_fwd          pinned: equals dense causal MQA (SDPA) when top-k covers the prefix;
                        brute-force fp64 loops in the general case; invariants.
                        attn_sink: the sink softmax written out as loops after the open torch
                        text at deepseek_v4_csa.py:571-579, plus the sink-share identity.
                        unpinned detail: p_out dtype / fill value of the closed flash_mla_fwd.
sparse_mla_bwd          pinned: torch.autograd through the forward restatement, gradcheck in
                        fp64, dense-attention gradients (SDPA autograd) in the covering case;
                        finite differences with a sink.
attn_dist, indexer_kl_loss   pinned: closed forms, F.kl_div, analytic special cases.
attn_dist_from_lse      pinned: equals attn_dist on the forward's logits (softmax = exp(z - logsumexp)).
indexer_bwd             pinned: autograd through the gathered logits; finite differences.
                        unpinned detail: duplicate / out-of-window id handling of the closed
                        lightning_indexer_bwd wheel.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

FP8_MAX = 448.0
NEG_INF = float("-inf")


# --------------------------------------------------------------------------------------------
# a2. Row-wise FP8 quantiser
# --------------------------------------------------------------------------------------------
def quant_rowwise_e4m3(
    x: torch.Tensor, eps: float = 1e-12, pow2: bool = True
) -> Tuple[torch.Tensor, torch.Tensor]:
    """1x128-block (one block per row here) e4m3 quantisation with power-of-two scales.

    Follows the quantiser configured at
    loongforge/models/common/experimental_attention_variant/dsa_fused_kernels.py:2308-2315
    (``amax_epsilon=1e-12, force_pow_2_scales=True``) and used at :2341-2346; the constants are
    confirmed by loongforge/models/foundation/deepseek_v4/deepseek_v4_csa.py:1528-1534.

    Returns ``(x8, scale_inv)`` with ``x8`` float8_e4m3fn of x's shape and ``scale_inv`` fp32 of
    shape ``x.shape[:-1]`` such that ``x ~= x8 * scale_inv``.
    """
    xf = x.float()
    amax = xf.abs().amax(dim=-1).clamp_min(eps)
    if pow2:
        # scale = 2 ** floor(log2(448 / amax)); frexp keeps this exact for every fp32 input
        ratio = (FP8_MAX / amax.double())
        mant, expo = torch.frexp(ratio)          # ratio = mant * 2**expo, mant in [0.5, 1)
        scale = torch.ldexp(torch.ones_like(ratio), expo - 1)
    else:
        scale = (FP8_MAX / amax.double())
    scale = scale.float()
    y = (xf * scale.unsqueeze(-1)).clamp(-FP8_MAX, FP8_MAX)
    x8 = y.to(torch.float8_e4m3fn)
    scale_inv = (1.0 / scale.double()).float()
    return x8, scale_inv


# --------------------------------------------------------------------------------------------
# a1/a3. Indexer window + logits
# --------------------------------------------------------------------------------------------
def indexer_window(
    sq: int, chunk_offset: int = 0, cu_seqlens: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Visible key window ``[ks_i, ke_i)`` of every local query.

    dsa_fused_kernels.py:2348-2360 -- ``ke = arange(sq) + chunk_offset + 1``; ``ks = 0`` for a
    single sequence, else the start of the document containing the query's global position
    (``repeat_interleave`` over ``cu_seqlens_kv``).
    """
    pos = torch.arange(sq, dtype=torch.int64) + int(chunk_offset)
    ke = (pos + 1).to(torch.int32)
    if cu_seqlens is None:
        ks = torch.zeros(sq, dtype=torch.int32)
    else:
        cu = cu_seqlens.to(torch.int64)
        lens = cu[1:] - cu[:-1]
        doc = torch.repeat_interleave(torch.arange(len(lens)), lens)
        ks = cu[doc[pos]].to(torch.int32)
    return ks, ke


def indexer_logits(
    q8: torch.Tensor,        # [sq, h, d]  float8 / any float holding the fp8 payload
    weight_scaled: torch.Tensor,  # [sq, h]  = weights * q_scale * d**-0.5
    k8: torch.Tensor,        # [sk, d]
    k_scale: torch.Tensor,   # [sk]
    ks: torch.Tensor,
    ke: torch.Tensor,
    dtype: torch.dtype = torch.float32,
    chunk: int = 256,
) -> torch.Tensor:
    """``L[i,j] = k_scale[j] * sum_h w'[i,h] * relu(q8[i,h,:] . k8[j,:])``; -inf outside the window.

    Math of deep_gemm.fp8_mqa_logits as called at dsa_fused_kernels.py:2362-2380; readable
    definition: ops/tilelang_ops/lightning_indexer.py:12-32 (einsum -> relu -> * q_s -> sum over
    heads -> * k_s).  Returns the dense ``[sq, sk]`` matrix (small shapes only).
    """
    sq, h, d = q8.shape
    sk = k8.shape[0]
    qf, kf = q8.to(dtype), k8.to(dtype)
    w = weight_scaled.to(dtype)
    out = torch.empty(sq, sk, dtype=dtype)
    cols = torch.arange(sk)
    for s in range(0, sq, chunk):
        e = min(sq, s + chunk)
        logits = torch.einsum("mhd,nd->mhn", qf[s:e], kf)
        logits = torch.relu(logits) * w[s:e].unsqueeze(-1)
        acc = logits.sum(dim=1) * k_scale.to(dtype).unsqueeze(0)
        vis = (cols[None, :] >= ks[s:e, None]) & (cols[None, :] < ke[s:e, None])
        out[s:e] = acc.masked_fill(~vis, NEG_INF)
    return out


# --------------------------------------------------------------------------------------------
# a4. Top-k
# --------------------------------------------------------------------------------------------
def topk_select(logits: torch.Tensor, topk: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row top-``topk`` by value, descending; rows with fewer finite entries are padded.

    dsa_fused_kernels.py:1958-1998 (``padded_flashinfer_topk``) + :2382-2387.  This build's
    contract pads with score ``-inf`` / id ``-1`` where the reference leaves ids of ``-inf``
    entries (which its attention kernel later rejects); the *valid* sets are the contract.
    """
    sq, width = logits.shape
    k_eff = min(topk, width)
    vals, idx = torch.topk(logits, k_eff, dim=-1, largest=True, sorted=True)
    if k_eff < topk:
        vals = torch.cat([vals, vals.new_full((sq, topk - k_eff), NEG_INF)], dim=-1)
        idx = torch.cat([idx, idx.new_full((sq, topk - k_eff), -1)], dim=-1)
    idx = torch.where(vals == NEG_INF, torch.full_like(idx, -1), idx)
    return vals, idx.to(torch.int32)


def indexer_forward(
    index_q: torch.Tensor,   # [sq, h, d] bf16
    index_k: torch.Tensor,   # [sk, d]   bf16
    weights: torch.Tensor,   # [sq, h]
    index_topk: int,
    chunk_offset: int = 0,
    cu_seqlens: Optional[torch.Tensor] = None,
    dtype: torch.dtype = torch.float32,
):
    """Quantise -> window -> logits -> top-k (``DSAIndexerKernelFunction.forward``,
    dsa_fused_kernels.py:2318-2393).  Returned ids are global key rows."""
    d = index_q.shape[-1]
    q8, q_scale = quant_rowwise_e4m3(index_q)
    k8, k_scale = quant_rowwise_e4m3(index_k)
    ks, ke = indexer_window(index_q.shape[0], chunk_offset, cu_seqlens)
    weight_scaled = weights.float() * q_scale * (d ** -0.5)
    logits = indexer_logits(q8, weight_scaled, k8, k_scale, ks, ke, dtype=dtype)
    scores, idx = topk_select(logits, index_topk)
    return scores, idx, dict(q8=q8, k8=k8, q_scale=q_scale, k_scale=k_scale,
                             weight_scaled=weight_scaled, ks=ks, ke=ke, logits=logits)


def gathered_indexer_logits(q8, weight_scaled, k8, k_scale, idx, dtype=torch.float32, chunk=256):
    """Logits of the *selected* pairs only: ``out[i,t] = L[i, idx[i,t]]`` (-inf where idx < 0).

    Gather formulation as in deepseek_v4_csa.py:636-649; used for the indexer backward
    (dsa_fused_kernels.py:2419-2442) which differentiates w.r.t. the fp8 payloads, the scaled
    weights and nothing else (scales are constants).
    """
    sq, h, d = q8.shape
    valid = idx >= 0
    safe = idx.clamp(min=0).long()
    outs = []
    for s in range(0, sq, chunk):
        e = min(sq, s + chunk)
        ksel = k8.to(dtype)[safe[s:e]]                       # [c, K, d]
        sc = torch.einsum("mhd,mkd->mhk", q8[s:e].to(dtype), ksel)
        sc = torch.relu(sc) * weight_scaled[s:e].to(dtype).unsqueeze(-1)
        outs.append(sc.sum(dim=1) * k_scale.to(dtype)[safe[s:e]])
    out = torch.cat(outs)
    return out.masked_fill(~valid, NEG_INF)


# --------------------------------------------------------------------------------------------
# a7. Sparse MLA forward
# --------------------------------------------------------------------------------------------
def sparse_mla_valid(idx: torch.Tensor, s_kv: int, q_start: int) -> torch.Tensor:
    """Slot validity: ``idx != -1  and  0 <= idx < s_kv  and  idx <= q_start + i``.

    ops/tilelang_ops/sparse_mla_fwd.py:129-132 (mask) and the contract quoted at
    dsa_fused_kernels.py:2051 ("invalid indices should be set to -1 or numbers >= s_kv").
    """
    sq = idx.shape[0]
    pos = torch.arange(sq, dtype=torch.int64, device=idx.device).unsqueeze(-1) + int(q_start)
    i64 = idx.to(torch.int64)
    return (i64 >= 0) & (i64 < s_kv) & (i64 <= pos)


def sparse_mla_fwd(
    q: torch.Tensor,      # [sq, h, dqk]
    kv: torch.Tensor,     # [skv, dqk]
    idx: torch.Tensor,    # [sq, K] int
    q_start: int = 0,
    sm_scale: Optional[float] = None,
    d_v: int = 512,
    dtype: torch.dtype = torch.float32,
    chunk: int = 64,
    attn_sink: Optional[torch.Tensor] = None,   # [h] per-head sink logit
):
    """Gather formulation of sparse MQA-MLA attention.

    Math: ops/tilelang_ops/sparse_mla_fwd.py:129-180 (kernel) and :218-265 (dense-mask torch
    reference); gather restatement as in deepseek_v4_csa.py:506-592 without the sink term.
    Returns ``out [sq,h,d_v]``, natural-log ``lse [sq,h]`` (+inf for rows without a valid slot,
    whose ``out`` is 0) and ``p_out [sq,h,K]`` = raw (unscaled) logits, -inf on invalid slots
    (consumer applies ``* sm_scale`` and softmax: dsa_fused_kernels.py:1884-1890).
    ``attn_sink``: the denominator gains ``exp(attn_sink[h])`` (deepseek_v4_csa.py:571-579): the
    sink is one more logit without a value row, so ``lse`` includes it and an empty row has
    ``lse = attn_sink`` and ``out = 0``.
    Differentiable in q and kv.
    """
    sq, h, dqk = q.shape
    skv = kv.shape[0]
    if sm_scale is None:
        sm_scale = dqk ** -0.5
    valid = sparse_mla_valid(idx, skv, q_start)
    safe = torch.where(valid, idx.to(torch.int64), torch.zeros_like(idx, dtype=torch.int64))
    qf, kvf = q.to(dtype), kv.to(dtype)
    outs, lses, pouts = [], [], []
    for s in range(0, sq, chunk):
        e = min(sq, s + chunk)
        kvg = kvf[safe[s:e]]                                   # [c, K, dqk]
        sc = torch.einsum("mhd,mkd->mhk", qf[s:e], kvg)        # raw logits
        sc = sc.masked_fill(~valid[s:e].unsqueeze(1), NEG_INF)
        z = sc * sm_scale
        if attn_sink is not None:
            zs = torch.cat([z, attn_sink.to(dtype).view(1, h, 1).expand(e - s, h, 1)], dim=-1)
            lse = torch.logsumexp(zs, dim=-1)
        else:
            lse = torch.logsumexp(z, dim=-1)                   # -inf for empty rows
        empty = torch.isinf(lse) & (lse < 0)
        p = torch.exp(z - lse.masked_fill(empty, 0.0).unsqueeze(-1))
        p = p.masked_fill(empty.unsqueeze(-1), 0.0)
        outs.append(torch.einsum("mhk,mkd->mhd", p, kvg[..., :d_v]))
        lses.append(lse.masked_fill(empty, float("inf")))
        pouts.append(sc)
    return torch.cat(outs), torch.cat(lses), torch.cat(pouts)


def sparse_mla_bwd(q, kv, idx, dout, q_start=0, sm_scale=None, d_v=512, dtype=torch.float32, attn_sink=None):
    """dQ, dKV by autograd through :func:`sparse_mla_fwd` -- exactly what the reference's own
    check does (ops/tilelang_ops/sparse_mla_bwd.py:310-319).  The closed form it must agree
    with is in that file's kernel, :176-231: ``dS = P*(dP - Delta)*scale``, ``dQ = dS.KV``,
    ``dKV[idx] += dS^T.Q (+ P^T.dO on the first d_v dims)``."""
    qd = q.detach().to(dtype).requires_grad_(True)
    kvd = kv.detach().to(dtype).requires_grad_(True)
    out, _, _ = sparse_mla_fwd(qd, kvd, idx, q_start, sm_scale, d_v, dtype=dtype, attn_sink=attn_sink)
    out.backward(dout.to(dtype))
    return qd.grad, kvd.grad


def sparse_mla_bwd_kernel_rounding(q, kv, idx, dout, q_start=0, sm_scale=None, d_v=512, out=None, lse=None,
                                   round_p_ds_bf16=True, round_rows_bf16=False, return_abs_sum=False, chunk=32,
                                   attn_sink=None, dtype=torch.float32):
    """dQ, dKV by the closed form of the reference's backward kernel, with that kernel's rounding
    points (ops/tilelang_ops/sparse_mla_bwd.py): every product accumulates in fp32 from bf16
    operands; ``P = exp(S*scale - lse)`` (:192-193) and ``dS = P*(dP - Delta)*scale`` (:197-199,
    from the fp32 P) are each cast to bf16 (``P_shared_cast``, ``dP_shared_cast``: :194, :200)
    before they enter ``dQ = dS.KV`` (:201-202) and ``dKV[idx] += dS^T.Q + P^T.dO`` (:203-209);
    dKV is accumulated in fp32 (atomic adds of the fp32 tile, :210-227).  ``Delta = rowsum(O*dO)``
    (preprocess kernel, :26-43) uses the forward's output as stored (bf16) and ``lse`` is the
    forward's; both default to this oracle's fp32 forward with the output rounded to bf16.  With ``round_p_ds_bf16=False`` this is the same closed form in fp32,
    which must agree with autograd (:func:`sparse_mla_bwd`).  Returns fp32 ``(dQ, dKV)``.
    ``round_rows_bf16`` adds the one rounding the HIP build has on top of the reference kernel's:
    the contribution of a (query, key) pair to dKV - the sum over all heads, one row of 576 values
    - is rounded to bf16 before the rows of a key are summed in fp32.  ``return_abs_sum`` also
    returns ``A[key, d] = sum over pairs |row[d]|`` and ``M[key, d] = max over pairs |row[d]|``:
    ``2**-9 * A`` bounds what that rounding can change (round-to-nearest bf16 moves a value by at
    most 2**-9 of its size), and ``2**-7 * M`` is one step of the bf16 grid at the largest row, i.e.
    what two evaluations differ by when that row lands on either side of a rounding boundary.
    Written with device-agnostic tensor ops, so a test may evaluate it on tensors that live on
    the GPU when the full benchmark sizes are too slow for the host (it stays a torch fp32
    evaluation of the same lines either way).  ``attn_sink`` only enters through ``lse`` (the sink
    is one more term of the softmax denominator and has no value row), i.e. through the default
    forward when ``lse`` is not given.  ``dtype`` is the arithmetic between the rounding points:
    fp32 as in the kernel, or fp64, which makes the result independent of the host's summation
    order (an fp32 sum that lands on the other side of a bf16 rounding boundary on another CPU
    would move a term by 2**-8 of its size).
    """
    sq, h, dqk = q.shape
    skv = kv.shape[0]
    if sm_scale is None:
        sm_scale = dqk ** -0.5
    if out is None or lse is None:
        o32, l32, _ = sparse_mla_fwd(q, kv, idx, q_start, sm_scale, d_v, attn_sink=attn_sink)
        out = o32.to(torch.bfloat16) if out is None else out
        lse = l32 if lse is None else lse
    valid = sparse_mla_valid(idx, skv, q_start)
    safe = torch.where(valid, idx.to(torch.int64), torch.zeros_like(idx, dtype=torch.int64))
    qf, kvf, dof = q.to(dtype), kv.to(dtype), dout.to(dtype)
    delta = (out.to(dtype) * dof).sum(-1)                                # [sq, h]
    lse_f = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse).to(dtype)
    dq = torch.zeros(sq, h, dqk, device=q.device, dtype=dtype)
    dkv = torch.zeros(skv, dqk, device=q.device, dtype=dtype)
    abs_sum = torch.zeros(skv, dqk, device=q.device, dtype=dtype) if return_abs_sum else None
    abs_max = torch.zeros(skv, dqk, device=q.device, dtype=dtype) if return_abs_sum else None
    rnd = (lambda t: t.to(torch.bfloat16).to(dtype)) if round_p_ds_bf16 else (lambda t: t)
    for s in range(0, sq, chunk):
        e = min(sq, s + chunk)
        kvg = kvf[safe[s:e]]                                             # [c, K, dqk]
        sc = torch.einsum("mhd,mkd->mhk", qf[s:e], kvg)
        p = torch.exp(sc * sm_scale - lse_f[s:e].unsqueeze(-1))
        p = p.masked_fill(~valid[s:e].unsqueeze(1), 0.0)
        dp = torch.einsum("mhd,mkd->mhk", dof[s:e], kvg[..., :d_v])
        ds = p * (dp - delta[s:e].unsqueeze(-1)) * sm_scale
        p_b, ds_b = rnd(p), rnd(ds)
        dq[s:e] = torch.einsum("mhk,mkd->mhd", ds_b, kvg)
        contrib = torch.einsum("mhk,mhd->mkd", ds_b, qf[s:e])
        contrib[..., :d_v] += torch.einsum("mhk,mhd->mkd", p_b, dof[s:e])
        if round_rows_bf16:
            contrib = contrib.to(torch.bfloat16).to(dtype)
        dkv.index_add_(0, safe[s:e].reshape(-1), contrib.reshape(-1, dqk))   # invalid slots add zeros to row 0
        if return_abs_sum:
            abs_sum.index_add_(0, safe[s:e].reshape(-1), contrib.abs().reshape(-1, dqk))
            abs_max.scatter_reduce_(0, safe[s:e].reshape(-1, 1).expand(-1, dqk), contrib.abs().reshape(-1, dqk), "amax")
    if return_abs_sum:
        return dq, dkv, abs_sum, abs_max
    return dq, dkv


# --------------------------------------------------------------------------------------------
# a9/a10. Attention distribution + KL loss
# --------------------------------------------------------------------------------------------
def attn_dist(p_out: torch.Tensor, sm_scale: float) -> torch.Tensor:
    """``target[i,t] = mean_h softmax_t(p_out[i,h,:] * sm_scale)[t]`` in fp32.

    dsa_fused_kernels.py:1877-1895.  Slots holding -inf get probability 0.
    """
    z = p_out.float() * sm_scale
    return torch.softmax(z, dim=-1).mean(dim=1)


def attn_dist_from_lse(q, kv, idx, lse, q_start: int, sm_scale: float, heads: Optional[int] = None,
                       dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``target[i,t] = mean_{h<heads} exp(q[i,h].kv[idx[i,t]] * sm_scale - lse[i,h])``, 0 on invalid slots.

    The distribution of :func:`attn_dist` (dsa_fused_kernels.py:1877-1895 applied to the forward's
    logits, dsa_fused.py:928-929) written from the forward's log-sum-exp: per head
    ``softmax_t(z)[t] = exp(z_t - logsumexp(z))``.  ``heads`` restricts the mean to the leading
    heads (the reference slices padded heads off before the call, dsa_fused.py:915-917).
    """
    sq, h, _ = q.shape
    heads = h if heads is None else heads
    valid = sparse_mla_valid(idx, kv.shape[0], q_start)
    safe = torch.where(valid, idx.to(torch.int64), torch.zeros_like(idx, dtype=torch.int64))
    out = torch.zeros(sq, idx.shape[1], dtype=dtype)
    qf, kvf, lf = q.to(dtype), kv.to(dtype), lse.to(dtype)
    for s in range(0, sq, 64):
        e = min(sq, s + 64)
        z = torch.einsum("mhd,mkd->mhk", qf[s:e, :heads], kvf[safe[s:e]]) * sm_scale
        p = torch.exp(z - lf[s:e, :heads].unsqueeze(-1)).masked_fill(~valid[s:e].unsqueeze(1), 0.0)
        out[s:e] = p.mean(dim=1)
    return out


def indexer_kl_loss(index_score_topk, target, coeff: float, sq_norm: int, eps: float = 1e-10):
    """``coeff * KL(target+eps || softmax(score)+eps) / sq`` with ``reduction='sum'``.

    loongforge/models/common/experimental_attention_variant/dsa_fused.py:931-944.
    """
    pred = torch.softmax(index_score_topk.float(), dim=-1)
    tgt = target.float() + eps
    loss = (tgt * (tgt.log() - (pred + eps).log())).sum()
    return coeff * loss / sq_norm


# --------------------------------------------------------------------------------------------
# a5. Indexer backward
# --------------------------------------------------------------------------------------------
def unscale_indexer_grad(grad: torch.Tensor, scale_inv: torch.Tensor) -> torch.Tensor:
    """``grad / scale_inv`` with rows sitting on the quantiser's epsilon floor forced to 0.

    deepseek_v4_csa.py:1525-1541 (floor = 1.5 * 2**-48).
    """
    floor = 2.0 ** -48 * 1.5
    si = scale_inv.unsqueeze(-1)
    usable = torch.isfinite(si) & (si > floor)
    safe = torch.where(usable, si, torch.ones_like(si))
    return (grad / safe).masked_fill(~usable.expand_as(grad), 0.0)


def indexer_bwd(grad_score, q8, k8, q_scale, k_scale, weight_scaled, idx, dtype=torch.float32):
    """Gradients of the selected logits (dsa_fused_kernels.py:2396-2442).

    Differentiates ``gathered_indexer_logits`` w.r.t. the fp8 payloads (as floats) and
    ``weight_scaled`` with the scales held constant, then applies the reference's un-scaling:
    ``d_weights = d_w' * q_scale * d**-0.5``, ``d_q = d_q8 / q_scale``, ``d_k = d_k8 / k_scale``.
    """
    d = q8.shape[-1]
    qf = q8.to(dtype).detach().requires_grad_(True)
    kf = k8.to(dtype).detach().requires_grad_(True)
    wf = weight_scaled.to(dtype).detach().requires_grad_(True)
    sel = gathered_indexer_logits(qf, wf, kf, k_scale, idx, dtype=dtype)
    valid = idx >= 0
    g = torch.where(valid, grad_score.to(dtype), torch.zeros_like(sel))
    sel = torch.where(valid, sel, torch.zeros_like(sel))
    (sel * g).sum().backward()
    d_w = wf.grad * q_scale.to(dtype) * (d ** -0.5)
    d_q = unscale_indexer_grad(qf.grad, q_scale.to(dtype))
    d_k = unscale_indexer_grad(kf.grad, k_scale.to(dtype))
    return d_q, d_k, d_w


# --------------------------------------------------------------------------------------------
# End-to-end fused DSA forward (+ loss), for config 1 / config 5 style checks
# --------------------------------------------------------------------------------------------
def dsa_forward(q, kv, index_q, index_k, weights, topk, sm_scale, chunk_offset=0,
                cu_seqlens=None, loss_coeff=1.0, d_v=512, n_heads=None):
    """indexer -> top-k -> sparse MLA -> attn_dist -> KL (dsa_fused.py:796-956)."""
    scores, idx, aux = indexer_forward(index_q, index_k, weights, topk, chunk_offset, cu_seqlens)
    out, lse, p_out = sparse_mla_fwd(q, kv, idx, chunk_offset, sm_scale, d_v)
    h = n_heads if n_heads is not None else q.shape[1]
    target = attn_dist(p_out[:, :h], sm_scale)
    loss = indexer_kl_loss(scores, target, loss_coeff, q.shape[0])
    return dict(out=out, lse=lse, p_out=p_out, scores=scores, idx=idx, target=target,
                loss=loss, aux=aux)


# --------------------------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations (CPU RNG so oracle and GPU see equal bits)
# --------------------------------------------------------------------------------------------
def causal_random_topk_indices(sq: int, topk: int, seed: int, q_start: int = 0,
                               cu_seqlens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``idx[i] = randperm(prefix_i)[:topk]`` (all of the prefix when it is shorter), -1 padded.

    Same recipe as the reference's self-checks (ops/tilelang_ops/sparse_mla_fwd.py:291-298) but
    including the query's own position; vectorised with random keys + argsort-free top-k.
    """
    g = torch.Generator().manual_seed(seed)
    ks, ke = indexer_window(sq, q_start, cu_seqlens)
    out = torch.full((sq, topk), -1, dtype=torch.int32)
    width = int(ke.max())
    step = 512
    cols = torch.arange(width)
    for s in range(0, sq, step):
        e = min(sq, s + step)
        r = torch.rand(e - s, width, generator=g)
        vis = (cols[None] >= ks[s:e, None]) & (cols[None] < ke[s:e, None])
        r = r.masked_fill(~vis, -1.0)
        kk = min(topk, width)
        v, i = torch.topk(r, kk, dim=-1)
        i = torch.where(v >= 0, i, torch.full_like(i, -1))
        out[s:e, :kk] = i.to(torch.int32)
    return out


@dataclass
class MlaInputs:
    q: torch.Tensor
    kv: torch.Tensor
    idx: torch.Tensor
    dout: torch.Tensor
    sm_scale: float


def make_mla_inputs(sq: int, h: int = 128, topk: int = 2048, dqk: int = 576, d_v: int = 512,
                    seed: int = 0, skv: Optional[int] = None, q_start: int = 0) -> MlaInputs:
    """bf16 ~N(0,1) q / kv / dO and random causal top-k ids (benchmark configs 3 and 4)."""
    skv = sq + q_start if skv is None else skv
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(sq, h, dqk, generator=g).to(torch.bfloat16)
    kv = torch.randn(skv, dqk, generator=g).to(torch.bfloat16)
    g2 = torch.Generator().manual_seed(seed + 1)
    dout = torch.randn(sq, h, d_v, generator=g2).to(torch.bfloat16)
    idx = causal_random_topk_indices(sq, topk, seed + 2, q_start)
    return MlaInputs(q, kv, idx, dout, 1.0 / math.sqrt(192.0))


def make_indexer_inputs(sq: int, h: int = 64, d: int = 128, seed: int = 42, w_std: float = 0.1,
                        w_uniform: bool = False):
    """bf16 ~N(0,1) indexer q / k and fp32 head weights (benchmark configs 1 and 2)."""
    g = torch.Generator().manual_seed(seed)
    iq = torch.randn(sq, h, d, generator=g).to(torch.bfloat16)
    ik = torch.randn(sq, d, generator=g).to(torch.bfloat16)
    if w_uniform:
        w = torch.rand(sq, h, generator=g)
    else:
        w = torch.randn(sq, h, generator=g) * w_std
    return iq, ik, w


def make_packed_cu_seqlens(total: int, n_docs: int, min_len: int, seed: int) -> torch.Tensor:
    """Seeded random document lengths >= min_len summing to ``total`` (benchmark config 5)."""
    g = torch.Generator().manual_seed(seed)
    rest = total - n_docs * min_len
    assert rest >= 0
    cuts = torch.sort(torch.randint(0, rest + 1, (n_docs - 1,), generator=g)).values
    parts = torch.diff(torch.cat([torch.zeros(1, dtype=torch.int64), cuts,
                                  torch.tensor([rest])]))
    lens = parts + min_len
    return F.pad(lens.cumsum(0), (1, 0)).to(torch.int32)
