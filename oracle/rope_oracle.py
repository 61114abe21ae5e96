"""CPU restatement of the reference's MLA rotary-embedding kernels.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the
product (loongforge_amd/) never does.

The reference's kernels are Triton text in
loongforge/models/common/experimental_attention_variant/dsa_fused_kernels.py (cited per function
below); they were read, not run (Triton and Megatron are absent here).  `_get_thd_token_idx` comes
from megatron.core.fusions.fused_mla_yarn_rope_apply (Loong-Megatron, an un-vendored submodule): for
context-parallel size 1 it returns the index of a packed token inside its own sequence, which is
what `thd_positions` restates; larger context-parallel sizes are out of scope (one GPU).

Parity status
-------------
rotate                  pinned: equals complex multiplication (adjacent pairs) and the textbook
                        x*cos + rotate_half(x)*sin (split pairs) on genuine rotary tables; the
                        inverse is pinned as the adjoint (<rope(x), g> == <x, rope^T(g)>, fp64) on
                        generic tables where c1 != c2, s1 != s2, so every index convention counts.
fused_apply_mla_rope, fused_rope_permute_cat, absorb_kv (+ backward)
                        pinned: compositions of `rotate` with slicing / permutation written out as
                        loops in the tests; backward pinned as the adjoint of the forward in fp64.
                        unpinned detail: the rounding of intermediate products inside Triton when
                        cos / sin are bf16 (this restatement computes in fp32 and rounds once).
"""
from __future__ import annotations

from typing import Optional

import torch

ADJACENT, SPLIT = 0, 1


def _split(x, pairing):
    half = x.shape[-1] // 2
    return (x[..., 0::2], x[..., 1::2]) if pairing == ADJACENT else (x[..., :half], x[..., half:])


def _join(y1, y2, pairing):
    if pairing == ADJACENT:
        return torch.stack([y1, y2], dim=-1).flatten(-2)
    return torch.cat([y1, y2], dim=-1)


def rotate(x, cos, sin, in_pairing, out_pairing, inverse=False, dtype=torch.float32):
    """Rotation of the last dimension, pair by pair (dsa_fused_kernels.py:118-143 adjacent pairs,
    :401-425 split pairs, :685-706 adjacent in / split out; inverses :206-228, :476-499, :889-907,
    :994-1008).  cos / sin broadcast against x and are indexed with the pairing of the rotated side.
    Products and sums are separate `dtype` operations; the caller rounds."""
    x1, x2 = _split(x.to(dtype), in_pairing)
    cs_pairing = in_pairing if inverse else out_pairing
    c1, c2 = _split(cos.to(dtype), cs_pairing)
    s1, s2 = _split(sin.to(dtype), cs_pairing)
    if not inverse:
        y1 = x1 * c1 - x2 * s1
        y2 = x2 * c2 + x1 * s2
    else:
        y1 = x1 * c1 + x2 * s2
        y2 = (-x1) * s1 + x2 * c2
    return _join(y1, y2, out_pairing)


def thd_positions(cu_seqlens, tokens, offset=0):
    """Index of each packed token inside its own sequence (context-parallel size 1)."""
    cu = [int(v) for v in cu_seqlens]
    out = torch.zeros(tokens, dtype=torch.int64)
    for t in range(tokens):
        gt = t + offset
        for s in range(len(cu) - 1):
            if cu[s] <= gt < cu[s + 1]:
                out[t] = gt - cu[s]
                break
    return out


def _rows(cos, sin, positions, emb):
    cos2, sin2 = cos.reshape(-1, emb), sin.reshape(-1, emb)
    return cos2[positions].unsqueeze(1), sin2[positions].unsqueeze(1)      # [tokens, 1, emb]


def fused_apply_mla_rope(t3, cos, sin, emb_offset, emb_dim, positions, interleaved, inverse=False, dtype=torch.float32):
    """t3 [tokens, heads, d]: rotates columns [emb_offset, emb_offset + emb_dim) in place of a copy
    (dsa_fused_kernels.py:69-143, 367-425; backward :159-228, :443-499; wrapper :1168-1212)."""
    p = ADJACENT if interleaved else SPLIT
    c, s = _rows(cos, sin, positions, emb_dim)
    out = t3.clone()
    pe = rotate(t3[:, :, emb_offset: emb_offset + emb_dim], c, s, p, p, inverse, dtype)
    out[:, :, emb_offset: emb_offset + emb_dim] = pe.to(t3.dtype)
    return out


def fused_rope_permute_cat(q_content, q_pos_emb, cos, sin, positions, interleaved, dtype=torch.float32):
    """q_content [h, S, d], q_pos_emb [S, h, emb] -> [S, h, d + emb] (dsa_fused_kernels.py:620-806)."""
    emb = q_pos_emb.shape[-1]
    c, s = _rows(cos, sin, positions, emb)
    pe = rotate(q_pos_emb, c, s, ADJACENT, ADJACENT if interleaved else SPLIT, False, dtype).to(q_content.dtype)
    return torch.cat([q_content.permute(1, 0, 2), pe], dim=-1)


def fused_rope_permute_cat_bwd(grad, d_out, cos, sin, positions, interleaved, dtype=torch.float32):
    """grad [S, h, d + emb] -> (grad_q_content [h, S, d], grad_q_pos_emb [S, h, emb])
    (dsa_fused_kernels.py:822-1008)."""
    emb = grad.shape[-1] - d_out
    c, s = _rows(cos, sin, positions, emb)
    gpe = rotate(grad[:, :, d_out:], c, s, ADJACENT if interleaved else SPLIT, ADJACENT, True, dtype).to(grad.dtype)
    return grad[:, :, :d_out].permute(1, 0, 2).contiguous(), gpe


def absorb_kv(kv3, k_pos_emb, cos, sin, positions, interleaved, dtype=torch.float32):
    """kv3 [T, h, k_dim], k_pos_emb [T, emb] -> key [T, h, k_dim + emb] (dsa_fused_kernels.py:1229-1312,
    :1426-1502)."""
    emb = k_pos_emb.shape[-1]
    c, s = _rows(cos, sin, positions, emb)
    pe = rotate(k_pos_emb.unsqueeze(1), c, s, ADJACENT, ADJACENT if interleaved else SPLIT, False, dtype).to(kv3.dtype)
    return torch.cat([kv3, pe.expand(-1, kv3.shape[1], -1)], dim=-1)


def absorb_kv_bwd(dk3, k_dim, cos, sin, positions, interleaved, dtype=torch.float32, round_sum=True):
    """dk3 [T, h, k_dim + emb] -> (d_kv [T, h, k_dim], d_emb [T, emb]) (dsa_fused_kernels.py:1328-1410,
    :1518-1608): head-sum of the rotary part in `dtype`, rounded to the tensor dtype (:1391-1392), then
    the inverse rotation."""
    emb = dk3.shape[-1] - k_dim
    c, s = _rows(cos, sin, positions, emb)
    tot = dk3[:, :, k_dim:].to(dtype).sum(dim=1, keepdim=True)
    if round_sum:
        tot = tot.to(dk3.dtype)
    d_emb = rotate(tot, c, s, ADJACENT if interleaved else SPLIT, ADJACENT, True, dtype).to(dk3.dtype)
    return dk3[:, :, :k_dim].contiguous(), d_emb.squeeze(1)


def rope_tables(max_pos, emb, base=10000.0, interleaved=False, dtype=torch.float32, seed: Optional[int] = None):
    """Genuine rotary tables [max_pos, emb]: angle(pos, j) = pos * base^(-2 j / emb), laid out so that both
    elements of pair j carry angle j.  With `seed`, generic tables (independent entries) instead."""
    if seed is not None:
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(max_pos, emb, generator=g).to(dtype), torch.randn(max_pos, emb, generator=g).to(dtype))
    inv = base ** (-torch.arange(0, emb, 2, dtype=torch.float64) / emb)
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]          # [max_pos, emb/2]
    ang = ang.repeat_interleave(2, dim=-1) if interleaved else torch.cat([ang, ang], dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)
