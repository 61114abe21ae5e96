"""CPU restatement of the indexer front end behind its projections (TEST INFRASTRUCTURE: only tests/,
``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import this; the product path never does).

Reference: loongforge/models/common/experimental_attention_variant/dsa_fused.py
  :583-584   k = k_norm(linear_wk(x))              LayerNorm over the 128 channels of an indexer key
  :423-487   _apply_rope                           rotary embedding of the leading 64 channels ("PE first")
  :74-90     rotate_activation                     Hadamard rotation scaled by 128^-0.5, bf16 in / bf16 out
  dsa_fused_kernels.py:2341-2346, :2362            row-wise e4m3 quantiser, weight_scaled = w * q_scale * d^-0.5
The reference runs these as separate bf16 -> bf16 operations; this file keeps a bf16 rounding after each
of them.  The fp32 sums inside LayerNorm and the rotation are taken in a fixed order (8 consecutive
elements in sequence, then the 16 groups of a row pairwise by xor 1, 2, 4, 8), which is the order the HIP
kernel uses, so that kernel and oracle agree bit for bit; the reference's own summation order (inside
TransformerEngine's LayerNorm and a Hadamard wheel) is not visible, so against IT parity holds to rounding
only: parity of the summation order is unpinned.

What pins each function (tests/test_oracle_front.py):
  layer_norm_rows   torch.nn.functional.layer_norm in fp64 (to fp32 rounding); constant rows give beta
  hadamard_rows     the Sylvester matrix product in fp64 (to one bf16 step); applying it twice returns x
  rope part         oracle/rope_oracle.py (pinned in tests/test_oracle_rope.py)
  quantiser         oracle/dsa_oracle.py quant_rowwise_e4m3 (pinned in tests/test_oracle_quant_indexer.py)
  indexer_front     the same pipeline written with library routines in fp64, to bf16 / fp8 rounding
"""
import torch

from . import dsa_oracle as O
from . import rope_oracle as R

_IDX = torch.arange(16)


def _row_sum(t):
    """Sum of [rows, 16, 8] fp32 over the last two dims: in-group sequence, then xor-butterfly over the groups."""
    s = t[..., 0]
    for i in range(1, 8):
        s = s + t[..., i]
    for m in (1, 2, 4, 8):
        s = s + s[..., _IDX ^ m]
    return s                                            # [rows, 16], every group holding the total


def _bf16(t):
    return t.to(torch.bfloat16).float()


def layer_norm_rows(x, weight, bias, eps):
    """LayerNorm of bf16 rows of 128 (dsa_fused.py:584; statistics and affine map in fp32, one rounding)."""
    v = x.float().reshape(-1, 16, 8)
    mean = _row_sum(v) * 0.0078125
    d = v - mean.unsqueeze(-1)
    var = _row_sum(d * d) * 0.0078125
    rstd = 1.0 / torch.sqrt(var + torch.tensor(eps, dtype=torch.float32))
    w, b = weight.float().reshape(16, 8), bias.float().reshape(16, 8)
    y = (d * rstd.unsqueeze(-1)) * w + b
    return y.reshape(x.shape).to(torch.bfloat16)


def hadamard_rows(x):
    """rotate_activation (dsa_fused.py:74-90): Sylvester-Hadamard rotation of bf16 rows of 128 times 128^-0.5,
    as a butterfly over the 7 index bits, lowest bit first."""
    v = x.float().reshape(-1, 16, 8).clone()
    for m in (1, 2, 4):
        lo = [i for i in range(8) if not i & m]
        hi = [i | m for i in lo]
        a, b = v[..., lo], v[..., hi]
        v[..., lo], v[..., hi] = a + b, a - b
    for m in (1, 2, 4, 8):
        o = v[:, _IDX ^ m, :]
        upper = ((_IDX & m) != 0).reshape(1, 16, 1)
        v = torch.where(upper, o - v, v + o)
    v = v * torch.tensor(0.08838834764831845, dtype=torch.float32)
    return v.reshape(x.shape).to(torch.bfloat16)


def indexer_front(x, rows_per_token=1, ln_weight=None, ln_bias=None, ln_eps=1e-5, cos=None, sin=None, pairing=-1,
                  positions=None, batch=1, rotate=True, weights=None, factor=1.0):
    """bf16 ``[..., 128]`` rows -> ``(x8, scale_inv, rows, weight_scaled)``: the payload and scale of the quantised
    rows, the bf16 rows that were quantised, and ``(weights * scale_inv) * factor`` (None without weights)."""
    shape = x.shape
    v = x.reshape(-1, 128)
    if ln_weight is not None:
        v = layer_norm_rows(v, ln_weight, ln_bias, ln_eps)
    if pairing >= 0:
        tokens = v.shape[0] // rows_per_token
        pos = positions.long() if positions is not None else torch.arange(tokens) // batch
        c = cos.reshape(-1, 64)[pos].repeat_interleave(rows_per_token, 0)
        s = sin.reshape(-1, 64)[pos].repeat_interleave(rows_per_token, 0)
        pe = R.rotate(v[:, :64], c, s, pairing, pairing, False, torch.float32)
        v = torch.cat([pe.to(torch.bfloat16), v[:, 64:]], dim=-1)
    if rotate:
        v = hadamard_rows(v)
    v = v.reshape(shape)
    x8, scale_inv = O.quant_rowwise_e4m3(v)
    ws = None
    if weights is not None:
        ws = (weights.float() * scale_inv) * torch.tensor(factor, dtype=torch.float32)
    return x8, scale_inv, v, ws
