"""Textbook (non-absorbed) multi-latent attention, dense and causal, in plain torch on the CPU.

TEST INFRASTRUCTURE: only tests/ may import this; the product path never does.

It states what the absorbed data flow of ``MLASelfAttentionFused``
(loongforge/models/common/experimental_attention_variant/multi_latent_attention.py:870-1026, :1028-1338)
must equal when every query attends to its whole causal prefix: keys and values are up-projected from the
normalised latent, ``k[h] = [W_UK[h] c | rope(k_pe)]``, ``v[h] = W_UV[h] c``, queries are
``[q_nope[h] | rope(q_pe[h])]``, attention is softmax(q k^T / sqrt(192)) v per head.  The absorbed form moves
W_UK to the query side and W_UV behind the attention; the two agree because
``q_nope . (W_UK c) = (W_UK^T q_nope) . c`` and ``sum_t p_t (W_UV c_t) = W_UV (sum_t p_t c_t)``.
The rotary embedding takes adjacent channel pairs in and writes split halves out, the same for queries and
keys (oracle/rope_oracle.py, pinned in tests/test_oracle_rope.py).  Pinned in tests/test_oracle_mla_module.py
against torch's scaled_dot_product_attention on the up-projected keys and values.
"""
import torch

from . import rope_oracle as R


def layer_norm(x, weight, bias, eps):
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), weight, bias, eps)


def mla_dense(x, p, heads, qk_head_dim=128, pos_dim=64, v_head_dim=128, kv_lora_rank=512, eps=1e-5, rotary_base=10000.0,
              dtype=torch.float64):
    """``x [S, hidden]``, ``p`` a dict of weights (``q_down, q_ln_w, q_ln_b, q_up, kv_down, kv_ln_w, kv_ln_b, kv_up,
    proj``, each ``[out, in]`` like torch.nn.Linear) -> ``y [S, hidden]``."""
    p = {k: v.to(dtype) for k, v in p.items()}
    x = x.to(dtype)
    S = x.shape[0]
    q_c = layer_norm(x @ p["q_down"].T, p["q_ln_w"], p["q_ln_b"], eps)
    q = (q_c @ p["q_up"].T).view(S, heads, qk_head_dim + pos_dim)
    kv = x @ p["kv_down"].T
    c = layer_norm(kv[:, :kv_lora_rank], p["kv_ln_w"], p["kv_ln_b"], eps)
    inv_freq = 1.0 / (rotary_base ** (torch.arange(0, pos_dim, 2, dtype=dtype) / pos_dim))
    ang = torch.outer(torch.arange(S, dtype=dtype), inv_freq)
    ang = torch.cat([ang, ang], dim=-1)
    cos, sin = ang.cos(), ang.sin()
    q_pe = R.rotate(q[:, :, qk_head_dim:], cos.unsqueeze(1), sin.unsqueeze(1), R.ADJACENT, R.SPLIT, False, dtype)
    k_pe = R.rotate(kv[:, kv_lora_rank:], cos, sin, R.ADJACENT, R.SPLIT, False, dtype)
    up = (c @ p["kv_up"].T).view(S, heads, qk_head_dim + v_head_dim)
    k = torch.cat([up[:, :, :qk_head_dim], k_pe.unsqueeze(1).expand(S, heads, pos_dim)], dim=-1)
    v = up[:, :, qk_head_dim:]
    qq = torch.cat([q[:, :, :qk_head_dim], q_pe], dim=-1)
    scores = torch.einsum("shd,thd->hst", qq, k) * (qk_head_dim + pos_dim) ** -0.5
    scores = scores.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), float("-inf"))
    out = torch.einsum("hst,thd->shd", scores.softmax(-1), v).reshape(S, heads * v_head_dim)
    return out @ p["proj"].T
