"""Pin of oracle/mla_module_oracle.py: with the layer norms and projections taken out of the picture it is
torch's scaled_dot_product_attention on explicitly up-projected keys and values."""
import torch

from oracle import mla_module_oracle as M
from oracle import rope_oracle as R


def test_dense_mla_is_sdpa_on_up_projected_keys_and_values():
    g = torch.Generator().manual_seed(0)
    S, H, hid, ql = 40, 3, 32, 24
    f = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.3      # noqa: E731
    p = dict(q_down=f(ql, hid), q_ln_w=1 + f(ql), q_ln_b=f(ql), q_up=f(H * 192, ql), kv_down=f(576, hid),
             kv_ln_w=1 + f(512), kv_ln_b=f(512), kv_up=f(H * 256, 512), proj=f(hid, H * 128))
    x = f(S, hid)
    y = M.mla_dense(x, p, H)
    # the same by hand, attention through the library routine
    q = (M.layer_norm(x @ p["q_down"].T, p["q_ln_w"], p["q_ln_b"], 1e-5) @ p["q_up"].T).view(S, H, 192)
    kv = x @ p["kv_down"].T
    c = M.layer_norm(kv[:, :512], p["kv_ln_w"], p["kv_ln_b"], 1e-5)
    cos, sin = R.rope_tables(S, 64, dtype=torch.float64)
    rot = lambda t, cs, sn: R.rotate(t, cs, sn, R.ADJACENT, R.SPLIT, False, torch.float64)   # noqa: E731
    up = (c @ p["kv_up"].T).view(S, H, 256)
    k = torch.cat([up[:, :, :128], rot(kv[:, 512:], cos, sin).unsqueeze(1).expand(S, H, 64)], -1)
    qq = torch.cat([q[:, :, :128], rot(q[:, :, 128:], cos.unsqueeze(1), sin.unsqueeze(1))], -1)
    o = torch.nn.functional.scaled_dot_product_attention(qq.transpose(0, 1), k.transpose(0, 1), up[:, :, 128:].transpose(0, 1),
                                                         is_causal=True, scale=192 ** -0.5)
    ref = o.transpose(0, 1).reshape(S, H * 128) @ p["proj"].T
    torch.testing.assert_close(y, ref, rtol=1e-9, atol=1e-9)
    # causality: the first token attends to itself only, so its output is the projected value of token 0
    torch.testing.assert_close(y[0], up[0, :, 128:].reshape(-1) @ p["proj"].T, rtol=1e-9, atol=1e-9)
