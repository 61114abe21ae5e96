"""Pins for the oracle's rotary-embedding restatement (oracle/rope_oracle.py)."""
import torch

from oracle import rope_oracle as R

F64 = torch.float64


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def test_adjacent_pairs_are_a_complex_multiplication():
    cos, sin = R.rope_tables(50, 16, interleaved=True, dtype=F64)
    x = _rand(7, 3, 16)
    pos = torch.tensor([0, 1, 5, 9, 20, 33, 49])
    y = R.rotate(x, cos[pos].unsqueeze(1), sin[pos].unsqueeze(1), R.ADJACENT, R.ADJACENT, dtype=F64)
    z = torch.view_as_complex(x.reshape(7, 3, 8, 2).contiguous())
    ang = torch.polar(torch.ones(50, 8, dtype=F64), torch.arange(50, dtype=F64)[:, None] * 10000.0 ** (-torch.arange(0, 16, 2, dtype=F64) / 16))
    ref = torch.view_as_real(z * ang[pos].unsqueeze(1)).reshape(7, 3, 16)
    torch.testing.assert_close(y, ref, rtol=1e-12, atol=1e-12)


def test_split_pairs_are_the_rotate_half_formula():
    cos, sin = R.rope_tables(40, 8, interleaved=False, dtype=F64)
    x = _rand(5, 2, 8, seed=1)
    pos = torch.tensor([3, 0, 39, 17, 8])
    c, s = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
    y = R.rotate(x, c, s, R.SPLIT, R.SPLIT, dtype=F64)
    rot_half = torch.cat([-x[..., 4:], x[..., :4]], dim=-1)
    torch.testing.assert_close(y, x * c + rot_half * s, rtol=1e-12, atol=1e-12)
    # adjacent in / split out = de-interleave, then the same formula
    y2 = R.rotate(x, c, s, R.ADJACENT, R.SPLIT, dtype=F64)
    xd = torch.cat([x[..., 0::2], x[..., 1::2]], dim=-1)
    torch.testing.assert_close(y2, xd * c + torch.cat([-xd[..., 4:], xd[..., :4]], dim=-1) * s, rtol=1e-12, atol=1e-12)


def test_rotation_preserves_norm_and_inverse_undoes_it_on_genuine_tables():
    for inter, pin, pout in [(True, R.ADJACENT, R.ADJACENT), (False, R.SPLIT, R.SPLIT), (False, R.ADJACENT, R.SPLIT)]:
        cos, sin = R.rope_tables(30, 32, interleaved=inter, dtype=F64)
        x = _rand(6, 4, 32, seed=2)
        pos = torch.arange(6) * 5
        c, s = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
        y = R.rotate(x, c, s, pin, pout, dtype=F64)
        torch.testing.assert_close(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-12, atol=1e-12)
        back = R.rotate(y, c, s, pout, pin, inverse=True, dtype=F64)
        torch.testing.assert_close(back, x, rtol=1e-12, atol=1e-12)


def test_inverse_is_the_adjoint_on_generic_tables():
    # with independent entries in cos / sin (c1 != c2, s1 != s2) every index convention matters
    cos, sin = R.rope_tables(20, 16, dtype=F64, seed=7)
    pos = torch.tensor([4, 19, 0])
    c, s = cos[pos].unsqueeze(1), sin[pos].unsqueeze(1)
    for pin in (R.ADJACENT, R.SPLIT):
        for pout in (R.ADJACENT, R.SPLIT):
            x, g = _rand(3, 5, 16, seed=3), _rand(3, 5, 16, seed=4)
            lhs = (R.rotate(x, c, s, pin, pout, dtype=F64) * g).sum()
            rhs = (x * R.rotate(g, c, s, pout, pin, inverse=True, dtype=F64)).sum()
            assert abs(lhs.item() - rhs.item()) < 1e-10


def test_public_functions_against_loops_and_adjoints():
    T, H, d, emb = 9, 3, 8, 8
    cos, sin = R.rope_tables(16, emb, dtype=F64, seed=11)
    cu = torch.tensor([0, 4, 9])
    pos = R.thd_positions(cu, T)
    assert pos.tolist() == [0, 1, 2, 3, 0, 1, 2, 3, 4]
    assert R.thd_positions(cu, 3, offset=3).tolist() == [3, 0, 1]
    for inter in (False, True):
        # query rope in place, rotary part first or last
        for off in (0, d):
            t3 = _rand(T, H, d + emb, seed=5)
            out = R.fused_apply_mla_rope(t3, cos, sin, off, emb, pos, inter, dtype=F64)
            p = R.ADJACENT if inter else R.SPLIT
            for t in range(T):
                for h in range(H):
                    ref = t3[t, h].clone()
                    ref[off: off + emb] = R.rotate(t3[t, h, off: off + emb], cos[pos[t]], sin[pos[t]], p, p, dtype=F64)
                    torch.testing.assert_close(out[t, h], ref, rtol=0, atol=0)
            g = _rand(T, H, d + emb, seed=6)
            gi = R.fused_apply_mla_rope(g, cos, sin, off, emb, pos, inter, inverse=True, dtype=F64)
            assert abs((out * g).sum().item() - (t3 * gi).sum().item()) < 1e-9
        # permute + rope + cat
        qc, pe = _rand(H, T, d, seed=7), _rand(T, H, emb, seed=8)
        out = R.fused_rope_permute_cat(qc, pe, cos, sin, pos, inter, dtype=F64)
        po = R.ADJACENT if inter else R.SPLIT
        for t in range(T):
            for h in range(H):
                torch.testing.assert_close(out[t, h, :d], qc[h, t], rtol=0, atol=0)
                torch.testing.assert_close(out[t, h, d:], R.rotate(pe[t, h], cos[pos[t]], sin[pos[t]], R.ADJACENT, po, dtype=F64),
                                           rtol=0, atol=0)
        g = _rand(T, H, d + emb, seed=9)
        gqc, gpe = R.fused_rope_permute_cat_bwd(g, d, cos, sin, pos, inter, dtype=F64)
        assert abs((out * g).sum().item() - ((qc * gqc).sum() + (pe * gpe).sum()).item()) < 1e-9
        # absorbed key
        kv, ke = _rand(T, H, d, seed=10), _rand(T, emb, seed=12)
        key = R.absorb_kv(kv, ke, cos, sin, pos, inter, dtype=F64)
        for t in range(T):
            for h in range(H):
                torch.testing.assert_close(key[t, h, :d], kv[t, h], rtol=0, atol=0)
                torch.testing.assert_close(key[t, h, d:], R.rotate(ke[t], cos[pos[t]], sin[pos[t]], R.ADJACENT, po, dtype=F64),
                                           rtol=0, atol=0)
        dkv, demb = R.absorb_kv_bwd(g, d, cos, sin, pos, inter, dtype=F64, round_sum=False)
        assert abs((key * g).sum().item() - ((kv * dkv).sum() + (ke * demb).sum()).item()) < 1e-9
