"""GPU parity: rotary-embedding kernels (query in place, permute + rope + cat, absorbed key) against the oracle."""
import pytest
import torch

from oracle import rope_oracle as R

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(BF)


def _tables(max_pos, emb, inter, dt, generic):
    cos, sin = R.rope_tables(max_pos, emb, interleaved=inter, seed=3 if generic else None)
    return cos.to(dt).view(max_pos, 1, 1, emb).contiguous(), sin.to(dt).view(max_pos, 1, 1, emb).contiguous()


@pytest.mark.parametrize("inter", [False, True])
@pytest.mark.parametrize("thd", [False, True])
@pytest.mark.parametrize("dt,generic", [(torch.float32, False), (BF, True)])
def test_query_rope_in_place_and_its_backward(gpu, inter, thd, dt, generic):
    from loongforge_amd.dsa_fused_kernels import fused_apply_mla_rope

    s, b, h, d, emb = (37, 2, 128, 128, 64) if not thd else (61, 1, 64, 192, 64)
    cos, sin = _tables(80, emb, inter, dt, generic)
    for pe_first in (False, True):
        x = _rand(s, b, h, d + emb, seed=1) if not thd else _rand(s, h, d + emb, seed=1)
        cu = torch.tensor([0, 20, 21, 61], dtype=torch.int32) if thd else None
        sp = 0
        pos = R.thd_positions(cu, s, sp) if thd else torch.arange(s * b) // b
        x3 = x.view(-1, h, d + emb)
        ref = R.fused_apply_mla_rope(x3, cos, sin, 0 if pe_first else d, emb, pos, inter)
        xg = x.clone().to(gpu).requires_grad_(True)
        y = fused_apply_mla_rope(xg * 1, cos.to(gpu), sin.to(gpu), d, emb, cu.to(gpu) if thd else None, 0, 1, inter, pe_first, sp)
        assert y.shape == x.shape
        assert torch.equal(y.detach().cpu().view(-1, h, d + emb), ref)
        g = _rand(*x.shape, seed=2)
        y.backward(g.to(gpu))
        gref = R.fused_apply_mla_rope(g.view(-1, h, d + emb), cos, sin, 0 if pe_first else d, emb, pos, inter, inverse=True)
        assert torch.equal(xg.grad.cpu().view(-1, h, d + emb), gref)


@pytest.mark.parametrize("inter", [False, True])
@pytest.mark.parametrize("thd", [False, True])
def test_permute_rope_cat_and_its_backward(gpu, inter, thd):
    from loongforge_amd.dsa_fused_kernels import fused_rope_permute_cat

    s, b, h, d, emb = (45, 2, 128, 512, 64) if not thd else (90, 1, 128, 512, 64)
    S = s * b
    cos, sin = _tables(100, emb, inter, torch.float32, True)
    qc = _rand(h, S, d, seed=4)
    pe = _rand(s, b, h, emb, seed=5) if not thd else _rand(S, h, emb, seed=5)
    cu = torch.tensor([0, 33, 90], dtype=torch.int32) if thd else None
    pos = R.thd_positions(cu, S) if thd else torch.arange(S) // b
    ref = R.fused_rope_permute_cat(qc, pe.view(S, h, emb), cos, sin, pos, inter)
    qcg, peg = qc.to(gpu).requires_grad_(True), pe.to(gpu).requires_grad_(True)
    out = fused_rope_permute_cat(qcg, peg, cos.to(gpu), sin.to(gpu), cu.to(gpu) if thd else None, 0, 1, inter)
    assert out.shape == ((s, b, h, d + emb) if not thd else (S, h, d + emb))
    assert torch.equal(out.detach().cpu().view(S, h, d + emb), ref)
    g = _rand(*out.shape, seed=6)
    out.backward(g.to(gpu))
    gqc, gpe = R.fused_rope_permute_cat_bwd(g.view(S, h, d + emb), d, cos, sin, pos, inter)
    assert torch.equal(qcg.grad.cpu(), gqc)
    assert torch.equal(peg.grad.cpu().view(S, h, emb), gpe)


@pytest.mark.parametrize("inter", [False, True])
@pytest.mark.parametrize("thd", [False, True])
def test_absorbed_key_rope_and_its_backward(gpu, inter, thd):
    from loongforge_amd.dsa_fused_kernels import fused_apply_mla_rope_for_absorb_kv

    s, b, h, kd, emb = (40, 2, 16, 128, 64) if not thd else (75, 1, 128, 128, 64)
    T = s * b
    cos, sin = _tables(90, emb, inter, BF if inter else torch.float32, True)
    kv = _rand(s, b, h, kd, seed=7) if not thd else _rand(T, h, kd, seed=7)
    ke = _rand(s, b, 1, emb, seed=8) if not thd else _rand(T, 1, emb, seed=8)
    cu = torch.tensor([0, 5, 70, 75], dtype=torch.int32) if thd else None
    pos = R.thd_positions(cu, T) if thd else torch.arange(T) // b
    ref = R.absorb_kv(kv.view(T, h, kd), ke.view(T, emb), cos, sin, pos, inter)
    kvg, keg = kv.to(gpu).requires_grad_(True), ke.to(gpu).requires_grad_(True)
    key = fused_apply_mla_rope_for_absorb_kv(kvg, keg, cos.to(gpu), sin.to(gpu), emb, kd, cu.to(gpu) if thd else None, 0, 1, inter)
    assert key.shape == ((s, b, h, kd + emb) if not thd else (T, h, kd + emb))
    assert torch.equal(key.detach().cpu().view(T, h, kd + emb), ref)
    g = _rand(*key.shape, seed=9)
    key.backward(g.to(gpu))
    dkv, demb = R.absorb_kv_bwd(g.view(T, h, kd + emb), kd, cos, sin, pos, inter)
    assert torch.equal(kvg.grad.cpu().view(T, h, kd), dkv)
    # the head-sum runs in a different order: after the rounding to bf16 that is at most one unit in the last place
    got = keg.grad.cpu().view(T, emb).float()
    err = (got - demb.float()).abs()
    assert (err <= 2.0 ** -7 * demb.float().abs().clamp_min(1e-3) * 4).all()
    assert (err == 0).float().mean().item() > 0.9


def test_argument_errors_of_the_rope_entry(gpu):
    from loongforge_amd import ops

    x = torch.zeros(4, 2, 20, dtype=BF, device=gpu)
    cos = torch.zeros(8, 12, device=gpu)
    with pytest.raises(ValueError):          # emb_dim 12 is not a multiple of 8
        ops.rope_rows(x[:, :, 8:], x[:, :, 8:], cos, cos, 0, 0)
    with pytest.raises(ValueError):
        ops.rope_rows(x.float(), x.float(), cos, cos, 0, 0)
