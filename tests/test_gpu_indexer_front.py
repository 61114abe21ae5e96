"""GPU parity of the fused indexer front end (LayerNorm -> RoPE -> Hadamard rotation -> e4m3 quantiser in one
kernel): bit for bit against the CPU oracle, and against the separate kernels it replaces."""
import pytest
import torch

from oracle import front_oracle as F
from oracle import rope_oracle as R

pytestmark = pytest.mark.gpu


def _case(seed, tokens, heads, scale=2.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(tokens, heads, 128, generator=g) * scale).to(torch.bfloat16)
    w, b = torch.randn(128, generator=g), torch.randn(128, generator=g)
    hw = torch.randn(tokens, heads, generator=g)
    pos = torch.randint(0, 96, (tokens,), generator=g, dtype=torch.int32)
    return x, w, b, hw, pos


def _same(got, ref):
    x8, si, rows, ws = got
    r8, rs, rrows, rws = ref
    assert torch.equal(rows.cpu(), rrows), "rows that were quantised"
    assert torch.equal(x8.cpu().view(torch.uint8), r8.view(torch.uint8)) and torch.equal(si.cpu(), rs)
    if rws is not None:
        assert torch.equal(ws.cpu(), rws)


@pytest.mark.parametrize("pairing", [R.ADJACENT, R.SPLIT])
@pytest.mark.parametrize("table_dtype", [torch.bfloat16, torch.float32])
def test_front_end_kernel_equals_the_oracle_bit_for_bit(gpu, pairing, table_dtype):
    from loongforge_amd import ops

    cos, sin = R.rope_tables(96, 64, dtype=table_dtype)
    # key side: one row per token, LayerNorm, positions from a table (packed documents)
    x, w, b, hw, pos = _case(1, 333, 1)
    x[7] = 0                                     # LayerNorm of a zero row is the bias
    x[8] = 3.0                                   # ... and so is that of a constant row
    got = ops.indexer_front_e4m3(x.to(gpu), 1, w.to(gpu), b.to(gpu), 1e-6, cos.to(gpu), sin.to(gpu), pairing, pos.to(gpu),
                                 1, True, return_rows=True)
    _same(got, F.indexer_front(x, 1, w, b, 1e-6, cos, sin, pairing, pos, 1, True))
    # query side: 64 rows per token, no LayerNorm, position = token // batch, scaled head weights
    x, w, b, hw, pos = _case(2, 190, 64)
    got = ops.indexer_front_e4m3(x.to(gpu), 64, None, None, 0.0, cos.to(gpu), sin.to(gpu), pairing, None, 2, True,
                                 hw.to(gpu), 128 ** -0.5, return_rows=True)
    _same(got, F.indexer_front(x, 64, None, None, 0.0, cos, sin, pairing, None, 2, True, hw, 128 ** -0.5))
    # no rotation (models that do not rotate their indexer activations)
    x, w, b, hw, pos = _case(3, 50, 4)
    got = ops.indexer_front_e4m3(x.to(gpu), 4, None, None, 0.0, cos.to(gpu), sin.to(gpu), pairing, pos.to(gpu), 1, False,
                                 return_rows=True)
    _same(got, F.indexer_front(x, 4, None, None, 0.0, cos, sin, pairing, pos, 1, False))


def test_front_end_kernel_equals_the_separate_kernels(gpu):
    """The stages as the separate kernels run them: torch LayerNorm (fp32 statistics in torch's own summation
    order: a bf16 step apart now and then), the in-place rotary kernel, the rotation + quantiser kernel."""
    from loongforge_amd import ops

    x, w, b, hw, pos = _case(4, 2048, 1)
    cos, sin = R.rope_tables(96, 64, dtype=torch.bfloat16)
    xd, cd, sd, pd = x.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu)
    x8, si, rows, _ = ops.indexer_front_e4m3(xd, 1, w.to(gpu), b.to(gpu), 1e-5, cd, sd, R.SPLIT, pd, 1, True, return_rows=True)
    v = torch.nn.functional.layer_norm(xd.float(), (128,), w.to(gpu), b.to(gpu), 1e-5).to(torch.bfloat16)
    pe = v[:, :, :64]
    ops.rope_rows(pe, pe, cd, sd, ops.ROPE_SPLIT, ops.ROPE_SPLIT, False, pd, 1)
    r8, rs, rrows = ops.rotate_quant_e4m3(v, return_rotated=True)
    err = (rows.float() - rrows.float()).abs()
    assert (err <= 2.0 ** -7 * rrows.float().abs() + 2.0 ** -9 * rrows.float().abs().amax(-1, keepdim=True)).all()
    assert (err == 0).float().mean().item() > 0.97
    # without LayerNorm every stage is exact arithmetic on the same values: identical bits
    x8b, sib, rowsb, _ = ops.indexer_front_e4m3(xd, 1, None, None, 0.0, cd, sd, R.SPLIT, pd, 1, True, return_rows=True)
    v2 = xd.clone()
    pe2 = v2[:, :, :64]
    ops.rope_rows(pe2, pe2, cd, sd, ops.ROPE_SPLIT, ops.ROPE_SPLIT, False, pd, 1)
    r8, rs, rrows = ops.rotate_quant_e4m3(v2, return_rotated=True)
    assert torch.equal(rowsb, rrows) and torch.equal(x8b.view(torch.uint8), r8.view(torch.uint8)) and torch.equal(sib, rs)
    with pytest.raises(ValueError):
        ops.indexer_front_e4m3(xd, 1, w.to(gpu), None)
    with pytest.raises(ValueError):
        ops.indexer_front_e4m3(xd, 3)


class _Linear(torch.nn.Module):
    def __init__(self, n_in, n_out, **_):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty(n_out, n_in))

    def forward(self, x):
        return torch.nn.functional.linear(x, self.weight.to(x.dtype)), None


class _Norm(torch.nn.LayerNorm):
    def __init__(self, config=None, hidden_size=None, eps=1e-5):
        super().__init__(hidden_size, eps=eps)

    def forward(self, x):
        return super().forward(x.float()).to(x.dtype)


@pytest.mark.parametrize("packed", [False, True])
def test_indexer_module_with_the_front_end_inside_the_kernel(gpu, packed):
    """DSAIndexerFused.forward with the fused front end (projections -> one kernel per side) against the
    same module running k_norm, the rotary kernel and the rotating quantiser one after the other: same
    selection, same scores to the rounding of the LayerNorm statistics, and gradients of every indexer
    weight (the LayerNorm's included) that agree."""
    import copy
    from types import SimpleNamespace

    from loongforge_amd import dsa_fused
    from loongforge_amd.megatron_compat import PackedSeqParams

    S, Hi, hid, qlr, K = 384, 8, 96, 48, 64
    cfg = SimpleNamespace(qk_pos_emb_head_dim=64, v_head_dim=128, kv_lora_rank=512, apply_rope_fusion=True,
                          num_attention_heads=16, kv_channels=192, num_layers=2, hidden_size=hid, q_lora_rank=qlr,
                          dsa_indexer_n_heads=Hi, dsa_indexer_head_dim=128, dsa_indexer_topk=K, dsa_indexer_loss_coeff=1.0,
                          rope_type="rope", rotary_percent=1.0, rotary_base=10000, init_method=None, layernorm_epsilon=1e-5,
                          dsa_indexer_rotate_activation=True, enable_chunkpipe=False)
    sub = dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm, linear_weights_proj=_Linear)
    torch.manual_seed(11)
    fused = dsa_fused.DSAIndexerFused(cfg, sub)
    for p in fused.parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    with torch.no_grad():
        fused.k_norm.weight.add_(0.2 * torch.randn(128))
        fused.k_norm.bias.add_(0.2 * torch.randn(128))
    fused = fused.to(gpu)
    staged = copy.deepcopy(fused)
    staged.indexer_kernel.supports_fused_front_end = False           # instance attribute: this copy keeps the separate stages
    g = torch.Generator().manual_seed(12)
    shape = (S, hid) if packed else (S, 1, hid)
    x = torch.randn(*shape, generator=g).to(torch.bfloat16).to(gpu)
    qr = torch.randn(*shape[:-1], qlr, generator=g).to(torch.bfloat16).to(gpu)
    psp = None
    if packed:
        cu = torch.tensor([0, 100, 101, 384], dtype=torch.int32, device=gpu)
        psp = PackedSeqParams(qkv_format="thd", cu_seqlens_q=cu, cu_seqlens_kv=cu, max_seqlen_q=283, max_seqlen_kv=283)
    assert fused._fused_front_end(x, psp) is not None and staged._fused_front_end(x, psp) is None
    sc1, id1 = fused(x, qr, psp)
    sc2, id2 = staged(x, qr, psp)
    fin = torch.isfinite(sc2)
    assert torch.equal(torch.isfinite(sc1), fin)
    tol = 5e-3 * sc2[fin].abs().max().item()
    assert (sc1[fin] - sc2[fin]).abs().max().item() <= tol
    assert (torch.sort(id1, 1).values == torch.sort(id2, 1).values).float().mean().item() > 0.99
    gsc = torch.randn(S, K, generator=torch.Generator().manual_seed(13)).to(gpu)
    torch.where(fin, sc1, torch.zeros_like(sc1)).mul(gsc).sum().backward()
    torch.where(fin, sc2, torch.zeros_like(sc2)).mul(gsc).sum().backward()
    for (n, a), b in zip(fused.named_parameters(), staged.parameters()):
        assert a.grad is not None and b.grad is not None, n
        scale = b.grad.float().abs().max().item()
        assert (a.grad.float() - b.grad.float()).abs().max().item() <= 3e-2 * scale, n
