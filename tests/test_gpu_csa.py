"""GPU parity of the compressed-sparse-attention callers: the fp8 indexer over compressed keys
(CSAIndexerKernel) against the oracle, single sequence and packed, forward and backward; and the
attention call over [keys | compressed keys] with ids from the window / compressed-key helpers."""
from types import SimpleNamespace

import pytest
import torch

from oracle import csa_oracle as C
from oracle import dsa_oracle as O
from tests.gpu_util import FP32_DKV_EXCESS_LIMIT, FP32_DQ_EXCESS_LIMIT, assert_close, assert_mla_grads

pytestmark = pytest.mark.gpu


def _check_forward(sc, ids_global, sc_ref, aux, k_eff):
    """Scores are compared as sorted rows (slot order is not part of the contract); ids must name
    visible keys, each at most once, and carry the score the oracle's dense logits hold there."""
    S = sc.shape[0]
    assert sc.shape == (S, k_eff) and ids_global.shape == (S, k_eff)
    fin_ref = torch.isfinite(sc_ref)
    live = ids_global >= 0
    assert torch.equal(live.sum(1), fin_ref.sum(1))
    assert torch.equal(torch.isfinite(sc), live)
    scale = sc_ref[fin_ref].abs().max().item()
    a = torch.where(live, sc, torch.full_like(sc, -1e30)).sort(dim=1, descending=True).values
    b = torch.where(fin_ref, sc_ref.float(), torch.full_like(sc, -1e30)).sort(dim=1, descending=True).values
    assert (a - b).abs().max().item() <= 1e-4 * scale
    ks, ke = aux["ks"], aux["ke"]
    assert ((ids_global >= ks[:, None]) & (ids_global < ke[:, None]) | ~live).all()
    looked_up = aux["logits"].gather(1, ids_global.clamp(min=0).long())
    assert ((looked_up - sc).abs()[live]).max().item() <= 1e-4 * scale
    for i in range(0, S, 7):                                            # no key twice in a row
        row = ids_global[i][live[i]]
        assert row.unique().numel() == row.numel()


def _check_backward(q, k, wt, sc, ids_global, aux, seed):
    g = torch.randn(sc.shape, generator=torch.Generator().manual_seed(seed))
    torch.where(torch.isfinite(sc), sc, torch.zeros_like(sc)).mul(g.to(sc.device)).sum().backward()
    gz = torch.where(ids_global >= 0, g, torch.zeros_like(g))
    d_q, d_k, d_w = O.indexer_bwd(gz, aux["q8"], aux["k8"], aux["q_scale"], aux["k_scale"], aux["weight_scaled"],
                                  ids_global, dtype=torch.float64)
    assert q.grad.shape == q.shape and k.grad.shape == k.shape and wt.grad.shape == wt.shape
    for name, got, ref in (("d_q", q.grad.squeeze(1), d_q), ("d_k", k.grad.squeeze(1), d_k), ("d_w", wt.grad.squeeze(1), d_w)):
        err = (got.double().cpu() - ref).abs()
        lim = 2e-2 * ref.abs().max().item()       # bf16 grads; ReLU-gate flips are rarer than 1e-4 of pairs
        assert (err > lim).float().mean().item() < 1e-3, name


@pytest.mark.parametrize("sq,ratio,topk,offset,heads", [(512, 4, 64, 0, 64), (300, 4, 512, 212, 32), (256, 1, 96, 0, 8)])
def test_csa_indexer_single_sequence(gpu, sq, ratio, topk, offset, heads):
    from loongforge_amd.csa_kernels import CSAIndexerKernel

    sk = (sq + offset) // ratio
    iq, ik_full, w = O.make_indexer_inputs(sq, heads, 128, seed=11, w_uniform=True)
    ik = torch.randn(sk, 128, generator=torch.Generator().manual_seed(12)).to(torch.bfloat16)
    sc_ref, idx_ref, aux = C.csa_indexer_forward(iq, ik, w, topk, ratio, offset)
    k_eff = min(topk, sk)
    q = iq.to(gpu).unsqueeze(1).requires_grad_(True)
    k = ik.to(gpu).unsqueeze(1).requires_grad_(True)
    wt = w.to(gpu).unsqueeze(1).requires_grad_(True)
    sc, ids = CSAIndexerKernel(ratio)(q, k, wt, topk, offset)
    assert ids.dtype == torch.int32
    _check_forward(sc.detach().cpu(), ids.cpu(), sc_ref, aux, k_eff)
    # the first queries see no complete compressed key: the window is kept at one key (key 0)
    first = ids.cpu()[0]
    assert sorted(first[first >= 0].tolist()) == list(range(max((offset + 1) // ratio, 1)))
    _check_backward(q, k, wt, sc, ids.cpu(), aux, seed=13)


def test_csa_indexer_packed_returns_segment_local_ids(gpu):
    from loongforge_amd.csa_kernels import CSAIndexerKernel
    from loongforge_amd.megatron_compat import PackedSeqParams

    ratio, topk, heads = 4, 32, 64
    lens = [150, 3, 201, 30]
    lens_c = [n // ratio for n in lens]
    cu_q = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    cu_kv = torch.tensor([0] + list(torch.tensor(lens_c).cumsum(0)), dtype=torch.int32)
    sq, sk = int(cu_q[-1]), int(cu_kv[-1])
    iq, _, w = O.make_indexer_inputs(sq, heads, 128, seed=21, w_uniform=True)
    ik = torch.randn(sk, 128, generator=torch.Generator().manual_seed(22)).to(torch.bfloat16)
    sc_ref, idx_ref, aux = C.csa_indexer_forward(iq, ik, w, topk, ratio, 0, cu_q, cu_kv, max_seqlen_kv=max(lens_c))
    psp = PackedSeqParams(qkv_format="thd", cu_seqlens_q=cu_q.to(gpu), cu_seqlens_kv=cu_kv.to(gpu),
                          max_seqlen_q=max(lens), max_seqlen_kv=max(lens_c))
    q = iq.to(gpu).unsqueeze(1).requires_grad_(True)
    k = ik.to(gpu).unsqueeze(1).requires_grad_(True)
    wt = w.to(gpu).unsqueeze(1).requires_grad_(True)
    sc, ids = CSAIndexerKernel(ratio)(q, k, wt, topk, 0, psp)
    idc = ids.cpu()
    width = (aux["ke"] - aux["ks"])[:, None]
    assert ((idc >= 0) & (idc < width) | (idc == -1)).all()                     # relative to the segment's first key
    ids_global = torch.where(idc >= 0, idc + aux["ks"][:, None], idc)
    _check_forward(sc.detach().cpu(), ids_global, sc_ref, aux, min(topk, max(lens_c)))
    empty = (aux["ke"] == aux["ks"])
    assert empty.any() and (idc[empty] == -1).all() and torch.isinf(sc.detach().cpu()[empty]).all()
    _check_backward(q, k, wt, sc, ids_global, aux, seed=23)


def test_window_plus_compressed_attention_equals_dense_masked_attention(gpu):
    """The single-sequence CSA attention call (deepseek_v4_csa.py:2341-2346, :2806-2816): keys are
    [raw latent rows | compressed rows], slots are [window ids | every compressed id], the kernel's own
    causal test is switched off by chunk_offset = number of keys, a per-head sink joins the denominator.
    Expected result: dense attention in fp64 under the mask stated directly (raw key r visible to query
    p iff p - window < r <= p; compressed key c iff its last raw position c*ratio + ratio - 1 <= p)."""
    from loongforge_amd.csa_kernels import get_compress_topk_idxs, get_window_topk_idxs
    from loongforge_amd.dsa_fused_kernels import DSADotProductAttention

    sq, ratio, window, H = 200, 4, 64, 128
    n_c = sq // ratio
    g = torch.Generator().manual_seed(31)
    q = torch.randn(sq, H, 576, generator=g).to(torch.bfloat16)
    kv_full = torch.randn(sq + n_c, 576, generator=g).to(torch.bfloat16)
    dout = torch.randn(sq, H, 512, generator=g).to(torch.bfloat16)
    sink = torch.randn(H, generator=g)
    sm_scale = 192 ** -0.5
    ids = torch.cat([get_window_topk_idxs(window, 1, sq, "cpu"), get_compress_topk_idxs(ratio, 1, sq, sq, "cpu")], dim=-1)
    assert ids.shape == (1, sq, window + n_c)

    pos = torch.arange(sq)[:, None]
    raw = torch.arange(sq)[None, :]
    comp_last = (torch.arange(n_c) * ratio + ratio - 1)[None, :]
    mask = torch.cat([(raw <= pos) & (raw > pos - window), comp_last <= pos], dim=1)              # [sq, sq + n_c]
    qd = q.double().requires_grad_(True)
    kd = kv_full.double().requires_grad_(True)
    s = torch.einsum("shd,kd->shk", qd, kd) * sm_scale
    s = s.masked_fill(~mask[:, None, :], float("-inf"))
    s = torch.cat([s, sink.double()[None, :, None].expand(sq, H, 1)], dim=-1)
    p = torch.softmax(s, dim=-1)[..., :-1]
    ref = torch.einsum("shk,kd->shd", p, kd[:, :512])
    (ref * dout.double()).sum().backward()

    cfg = SimpleNamespace(qk_pos_emb_head_dim=64, v_head_dim=128, kv_lora_rank=512, apply_rope_fusion=False,
                          num_attention_heads=H, kv_channels=192, num_layers=2)
    attn = DSADotProductAttention(cfg, softmax_scale=sm_scale)
    qg = q.to(gpu).requires_grad_(True)
    kg = kv_full.to(gpu).requires_grad_(True)
    out = attn(qg.unsqueeze(1), kg.unsqueeze(1), ids.int().to(gpu), kv_full.shape[0], None, attn_sink=sink.to(gpu))
    assert out.shape == (1, sq, H, 512)
    assert_close(out[0], ref, "out")
    out.backward(dout.to(gpu).unsqueeze(0))
    # gradients: element by element against the oracle with the kernels' rounding points, then the distance
    # from the dense fp64 gradients, which a bf16-operand backward cannot bring under the elementwise bound
    d = (qg.grad.float().cpu().double() - qd.grad).abs() - (2e-2 + 1e-2 * qd.grad.abs())
    assert d.max().item() <= FP32_DQ_EXCESS_LIMIT
    assert_mla_grads(qg.grad, kg.grad, q, kv_full, ids[0].int(), dout, kv_full.shape[0], sm_scale, attn_sink=sink,
                     out=out[0])
    d = (kg.grad.float().cpu().double() - kd.grad).abs() - (2e-2 + 1e-2 * kd.grad.abs())
    assert d.max().item() <= FP32_DKV_EXCESS_LIMIT
