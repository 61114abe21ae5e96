"""GPU parity: sparse backward of the indexer logits, and the autograd wrapper around the indexer."""
import pytest
import torch

from oracle import dsa_oracle as O

pytestmark = pytest.mark.gpu


def _reference(aux, idx, g, noise=2.0 ** -18):
    """fp64 autograd through the gathered logits + the set of (query, head) rows / keys touched by a
    ReLU gate whose exact pre-activation is within fp32 accumulation noise of zero (there the gate
    may legitimately fall on either side)."""
    q8f, k8f = aux["q8"], aux["k8"]
    qf = q8f.double().requires_grad_(True)
    kf = k8f.double().requires_grad_(True)
    wf = aux["weight_scaled"].double().requires_grad_(True)
    sel = O.gathered_indexer_logits(qf, wf, kf, aux["k_scale"], idx, dtype=torch.float64)
    (torch.where(idx >= 0, sel, torch.zeros_like(sel)) * g.double()).sum().backward()
    safe = idx.clamp(min=0).long()
    ksel = k8f.double()[safe]
    rex = torch.einsum("mhd,mkd->mhk", q8f.double(), ksel)
    mag = torch.einsum("mhd,mkd->mhk", q8f.double().abs(), ksel.abs())
    amb = (rex.abs() <= noise * mag) & (idx >= 0)[:, None, :]
    amb_key = torch.zeros(k8f.shape[0], dtype=torch.bool)
    amb_key[safe[amb.any(1)]] = True
    return qf.grad, kf.grad, wf.grad, amb.any(-1), amb_key


@pytest.mark.parametrize("S,Hi,K,seed", [(256, 64, 128, 1), (300, 32, 128, 2), (200, 64, 192, 3)])
def test_indexer_bwd_against_oracle(gpu, S, Hi, K, seed):
    from loongforge_amd import ops

    iq, ik, w = O.make_indexer_inputs(S, Hi, 128, seed=seed)
    _, idx, aux = O.indexer_forward(iq, ik, w, K, 0, None)
    g = torch.randn(S, K, generator=torch.Generator().manual_seed(seed + 1))
    g = torch.where(idx >= 0, g, torch.zeros_like(g))
    rq, rk, rw, amb_qh, amb_key = _reference(aux, idx, g)
    args = (g.to(gpu), aux["q8"].to(gpu), aux["k8"].to(gpu), aux["k_scale"].to(gpu),
            aux["weight_scaled"].to(gpu).contiguous(), idx.to(gpu))
    dq, dk, dw = ops.indexer_bwd(*args)
    dq2, dk2, dw2 = ops.indexer_bwd(*args)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dw, dw2)      # bit-identical
    eq = (dq.double().cpu() - rq).abs().masked_fill(amb_qh[..., None], 0)
    ek = (dk.double().cpu() - rk).abs().masked_fill(amb_key[:, None], 0)
    ew = (dw.double().cpu() - rw).abs()
    assert eq.max().item() <= 1e-4 * rq.abs().max().item()
    assert ek.max().item() <= 4e-3 * rk.abs().max().item()       # a key's rows are summed in fp32 from bf16 rows
    assert ew.max().item() <= 1e-4 * rw.abs().max().item()


def test_indexer_bwd_with_a_repeated_id_returns_nan_keys(gpu):
    from loongforge_amd import ops

    iq, ik, w = O.make_indexer_inputs(256, 64, 128, seed=5)
    _, idx, aux = O.indexer_forward(iq, ik, w, 128, 0, None)
    idx = idx.clone()
    idx[200, 3] = idx[200, 17]
    g = torch.ones(256, 128)
    dq, dk, dw = ops.indexer_bwd(g.to(gpu), aux["q8"].to(gpu), aux["k8"].to(gpu), aux["k_scale"].to(gpu),
                                 aux["weight_scaled"].to(gpu).contiguous(), idx.to(gpu))
    assert torch.isnan(dk).all()


def test_indexer_kernel_module_forward_and_backward(gpu):
    """DSAIndexerKernel with the reference's call signature: unpadded head count / head dim (the
    reference's own CPU-sized configuration uses 4 heads of dim 64), packed documents, autograd."""
    from loongforge_amd.dsa_fused_kernels import DSAIndexerKernel
    from loongforge_amd.megatron_compat import PackedSeqParams

    S, Hi, D, K = 384, 4, 64, 64
    cu = torch.tensor([0, 100, 257, 384], dtype=torch.int32)
    iq, ik, w = O.make_indexer_inputs(S, Hi, D, seed=7, w_uniform=True)
    sc_ref, idx_ref, aux = O.indexer_forward(iq, ik, w, K, 0, cu, dtype=torch.float64)
    psp = PackedSeqParams(qkv_format="thd", cu_seqlens_q=cu.to(gpu), cu_seqlens_kv=cu.to(gpu), max_seqlen_q=157,
                          max_seqlen_kv=157)
    q = iq.to(gpu).requires_grad_(True)
    k = ik.to(gpu).requires_grad_(True)
    wt = w.to(gpu).requires_grad_(True)
    sc, ids = DSAIndexerKernel()(q, k, wt, K, 0, psp)
    assert sc.shape == (S, K) and ids.dtype == torch.int32
    noise = 1e-4 * sc_ref[torch.isfinite(sc_ref)].abs().max().item()
    assert torch.equal(torch.isfinite(sc.cpu()), torch.isfinite(sc_ref))
    fin = torch.isfinite(sc_ref)
    assert (sc.cpu()[fin].double() - sc_ref[fin].double()).abs().max().item() <= noise   # both sorted descending
    v = ids.cpu() >= 0
    ks, ke = aux["ks"], aux["ke"]
    assert ((ids.cpu() >= ks[:, None]) | ~v).all() and ((ids.cpu() < ke[:, None]) | ~v).all()
    # backward: gradient of sum(score * g) through the HIP indexer backward vs the oracle
    g = torch.randn(S, K, generator=torch.Generator().manual_seed(8))
    torch.where(torch.isfinite(sc), sc, torch.zeros_like(sc)).mul(g.to(gpu)).sum().backward()
    idc = ids.cpu()
    gz = torch.where(idc >= 0, g, torch.zeros_like(g))
    d_q, d_k, d_w = O.indexer_bwd(gz, aux["q8"], aux["k8"], aux["q_scale"], aux["k_scale"], aux["weight_scaled"], idc,
                                  dtype=torch.float64)
    # the oracle's d_w is w.r.t. the un-scaled weights already (d_w' * q_scale * d^-0.5)
    for name, got, ref in (("d_q", q.grad, d_q), ("d_k", k.grad, d_k), ("d_w", wt.grad, d_w)):
        err = (got.double().cpu() - ref).abs()
        lim = 2e-2 * ref.abs().max().item()       # bf16 grads; ReLU-gate flips are rarer than 1e-4 of pairs
        assert (err > lim).float().mean().item() < 1e-3, name
