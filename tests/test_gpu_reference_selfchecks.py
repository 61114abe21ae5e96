"""The reference's own self-check recipes for the sparse attention kernels, run on the HIP path.

ops/tilelang_ops/sparse_mla_fwd.py:268-317, 335-351 and ops/tilelang_ops/sparse_mla_bwd.py:322-349,
370-372 build their inputs like this (seed 0, ids of query t = randperm(max(1, t))[:topk] padded with
the out-of-range sentinel s_kv, a chunk offset of 1024) and accept a result when
1 - 2<x, y> / (|x|^2 + |y|^2) stays below 1e-1 (out) and 1e-4 (dq, dkv)
(ops/tilelang_ops/utils.py:19-74).  Here that acceptance rule is applied next to this build's
elementwise tolerance, against the CPU oracle.
"""
import pytest
import torch

from oracle import dsa_oracle as O
from tests.gpu_util import assert_close, assert_mla_grads

pytestmark = pytest.mark.gpu


def _dissimilarity(x, y):
    x, y = x.detach().double().cpu(), y.detach().double().cpu()
    return 1.0 - (2 * (x * y).sum() / (x * x + y * y).sum()).item()


def _recipe(S, SKV, H, topk, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(S, H, 576, generator=g).to(torch.bfloat16)
    kv = torch.randn(SKV, 576, generator=g).to(torch.bfloat16)
    do = torch.randn(S, H, 512, generator=g).to(torch.bfloat16)
    idx = torch.full((S, topk), SKV, dtype=torch.int32)
    for t in range(S):
        i_i = torch.randperm(max(1, t), generator=g)[:topk]
        idx[t, : len(i_i)] = i_i.int()
    return q, kv, do, idx


def test_forward_recipe_s2048_skv4096_h128_topk512_offset1024(gpu):
    from loongforge_amd import ops

    q, kv, _, idx = _recipe(2048, 4096, 128, 512)
    sm = 576 ** -0.5
    out, lse, _ = ops.sparse_mla_fwd(q.to(gpu), kv.to(gpu), idx.to(gpu), 1024, sm)
    ro, rl, _ = O.sparse_mla_fwd(q, kv, idx, 1024, sm, 512)
    assert _dissimilarity(out, ro) <= 1e-1                     # the reference's own bar
    assert _dissimilarity(out, ro) <= 1e-5
    assert_close(out, ro, "out")
    assert (lse.cpu() - rl).abs().max().item() < 1e-4


def test_backward_recipe_s2048_skv8192_h64_topk512_offset1024(gpu):
    from loongforge_amd import ops

    q, kv, do, idx = _recipe(2048, 8192, 64, 512)
    sm = 576 ** -0.5
    qd, kvd, idd, dod = q.to(gpu), kv.to(gpu), idx.to(gpu), do.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(qd, kvd, idd, 1024, sm)
    dq, dkv = ops.sparse_mla_bwd(qd, kvd, out, dod, idd, lse, 1024, sm)
    rdq, rdkv = O.sparse_mla_bwd(q, kv, idx, do, 1024, sm, 512)
    assert _dissimilarity(dq, rdq) <= 1e-4 and _dissimilarity(dkv, rdkv) <= 1e-4     # the reference's own bar
    assert_mla_grads(dq, dkv, q, kv, idx, do, 1024, sm, out=out, lse=lse)


def test_indexer_recipe_m1024_n2048_h64_forward_and_dense_backward(gpu):
    """ops/tilelang_ops/lightning_indexer.py:744-773 (inputs: seed 42, q cast straight to e4m3, k
    quantised with scale 448 / amax, weights * 128^-0.5) and :11-65 (the torch baseline of the forward
    and of its dense backward, restated here in fp64).  With every key selected, the sparse backward
    of this build is that dense backward."""
    from loongforge_amd import ops

    M, N, Hi, D = 1024, 2048, 64, 128
    g = torch.Generator().manual_seed(42)
    q_bf = torch.randn(M, Hi, D, generator=g).to(torch.bfloat16)
    k_bf = torch.randn(N, D, generator=g).to(torch.bfloat16)
    q_s = torch.randn(M, Hi, generator=g) * D ** -0.5
    q8 = q_bf.to(torch.float8_e4m3fn)
    amax = k_bf.float().abs().amax(dim=-1).clamp_min(1e-6)
    scale = 448.0 / amax
    k8 = (k_bf.float() * scale.unsqueeze(-1)).to(torch.float8_e4m3fn)
    k_s = (1.0 / scale).float()
    # baseline, fp64
    qd, kd = q8.double(), k8.double()
    logits = torch.einsum("mhd,nd->mhn", qd, kd)
    relu = torch.relu(logits)
    lsum = (relu * q_s.double().unsqueeze(-1)).sum(dim=1)
    ref = lsum * k_s.double().unsqueeze(0)

    ks = torch.zeros(M, dtype=torch.int32)
    ke = torch.full((M,), N, dtype=torch.int32)
    dev = lambda t: t.to(gpu)
    got = ops.indexer_logits(dev(q8), dev(q_s), dev(k8), dev(k_s), dev(ks), dev(ke)).cpu().double()
    rel = (got - ref).abs() / (ref.abs() + 1e-8)
    # the reference prints the share of entries within 1e-4 relative; a score is a sum of 64 signed terms
    # about 100x its own size, and the matrix pipe's fp8 dot products carry ~1e-5 of the term size
    assert (rel < 1e-4).double().mean().item() > 0.9
    assert (rel < 1e-3).double().mean().item() > 0.99
    assert (got - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()

    d_out = torch.randn(M, N, generator=g)
    d_lsum = d_out.double() * k_s.double().unsqueeze(0)
    d_relu = d_lsum.unsqueeze(1) * q_s.double().unsqueeze(-1)
    r_dqs = (d_lsum.unsqueeze(1) * relu).sum(dim=-1)
    d_logits = d_relu * (logits > 0)
    r_dq = torch.einsum("mhn,nd->mhd", d_logits, kd)
    r_dk = torch.einsum("mhn,mhd->nd", d_logits, qd)
    ids = torch.arange(N, dtype=torch.int32).unsqueeze(0).expand(M, N).contiguous()
    dq, dk, dw = ops.indexer_bwd(dev(d_out), dev(q8), dev(k8), dev(k_s), dev(q_s), dev(ids))
    # A ReLU gate whose argument is within the matrix pipe's rounding of zero may open on one side and
    # not on the other; such a flip moves the gradient entries it feeds by one whole term.  Hence the
    # reference's global measure (two orders of magnitude tighter than its own bars) and a loose bound
    # on the worst entry; the gate-aware elementwise comparison is in test_gpu_indexer_bwd.py.
    for name, a, b in (("d_q", dq, r_dq), ("d_k", dk, r_dk), ("d_q_s", dw, r_dqs)):
        assert _dissimilarity(a, b) <= 1e-5, name
        err = (a.cpu().double() - b).abs()
        assert err.max().item() <= 5e-2 * b.abs().max().item(), name
