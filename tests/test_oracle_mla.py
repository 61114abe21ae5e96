"""Pins for the oracle's sparse-MLA forward/backward, attention distribution and KL loss."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import dsa_oracle as O


def _inputs(sq, h, K, dqk=24, seed=0, skv=None, q_start=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    skv = sq + q_start if skv is None else skv
    q = torch.randn(sq, h, dqk, generator=g, dtype=dtype)
    kv = torch.randn(skv, dqk, generator=g, dtype=dtype)
    idx = O.causal_random_topk_indices(sq, K, seed + 1, q_start)
    return q, kv, idx


def test_fwd_equals_dense_causal_sdpa_when_topk_covers_prefix():
    sq, h, dqk, dv = 48, 4, 24, 16
    q, kv, idx = _inputs(sq, h, K=64, dqk=dqk)            # K >= prefix for every query
    sm = 0.37
    out, lse, p_out = O.sparse_mla_fwd(q, kv, idx, 0, sm, dv, dtype=torch.float64)
    k = kv.unsqueeze(0).expand(h, -1, -1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k, k[..., :dv], is_causal=True, scale=sm)
    torch.testing.assert_close(out, ref.transpose(0, 1), rtol=1e-10, atol=1e-10)
    # lse against dense logsumexp
    z = torch.einsum("mhd,nd->mhn", q, kv) * sm
    z = z.masked_fill(torch.arange(sq)[None, None, :] > torch.arange(sq)[:, None, None], float("-inf"))
    torch.testing.assert_close(lse, torch.logsumexp(z, -1), rtol=1e-10, atol=1e-10)


def test_fwd_brute_force_general_case_with_invalid_ids():
    sq, h, dqk, dv, K = 20, 3, 12, 8, 6
    q, kv, idx = _inputs(sq, h, K, dqk, seed=3, q_start=4, skv=30)
    idx = idx.clone()
    idx[5, 0] = -1          # padding
    idx[6, 1] = 30          # == s_kv: out of range
    idx[7, 2] = 29          # in range but in the future of query 7 (pos 11)
    idx[8, :] = -1          # a row with no valid slot
    sm = 0.21
    out, lse, p_out = O.sparse_mla_fwd(q, kv, idx, 4, sm, dv, dtype=torch.float64)
    for i in range(sq):
        for hh in range(h):
            sc, rows = [], []
            for t in range(K):
                j = int(idx[i, t])
                ok = j != -1 and 0 <= j < 30 and j <= 4 + i
                assert math.isinf(p_out[i, hh, t].item()) != ok
                if ok:
                    s = float(np.dot(q[i, hh].numpy(), kv[j].numpy()))
                    assert math.isclose(p_out[i, hh, t].item(), s, rel_tol=1e-12, abs_tol=1e-12)
                    sc.append(s * sm)
                    rows.append(j)
            if not sc:
                assert out[i, hh].abs().max() == 0 and lse[i, hh] == float("inf")
                continue
            m = max(sc)
            w = [math.exp(s - m) for s in sc]
            tot = sum(w)
            ref = sum(wi / tot * kv[j, :dv].numpy() for wi, j in zip(w, rows))
            np.testing.assert_allclose(out[i, hh].numpy(), ref, rtol=1e-10, atol=1e-12)
            assert math.isclose(lse[i, hh].item(), m + math.log(tot), rel_tol=1e-12)


def test_fwd_with_sink_matches_the_sink_softmax_written_out():
    # deepseek_v4_csa.py:571-579: weights = exp(s - m) / (sum exp(s - m) + exp(sink - m)) with
    # m = max(max s, sink); the sink has no value row.  Written here as plain loops.
    sq, h, dqk, dv, K = 18, 3, 12, 8, 6
    q, kv, idx = _inputs(sq, h, K, dqk, seed=11, q_start=2, skv=24)
    idx = idx.clone()
    idx[4, :] = -1                                           # no valid slot: only the sink remains
    idx[5, 1] = -1
    sink = torch.tensor([-1.3, 0.4, 7.0], dtype=torch.float64)
    sm = 0.29
    out, lse, _ = O.sparse_mla_fwd(q, kv, idx, 2, sm, dv, dtype=torch.float64, attn_sink=sink)
    for i in range(sq):
        for hh in range(h):
            sc, rows = [], []
            for t in range(K):
                j = int(idx[i, t])
                if j != -1 and 0 <= j < 24 and j <= 2 + i:
                    sc.append(float(np.dot(q[i, hh].numpy(), kv[j].numpy())) * sm)
                    rows.append(j)
            m = max(sc + [float(sink[hh])])
            den = sum(math.exp(s - m) for s in sc) + math.exp(float(sink[hh]) - m)
            ref = np.zeros(dv)
            for s, j in zip(sc, rows):
                ref += math.exp(s - m) / den * kv[j, :dv].numpy()
            np.testing.assert_allclose(out[i, hh].numpy(), ref, rtol=1e-10, atol=1e-12)
            assert math.isclose(lse[i, hh].item(), m + math.log(den), rel_tol=1e-12, abs_tol=1e-12)
    assert torch.equal(lse[4], sink) and out[4].abs().max() == 0
    # a sink far below every logit changes nothing; the weights of a row sum to 1 - sink share
    o0, l0, _ = O.sparse_mla_fwd(q, kv, idx, 2, sm, dv, dtype=torch.float64)
    o1, l1, _ = O.sparse_mla_fwd(q, kv, idx, 2, sm, dv, dtype=torch.float64, attn_sink=torch.full((3,), -800.0, dtype=torch.float64))
    ok = torch.isfinite(l0)
    torch.testing.assert_close(o1[ok], o0[ok], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(l1[ok], l0[ok], rtol=1e-12, atol=1e-12)
    share = 1 - torch.exp(sink[None, :] - lse)
    torch.testing.assert_close(out[ok], o0[ok] * share[ok].unsqueeze(-1), rtol=1e-10, atol=1e-12)


def test_bwd_with_sink_matches_finite_differences():
    sq, h, dqk, dv, K = 6, 2, 8, 4, 4
    q, kv, idx = _inputs(sq, h, K, dqk, seed=13)
    sink = torch.tensor([0.3, -0.8], dtype=torch.float64)
    g = torch.Generator().manual_seed(5)
    dout = torch.randn(sq, h, dv, generator=g, dtype=torch.float64)
    dq, dkv = O.sparse_mla_bwd(q, kv, idx, dout, 0, 0.4, dv, dtype=torch.float64, attn_sink=sink)

    def f(q_, kv_):
        return (O.sparse_mla_fwd(q_, kv_, idx, 0, 0.4, dv, dtype=torch.float64, attn_sink=sink)[0] * dout).sum().item()

    eps = 1e-6
    for (i, hh, d) in [(0, 0, 0), (3, 1, 5), (5, 0, 7)]:
        qp, qm = q.clone(), q.clone()
        qp[i, hh, d] += eps
        qm[i, hh, d] -= eps
        assert math.isclose((f(qp, kv) - f(qm, kv)) / (2 * eps), dq[i, hh, d].item(), rel_tol=1e-6, abs_tol=1e-8)
    for (j, d) in [(0, 0), (2, 3), (4, 6)]:
        kp, km = kv.clone(), kv.clone()
        kp[j, d] += eps
        km[j, d] -= eps
        assert math.isclose((f(q, kp) - f(q, km)) / (2 * eps), dkv[j, d].item(), rel_tol=1e-6, abs_tol=1e-8)


def test_fwd_is_invariant_to_slot_permutation():
    q, kv, idx = _inputs(16, 2, 8, seed=5)
    perm = torch.randperm(8, generator=torch.Generator().manual_seed(9))
    o1, l1, p1 = O.sparse_mla_fwd(q, kv, idx, 0, 0.3, 16, dtype=torch.float64)
    o2, l2, p2 = O.sparse_mla_fwd(q, kv, idx[:, perm], 0, 0.3, 16, dtype=torch.float64)
    torch.testing.assert_close(o1, o2, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(l1, l2, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(p1[:, :, perm], p2, rtol=0, atol=0)


def test_bwd_equals_dense_attention_grads_when_topk_covers_prefix():
    sq, h, dqk, dv = 40, 3, 24, 16
    q, kv, idx = _inputs(sq, h, K=64, dqk=dqk, seed=7)
    g = torch.Generator().manual_seed(11)
    dout = torch.randn(sq, h, dv, generator=g, dtype=torch.float64)
    dq, dkv = O.sparse_mla_bwd(q, kv, idx, dout, 0, 0.4, dv, dtype=torch.float64)
    qd, kvd = q.clone().requires_grad_(True), kv.clone().requires_grad_(True)
    k = kvd.unsqueeze(0).expand(h, -1, -1)
    ref = F.scaled_dot_product_attention(qd.transpose(0, 1), k, k[..., :dv], is_causal=True, scale=0.4)
    ref.backward(dout.transpose(0, 1))
    torch.testing.assert_close(dq, qd.grad, rtol=1e-9, atol=1e-10)
    torch.testing.assert_close(dkv, kvd.grad, rtol=1e-9, atol=1e-10)


def test_bwd_closed_form_matches_autograd_and_dS_sums_to_zero():
    # closed form quoted from the reference kernel (ops/tilelang_ops/sparse_mla_bwd.py:192-205),
    # evaluated with explicit python loops over (query, slot)
    sq, h, dqk, dv, K = 10, 2, 12, 8, 4
    q, kv, idx = _inputs(sq, h, K, dqk, seed=13)
    g = torch.Generator().manual_seed(17)
    dout = torch.randn(sq, h, dv, generator=g, dtype=torch.float64)
    sm = 0.33
    dq, dkv = O.sparse_mla_bwd(q, kv, idx, dout, 0, sm, dv, dtype=torch.float64)
    out, lse, _ = O.sparse_mla_fwd(q, kv, idx, 0, sm, dv, dtype=torch.float64)
    dq_ref, dkv_ref = torch.zeros_like(q), torch.zeros_like(kv)
    for i in range(sq):
        for hh in range(h):
            delta = (out[i, hh] * dout[i, hh]).sum()
            tot = 0.0
            for t in range(K):
                j = int(idx[i, t])
                if j < 0 or j > i:
                    continue
                p = torch.exp((q[i, hh] * kv[j]).sum() * sm - lse[i, hh])
                dp = (dout[i, hh] * kv[j, :dv]).sum()
                ds = p * (dp - delta) * sm
                tot += ds.item()
                dq_ref[i, hh] += ds * kv[j]
                dkv_ref[j] += ds * q[i, hh]
                dkv_ref[j, :dv] += p * dout[i, hh]
            assert abs(tot) < 1e-12
    torch.testing.assert_close(dq, dq_ref, rtol=1e-9, atol=1e-12)
    torch.testing.assert_close(dkv, dkv_ref, rtol=1e-9, atol=1e-12)


def test_bwd_kernel_rounding_form_without_rounding_equals_autograd():
    sq, h, dqk, dv, K = 24, 4, 32, 16, 8
    q, kv, idx = _inputs(sq, h, K, dqk, seed=41, dtype=torch.float32)
    dout = torch.randn(sq, h, dv, generator=torch.Generator().manual_seed(43))
    out, lse, _ = O.sparse_mla_fwd(q, kv, idx, 0, 0.3, dv)
    dq, dkv = O.sparse_mla_bwd_kernel_rounding(q, kv, idx, dout, 0, 0.3, dv, out=out, lse=lse, round_p_ds_bf16=False)
    rdq, rdkv = O.sparse_mla_bwd(q, kv, idx, dout, 0, 0.3, dv)
    torch.testing.assert_close(dq, rdq, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dkv, rdkv, rtol=1e-4, atol=1e-5)


def test_bwd_kernel_rounding_form_matches_loops_with_bf16_casts():
    # the reference kernel's rounding points (ops/tilelang_ops/sparse_mla_bwd.py:192-209) written out
    # as loops over (query, head, slot) in fp64, the two casts done per element
    sq, h, dqk, dv, K = 9, 2, 16, 8, 4
    g = torch.Generator().manual_seed(47)
    q = torch.randn(sq, h, dqk, generator=g).to(torch.bfloat16)
    kv = torch.randn(sq, dqk, generator=g).to(torch.bfloat16)
    dout = torch.randn(sq, h, dv, generator=g).to(torch.bfloat16)
    idx = O.causal_random_topk_indices(sq, K, 48)
    idx[3, 1] = -1
    sm = 0.29
    o32, lse, _ = O.sparse_mla_fwd(q, kv, idx, 0, sm, dv)
    out = o32.to(torch.bfloat16)
    dq, dkv = O.sparse_mla_bwd_kernel_rounding(q, kv, idx, dout, 0, sm, dv, out=out, lse=lse)
    bf = lambda x: torch.tensor(x, dtype=torch.float32).to(torch.bfloat16).double().item()
    qd, kd, dd, od = q.double(), kv.double(), dout.double(), out.double()
    dq_ref, dkv_ref = torch.zeros(sq, h, dqk, dtype=torch.float64), torch.zeros(sq, dqk, dtype=torch.float64)
    n_changed = 0
    for i in range(sq):
        for hh in range(h):
            delta = (od[i, hh] * dd[i, hh]).sum().item()
            for t in range(K):
                j = int(idx[i, t])
                if j < 0 or j > i:
                    continue
                p = math.exp((qd[i, hh] * kd[j]).sum().item() * sm - lse[i, hh].item())
                dp = (dd[i, hh] * kd[j, :dv]).sum().item()
                ds = p * (dp - delta) * sm
                pb, dsb = bf(p), bf(ds)
                n_changed += (pb != p) + (dsb != ds)
                dq_ref[i, hh] += dsb * kd[j]
                dkv_ref[j] += dsb * qd[i, hh]
                dkv_ref[j, :dv] += pb * dd[i, hh]
    assert n_changed > 50                      # the casts are not no-ops on this input
    # fp32 evaluation of exp / products may flip a bf16 rounding of P or dS by one ulp (2^-8
    # relative) now and then; sums of a handful of such terms stay within a few 1e-3 of the loops
    torch.testing.assert_close(dq.double(), dq_ref, rtol=0, atol=4e-3 * dq_ref.abs().max().item())
    torch.testing.assert_close(dkv.double(), dkv_ref, rtol=0, atol=4e-3 * dkv_ref.abs().max().item())
    # and the rounding is visible: the fp32 closed form differs from the rounded one
    dq32, dkv32 = O.sparse_mla_bwd_kernel_rounding(q, kv, idx, dout, 0, sm, dv, out=out, lse=lse, round_p_ds_bf16=False)
    assert (dkv32 - dkv).abs().max() > 1e-4
    # median agreement with the loops is at fp32 level (the casts land on the same bf16 values)
    assert (dkv.double() - dkv_ref).abs().median().item() <= 1e-5 * dkv_ref.abs().max().item()


def test_bwd_gradcheck_fp64():
    sq, h, dqk, dv, K = 6, 2, 8, 4, 3
    q, kv, idx = _inputs(sq, h, K, dqk, seed=19)
    f = lambda a, b: O.sparse_mla_fwd(a, b, idx, 0, 0.5, dv, dtype=torch.float64)[0]
    assert torch.autograd.gradcheck(f, (q.requires_grad_(True), kv.requires_grad_(True)), eps=1e-6, atol=1e-6)


def test_attn_dist_rows_sum_to_one_and_matches_loop():
    g = torch.Generator().manual_seed(23)
    p_out = torch.randn(5, 3, 8, generator=g) * 4
    p_out[2, :, 5:] = float("-inf")
    t = O.attn_dist(p_out, 0.25)
    torch.testing.assert_close(t.sum(-1), torch.ones(5), rtol=1e-6, atol=1e-6)
    assert (t[2, 5:] == 0).all()
    for i in range(5):
        acc = np.zeros(8)
        for hh in range(3):
            z = p_out[i, hh].double().numpy() * 0.25
            e = np.exp(z - z[np.isfinite(z)].max())
            acc += e / e.sum()
        np.testing.assert_allclose(t[i].numpy(), acc / 3, rtol=1e-5, atol=1e-7)


def test_attn_dist_from_lse_equals_attn_dist_on_the_logits():
    sq, h, dqk, dv, K = 30, 6, 16, 8, 8
    q, kv, idx = _inputs(sq, h, K, dqk, seed=53, q_start=2, skv=40)
    idx = idx.clone()
    idx[4, 2] = -1
    sm = 0.31
    _, lse, p_out = O.sparse_mla_fwd(q, kv, idx, 2, sm, dv, dtype=torch.float64)
    a = O.attn_dist(p_out, sm).double()
    b = O.attn_dist_from_lse(q, kv, idx, lse, 2, sm, dtype=torch.float64)
    torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-8)          # attn_dist itself evaluates in fp32
    torch.testing.assert_close(b.sum(-1), torch.ones(sq, dtype=torch.float64), rtol=1e-9, atol=1e-9)
    # leading heads only: the same as slicing the logits
    a4 = O.attn_dist(p_out[:, :4], sm).double()
    b4 = O.attn_dist_from_lse(q, kv, idx, lse, 2, sm, heads=4, dtype=torch.float64)
    torch.testing.assert_close(a4, b4, rtol=1e-6, atol=1e-8)


def test_kl_loss_matches_library_and_special_cases():
    g = torch.Generator().manual_seed(29)
    sc = torch.randn(7, 16, generator=g)
    tgt = torch.softmax(torch.randn(7, 16, generator=g), -1)
    got = O.indexer_kl_loss(sc, tgt, 0.7, 7)
    ref = 0.7 * F.kl_div((torch.softmax(sc, -1) + 1e-10).log(), tgt + 1e-10, reduction="sum") / 7
    torch.testing.assert_close(got, ref, rtol=1e-6, atol=1e-8)
    # identical distributions -> 0 loss and 0 gradient
    s2 = sc.clone().requires_grad_(True)
    same = O.indexer_kl_loss(s2, torch.softmax(sc, -1), 1.0, 7)
    same.backward()
    assert abs(same.item()) < 1e-6 and s2.grad.abs().max() < 1e-6
    # uniform prediction vs one-hot target over n slots: KL = log n (up to the 1e-10 guards)
    n = 16
    onehot = torch.zeros(1, n)
    onehot[0, 3] = 1.0
    val = O.indexer_kl_loss(torch.zeros(1, n), onehot, 1.0, 1)
    assert math.isclose(val.item(), math.log(n), rel_tol=1e-5)


def test_kl_gradient_closed_form():
    g = torch.Generator().manual_seed(31)
    sc = torch.randn(4, 8, generator=g, dtype=torch.float64).requires_grad_(True)
    tgt = torch.softmax(torch.randn(4, 8, generator=g, dtype=torch.float64), -1)
    O.indexer_kl_loss(sc, tgt, 2.0, 4).backward()
    pi = torch.softmax(sc.detach(), -1)
    # d/ds of -sum tau*log(pi+eps)  ~=  pi*sum(tau) - tau   as eps -> 0
    approx = 2.0 / 4 * (pi * (tgt + 1e-10).sum(-1, keepdim=True) - tgt)
    torch.testing.assert_close(sc.grad.float(), approx.float(), rtol=1e-5, atol=1e-7)


def test_random_index_generator_is_causal_unique_and_padded():
    idx = O.causal_random_topk_indices(50, 16, seed=1, q_start=3)
    for i in range(50):
        row = idx[i]
        n = min(16, i + 4)
        sel = row[row >= 0]
        assert len(sel) == n and len(set(sel.tolist())) == n and sel.max() <= i + 3
    cu = O.make_packed_cu_seqlens(100, 4, 10, seed=7)
    assert cu[0] == 0 and cu[-1] == 100 and (torch.diff(cu) >= 10).all()
    idx = O.causal_random_topk_indices(100, 8, seed=2, cu_seqlens=cu)
    ks, ke = O.indexer_window(100, 0, cu)
    v = idx >= 0
    assert ((idx >= ks[:, None]) | ~v).all() and ((idx < ke[:, None]) | ~v).all()
    assert torch.equal(v.sum(-1), torch.minimum(ke - ks, torch.tensor(8)))
