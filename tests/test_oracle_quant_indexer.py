"""Pins for the oracle's quantiser, indexer logits and top-k (independent of the oracle's code)."""
import math

import numpy as np
import pytest
import torch

from oracle import dsa_oracle as O


# ---- quantiser -------------------------------------------------------------------------
def test_quant_known_answers_from_reference_docstring():
    # deepseek_v4_csa.py:1528-1534: zero rows sit at scale_inv = 2^-48, "real" rows ~1.56e-2 = 2^-6
    x = torch.zeros(3, 128, dtype=torch.bfloat16)
    x[1, 5] = 3.75      # amax in (3.5, 7]  -> scale 2^6
    x[2, 7] = -7.0      # amax == 7 exactly -> 448/7 = 64 = 2^6
    x8, si = O.quant_rowwise_e4m3(x)
    assert si[0].item() == 2.0 ** -48
    assert si[1].item() == 2.0 ** -6
    assert si[2].item() == 2.0 ** -6
    assert x8[0].float().abs().max() == 0
    assert x8[1, 5].float().item() == 240.0          # 3.75 * 64, exactly representable
    assert x8[2, 7].float().item() == -448.0


def test_quant_scale_is_floor_pow2_and_payload_is_rne():
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(64, 128, generator=g) * torch.logspace(-6, 4, 64).unsqueeze(-1)).to(torch.bfloat16)
    x8, si = O.quant_rowwise_e4m3(x)
    amax = x.float().abs().amax(-1).double()
    scale = 1.0 / si.double()
    # power of two, and the largest one with amax*scale <= 448
    m, e = np.frexp(scale.numpy())
    assert np.all(m == 0.5)
    assert torch.all(amax * scale <= 448.0)
    assert torch.all(amax * scale * 2 > 448.0)
    # payload: nearest e4m3 value (brute force over the 256-entry code book), ties to even mantissa
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    finite = codes[~torch.isnan(codes)]
    y = (x.float() * scale.float().unsqueeze(-1))
    got = x8.float()
    dist = (y.unsqueeze(-1) - finite).abs()
    best = dist.min(-1).values
    assert torch.equal((y - got).abs(), best)
    assert got.abs().max() <= 448.0
    # |x8 * scale_inv - x| <= 2^-4 |x| for values in the normal range of the scaled payload
    rel = ((got * si.unsqueeze(-1)) - x.float()).abs() / x.float().abs().clamp_min(1e-30)
    normal = y.abs() >= 2.0 ** -6
    assert rel[normal].max() <= 2.0 ** -4


def test_quant_row_exactly_at_power_of_two_boundary():
    x = torch.zeros(2, 128, dtype=torch.bfloat16)
    x[0, 0] = 3.5        # 448/3.5 = 128 exactly -> scale 2^7, payload 448
    x[1, 0] = 3.515625   # next bf16 above 3.5 -> scale 2^6
    x8, si = O.quant_rowwise_e4m3(x)
    assert si[0].item() == 2.0 ** -7 and x8[0, 0].float().item() == 448.0
    assert si[1].item() == 2.0 ** -6 and x8[1, 0].float().item() == 224.0  # 3.515625*64 = 225 -> RNE 224


# ---- indexer logits ----------------------------------------------------------------------
def _brute_logits(q8, w, k8, ksc, ks, ke):
    sq, h, d = q8.shape
    sk = k8.shape[0]
    out = np.full((sq, sk), -np.inf)
    qn, kn = q8.double().numpy(), k8.double().numpy()
    for i in range(sq):
        for j in range(int(ks[i]), min(int(ke[i]), sk)):
            acc = 0.0
            for hh in range(h):
                dot = float(np.dot(qn[i, hh], kn[j]))
                acc += float(w[i, hh]) * max(dot, 0.0)
            out[i, j] = acc * float(ksc[j])
    return out


def test_indexer_logits_brute_force():
    g = torch.Generator().manual_seed(0)
    sq, h, d = 12, 3, 16
    iq = torch.randn(sq, h, d, generator=g).to(torch.bfloat16)
    ik = torch.randn(sq, d, generator=g).to(torch.bfloat16)
    w = torch.randn(sq, h, generator=g)
    q8, qs = O.quant_rowwise_e4m3(iq)
    k8, ksc = O.quant_rowwise_e4m3(ik)
    ks, ke = O.indexer_window(sq, 0)
    ws = w * qs * d ** -0.5
    got = O.indexer_logits(q8, ws, k8, ksc, ks, ke, dtype=torch.float64).numpy()
    ref = _brute_logits(q8, ws.double().numpy(), k8, ksc.double().numpy(), ks, ke)
    assert np.array_equal(np.isinf(got), np.isinf(ref))
    m = ~np.isinf(ref)
    np.testing.assert_allclose(got[m], ref[m], rtol=1e-12, atol=1e-12)
    # strictly causal window: j > i masked
    assert np.all(np.isinf(got[np.triu_indices(sq, 1)]))


def test_indexer_logits_integer_special_case_is_exact_relu_matmul():
    g = torch.Generator().manual_seed(1)
    sq, d = 9, 32
    q = torch.randint(-4, 5, (sq, 1, d), generator=g).float()
    k = torch.randint(-4, 5, (sq, d), generator=g).float()
    ks = torch.zeros(sq, dtype=torch.int32)
    ke = torch.full((sq,), sq, dtype=torch.int32)
    got = O.indexer_logits(q.to(torch.float8_e4m3fn), torch.ones(sq, 1), k.to(torch.float8_e4m3fn),
                           torch.ones(sq), ks, ke)
    assert torch.equal(got, torch.relu(q[:, 0] @ k.T))


def test_indexer_logits_linear_in_weights_and_kscale():
    g = torch.Generator().manual_seed(2)
    sq, h, d = 8, 4, 16
    q8 = torch.randn(sq, h, d, generator=g).to(torch.float8_e4m3fn)
    k8 = torch.randn(sq, d, generator=g).to(torch.float8_e4m3fn)
    w1, w2 = torch.randn(sq, h, generator=g).double(), torch.randn(sq, h, generator=g).double()
    ksc = torch.rand(sq, generator=g).double()
    ks = torch.zeros(sq, dtype=torch.int32)
    ke = torch.full((sq,), sq, dtype=torch.int32)
    f = lambda w, s: O.indexer_logits(q8, w, k8, s, ks, ke, dtype=torch.float64)
    torch.testing.assert_close(f(w1 + 2 * w2, ksc), f(w1, ksc) + 2 * f(w2, ksc), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(f(w1, 3 * ksc), 3 * f(w1, ksc), rtol=1e-12, atol=1e-12)


def test_indexer_window_packed_closed_form():
    cu = torch.tensor([0, 3, 4, 9], dtype=torch.int32)
    ks, ke = O.indexer_window(9, 0, cu)
    assert ks.tolist() == [0, 0, 0, 3, 4, 4, 4, 4, 4]
    assert ke.tolist() == list(range(1, 10))
    ks2, ke2 = O.indexer_window(4, 5, cu)      # local chunk starting at global token 5
    assert ks2.tolist() == [4, 4, 4, 4] and ke2.tolist() == [6, 7, 8, 9]


# ---- top-k -------------------------------------------------------------------------------
def test_topk_matches_sort_and_invariants():
    g = torch.Generator().manual_seed(4)
    sq, K = 40, 8
    logits = torch.randn(sq, sq, generator=g)
    causal = torch.arange(sq)[None, :] > torch.arange(sq)[:, None]
    logits = logits.masked_fill(causal, float("-inf"))
    vals, idx = O.topk_select(logits, K)
    for i in range(sq):
        n = min(K, i + 1)
        order = torch.sort(logits[i, : i + 1], descending=True)
        assert torch.equal(vals[i, :n], order.values[:n])
        assert set(idx[i, :n].tolist()) == set(order.indices[:n].tolist())
        assert idx[i, n:].eq(-1).all() and torch.isinf(vals[i, n:]).all()
        sel = idx[i, :n].long()
        assert len(set(sel.tolist())) == n and sel.max() <= i
        rest = torch.ones(i + 1, dtype=torch.bool)
        rest[sel] = False
        if rest.any():
            assert logits[i, : i + 1][rest].max() <= vals[i, :n].min()


def test_topk_wider_than_row_pads_minus_one():
    logits = torch.tensor([[0.5, -1.0, 2.0]])
    vals, idx = O.topk_select(logits, 5)
    assert idx.tolist() == [[2, 0, 1, -1, -1]]
    assert vals[0, :3].tolist() == [2.0, 0.5, -1.0] and torch.isinf(vals[0, 3:]).all()


def test_indexer_forward_packed_equals_per_document_runs():
    g = torch.Generator().manual_seed(5)
    cu = torch.tensor([0, 20, 33, 64], dtype=torch.int32)
    iq = torch.randn(64, 2, 128, generator=g).to(torch.bfloat16)
    ik = torch.randn(64, 128, generator=g).to(torch.bfloat16)
    w = torch.rand(64, 2, generator=g)
    sc, idx, aux = O.indexer_forward(iq, ik, w, 16, 0, cu)
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        sc1, idx1, aux1 = O.indexer_forward(iq[a:b], ik[a:b], w[a:b], 16, 0, None)
        torch.testing.assert_close(sc[a:b], sc1, rtol=0, atol=0)
        # ids are global rows of the packed key array, inside the query's own document, and
        # point at entries holding exactly the reported score (ReLU makes exact ties common,
        # so the id sets themselves are only defined up to ties)
        sel = idx[a:b]
        valid = sel >= 0
        assert torch.equal(valid, idx1 >= 0)
        assert (sel[valid] >= a).all() and (sel[valid] < b).all()
        got = aux["logits"][a:b].gather(1, sel.clamp(min=0).long())
        assert torch.equal(got[valid], sc[a:b][valid])
        assert torch.equal(aux["logits"][a:b, a:b], aux1["logits"])


def test_indexer_bwd_matches_finite_differences_and_eps_floor():
    g = torch.Generator().manual_seed(6)
    sq, h, d, K = 10, 2, 16, 4
    q8 = torch.randn(sq, h, d, generator=g).to(torch.float8_e4m3fn)
    k8 = torch.randn(sq, d, generator=g).to(torch.float8_e4m3fn)
    k8[3] = 0
    qs = torch.rand(sq, h, generator=g) + 0.5
    ksc = torch.rand(sq, generator=g) + 0.5
    ksc[3] = 2.0 ** -48
    ws = torch.randn(sq, h, generator=g)
    idx = O.causal_random_topk_indices(sq, K, 0)
    gsc = torch.randn(sq, K, generator=g)
    dq, dk, dw = O.indexer_bwd(gsc, q8, k8, qs, ksc, ws, idx, dtype=torch.float64)
    assert dk[3].abs().max() == 0          # eps-floor row -> exactly zero
    # finite differences on the weights (the function is linear in them => exact up to rounding)
    base = O.gathered_indexer_logits(q8, ws.double(), k8, ksc, idx, dtype=torch.float64)
    valid = idx >= 0
    for (i, hh) in [(0, 0), (5, 1), (9, 0)]:
        w2 = ws.double().clone()
        w2[i, hh] += 1.0
        pert = O.gathered_indexer_logits(q8, w2, k8, ksc, idx, dtype=torch.float64)
        fd = ((pert - base).masked_fill(~valid, 0) * gsc.double()).sum()
        expect = fd * qs[i, hh].double() * d ** -0.5
        assert math.isclose(dw[i, hh].item(), expect.item(), rel_tol=1e-9, abs_tol=1e-12)
    # d_q: brute force for one (i, h): sum_t g * kscale[j] * w' * [r>0] * k8[j] / q_scale
    i, hh = 7, 1
    acc = torch.zeros(d, dtype=torch.float64)
    for t in range(K):
        j = int(idx[i, t])
        if j < 0:
            continue
        r = (q8[i, hh].double() * k8[j].double()).sum()
        if r > 0:
            acc += gsc[i, t].double() * ksc[j].double() * ws[i, hh].double() * k8[j].double()
    torch.testing.assert_close(dq[i, hh], acc / qs[i, hh].double(), rtol=1e-9, atol=1e-12)
