"""GPU parity of the fused KL indexer loss (softmax + F.kl_div + backward in one kernel) against the
oracle's restatement of dsa_fused.py:931-944 and torch autograd through it."""
import pytest
import torch
import torch.nn.functional as F

from oracle import dsa_oracle as O

pytestmark = pytest.mark.gpu


def _case(S, K, seed, pad_from=None, target_kind="dist"):
    g = torch.Generator().manual_seed(seed)
    sc = torch.randn(S, K, generator=g) * 3.0
    tg = torch.rand(S, K, generator=g)
    if pad_from is not None:                         # rows with fewer than K valid slots: score -inf, target 0 behind them
        for i in range(S):
            n = int(pad_from[i])
            sc[i, n:] = float("-inf")
            tg[i, n:] = 0.0
    if target_kind == "dist":
        tg = tg / tg.sum(-1, keepdim=True)
    elif target_kind == "onehot":
        tg = F.one_hot(torch.randint(0, K if pad_from is None else 1, (S,), generator=g), K).float()
    return sc, tg


@pytest.mark.parametrize("S,K,padded,kind", [(37, 64, False, "dist"), (130, 2048, True, "dist"), (9, 200, True, "dist"),
                                             (5, 4096, False, "onehot"), (3, 8192, True, "dist"), (1, 1, False, "dist")])
def test_kl_loss_and_gradient_match_the_oracle(gpu, S, K, padded, kind):
    from loongforge_amd import ops

    pad = torch.randint(1, K + 1, (S,), generator=torch.Generator().manual_seed(3)) if padded else None
    sc, tg = _case(S, K, seed=S + K, pad_from=pad, target_kind=kind)
    ref_sc = sc.double().requires_grad_(True)
    ref = O.indexer_kl_loss(ref_sc, tg.double(), 1.0, 1)       # coeff 1, norm 1: the plain "sum" reduction
    # the oracle computes in float: redo it in double for the comparison below
    pred = torch.softmax(ref_sc, -1)
    u = tg.double() + 1e-10
    ref64 = (u * (u.log() - (pred + 1e-10).log())).sum()
    ref64.backward()
    got_sc = sc.to(gpu).requires_grad_(True)
    loss = ops.indexer_kl_loss(got_sc, tg.to(gpu))
    (loss * 0.5).backward()                                     # an upstream factor must reach the gradient
    # float arithmetic against double: tolerance 1e-5 relative to the loss / the largest gradient of a row
    assert abs(loss.item() - ref64.item()) <= 1e-5 * max(1.0, abs(ref64.item())), (loss.item(), ref64.item())
    assert abs(ref.item() - ref64.item()) <= 1e-3 * max(1.0, abs(ref64.item()))
    gref = ref_sc.grad * 0.5
    err = (got_sc.grad.double().cpu() - gref).abs().max().item()
    assert err <= 1e-5 * max(1.0, gref.abs().max().item()), err
    if padded:
        assert (got_sc.grad.cpu()[sc == float("-inf")] == 0).all()


def test_kl_loss_equals_f_kl_div_and_vanishes_for_equal_distributions(gpu):
    from loongforge_amd import ops

    sc, tg = _case(64, 512, seed=11)
    want = F.kl_div((torch.softmax(sc, -1) + 1e-10).log(), tg + 1e-10, reduction="sum")
    got = ops.indexer_kl_loss(sc.to(gpu), tg.to(gpu))
    assert abs(got.item() - want.item()) <= 1e-4 * abs(want.item())
    # identical distributions: loss ~ 0 and zero gradient
    s2 = sc.to(gpu).requires_grad_(True)
    same = torch.softmax(sc, -1).to(gpu)
    l2 = ops.indexer_kl_loss(s2, same)
    l2.backward()
    assert abs(l2.item()) < 1e-4 and s2.grad.abs().max().item() < 1e-5
    # a sliced (strided) target, as the attention module hands it over
    wide = torch.cat([tg, torch.zeros(64, 64)], -1).to(gpu)
    got3 = ops.indexer_kl_loss(sc.to(gpu), wide[:, :512])
    assert got3.item() == got.item()
