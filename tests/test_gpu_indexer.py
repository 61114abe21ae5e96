"""GPU parity: quantiser, indexer logits, top-k (through the C ABI via loongforge_amd.ops)."""
import pytest
import torch

from oracle import dsa_oracle as O
from tests.gpu_util import valid_sets_equal_up_to_noise

pytestmark = pytest.mark.gpu


def _quant_pair(iq, ik, dev):
    from loongforge_amd import ops

    q8, qs = ops.quant_rowwise_e4m3(iq.to(dev))
    k8, ks = ops.quant_rowwise_e4m3(ik.to(dev))
    return q8, qs, k8, ks


def test_quantiser_is_bit_exact(gpu):
    from loongforge_amd import ops

    g = torch.Generator().manual_seed(3)
    x = (torch.randn(2000, 128, generator=g) * torch.logspace(-10, 6, 2000).unsqueeze(-1)).to(torch.bfloat16)
    x[7] = 0
    x[8, 0] = 3.5            # amax exactly on a power-of-two boundary of 448/amax
    x[9, 0] = 3.515625
    x[10, 3] = float(torch.finfo(torch.bfloat16).max)
    r8, rs = O.quant_rowwise_e4m3(x)
    x8, si = ops.quant_rowwise_e4m3(x.to(gpu))
    assert torch.equal(x8.view(torch.uint8).cpu(), r8.view(torch.uint8))
    assert torch.equal(si.cpu(), rs)
    assert si[7].item() == 2.0 ** -48
    # 3-D input (tokens, heads, 128) quantises per (token, head) row
    y = torch.randn(33, 5, 128, generator=g).to(torch.bfloat16)
    y8, ys = ops.quant_rowwise_e4m3(y.to(gpu))
    r8, rs = O.quant_rowwise_e4m3(y)
    assert ys.shape == (33, 5) and torch.equal(y8.view(torch.uint8).cpu(), r8.view(torch.uint8)) and torch.equal(ys.cpu(), rs)
    with pytest.raises(ValueError):
        ops.quant_rowwise_e4m3(torch.zeros(4, 64, dtype=torch.bfloat16, device=gpu))


@pytest.mark.parametrize("S,Hi,K,cu,seed", [
    (200, 64, 64, None, 42),
    (333, 32, 128, None, 5),
    (512, 64, 64, [0, 100, 101, 300, 512], 9),
    (70, 64, 128, None, 11),          # every row has fewer than K visible keys
])
def test_logits_and_topk_against_oracle(gpu, S, Hi, K, cu, seed):
    from loongforge_amd import ops

    cu_t = torch.tensor(cu, dtype=torch.int32) if cu else None
    iq, ik, w = O.make_indexer_inputs(S, Hi, 128, seed=seed)
    sc_ref, idx_ref, aux = O.indexer_forward(iq, ik, w, K, 0, cu_t, dtype=torch.float64)
    q8, qs, k8, ksc = _quant_pair(iq, ik, gpu)
    assert torch.equal(q8.view(torch.uint8).cpu(), aux["q8"].view(torch.uint8))
    ws = (w.to(gpu) * qs * 128 ** -0.5).contiguous()
    ks, ke = aux["ks"].to(gpu), aux["ke"].to(gpu)

    logits = ops.indexer_logits(q8, ws, k8, ksc, ks, ke)
    L, R = logits.cpu(), aux["logits"]
    fin = torch.isfinite(R)
    assert torch.equal(torch.isfinite(L), fin)                      # -inf exactly outside [ks, ke)
    # 64 signed terms of magnitude ~|w'| * |q.k| cancel; fp32 noise is relative to the term size
    noise = 1e-4 * R[fin].abs().max().item()
    assert (L[fin].double() - R[fin]).abs().max().item() <= noise

    for srt in (True, False):
        sc, ids = ops.topk(logits, K, ks, ke, None, sorted=srt)
        v2, _ = O.topk_select(L, K)                                  # library routine on the same logits
        scc, idc = sc.cpu(), ids.cpu()
        if srt:
            assert torch.equal(scc, v2)
        else:
            assert torch.equal(torch.sort(scc, descending=True).values, v2)
            big = torch.where(idc >= 0, idc, torch.full_like(idc, 1 << 30)).long()
            assert (torch.diff(big, dim=1) >= 0).all()             # ascending column order
        got = torch.where(idc >= 0, L.gather(1, idc.clamp(min=0).long()), torch.full_like(scc, float("-inf")))
        assert torch.equal(got, scc)                                # slot t of scores and ids stay aligned
        for i in range(S):
            a = idc[i][idc[i] >= 0]
            assert a.numel() == len(set(a.tolist())) == min(K, int(ke[i] - ks[i]))
            assert (a >= int(ks[i])).all() and (a < int(ke[i])).all()

    sc, ids = ops.indexer_topk(q8, ws, k8, ksc, ks, ke, K)
    assert valid_sets_equal_up_to_noise(ids, idx_ref, R, band=2 * noise) == 0


def test_topk_is_bit_exact_when_the_arithmetic_is_exact(gpu):
    """Small-integer payloads, unit scales and power-of-two weights make every product and sum
    exact in fp32, so the selected sets must equal the oracle's with no tolerance band (scores are
    made distinct so that there are no ties at the boundary)."""
    from loongforge_amd import ops

    g = torch.Generator().manual_seed(0)
    S, Hi, K = 300, 32, 64
    q = torch.randint(-3, 4, (S, Hi, 128), generator=g).float()
    k = torch.randint(-3, 4, (S, 128), generator=g).float()
    w = torch.full((S, Hi), 2.0 ** -4)
    k[:, 0] = 0
    q8, k8 = q.to(torch.float8_e4m3fn), k.to(torch.float8_e4m3fn)
    ksc = torch.ones(S) + torch.arange(S) * 2.0 ** -12              # distinct, exactly representable scales
    ks, ke = O.indexer_window(S, 0)
    R = O.indexer_logits(q8, w, k8, ksc, ks, ke, dtype=torch.float64)
    L = ops.indexer_logits(q8.to(gpu), w.to(gpu), k8.to(gpu), ksc.to(gpu), ks.to(gpu), ke.to(gpu)).cpu()
    fin = torch.isfinite(R)
    assert torch.equal(L[fin].double(), R[fin])
    sc, ids = ops.indexer_topk(q8.to(gpu), w.to(gpu), k8.to(gpu), ksc.to(gpu), ks.to(gpu), ke.to(gpu), K)
    vref, iref = O.topk_select(R.float(), K)
    assert torch.equal(sc.cpu(), vref)
    for i in range(S):
        row = vref[i][vref[i] > float("-inf")]
        if row.numel() == K and (R[i, : i + 1] == row.min().item()).sum() > 1:
            continue                                                # an exact tie at the K-th value
        assert set(ids[i][ids[i] >= 0].tolist()) == set(iref[i][iref[i] >= 0].tolist())


def test_padded_flashinfer_topk_wrapper(gpu):
    from loongforge_amd.dsa_fused_kernels import padded_flashinfer_topk

    g = torch.Generator().manual_seed(1)
    logits = torch.randn(10, 20, generator=g)
    vals, idx = padded_flashinfer_topk(logits.to(gpu), 5, 20)
    rv, ri = torch.topk(logits, 5)
    assert torch.equal(vals.cpu(), rv) and torch.equal(idx.cpu().long(), ri)
    vals, idx = padded_flashinfer_topk(logits.to(gpu), 25, 20)
    assert vals.shape == (10, 25) and torch.isinf(vals[:, 20:]).all() and (idx[:, 20:] == 20).all()
    assert torch.equal(vals[:, :20].cpu(), torch.sort(logits, descending=True).values)


def test_relative_layout_of_packed_logits(gpu):
    from loongforge_amd import ops

    cu = torch.tensor([0, 40, 41, 128], dtype=torch.int32)
    iq, ik, w = O.make_indexer_inputs(128, 64, 128, seed=3)
    _, _, aux = O.indexer_forward(iq, ik, w, 16, 0, cu)
    q8, qs, k8, ksc = _quant_pair(iq, ik, gpu)
    ws = (w.to(gpu) * qs * 128 ** -0.5).contiguous()
    ks, ke = aux["ks"].to(gpu), aux["ke"].to(gpu)
    dense = ops.indexer_logits(q8, ws, k8, ksc, ks, ke).cpu()
    rel = ops.indexer_logits(q8, ws, k8, ksc, ks, ke, width=87, relative=True).cpu()
    for i in range(128):
        n = int(ke[i] - ks[i])
        assert torch.equal(rel[i, :n], dense[i, int(ks[i]): int(ke[i])])
        assert torch.isinf(rel[i, n:]).all()


@pytest.mark.parametrize("kind", ["normal", "ties", "constant", "outlier", "holes", "short", "two_values", "plus_inf"])
@pytest.mark.parametrize("K,sorted_out", [(2048, True), (1000, True), (256, True), (512, False)])
def test_topk_rule_on_crafted_rows(gpu, kind, K, sorted_out):
    """The selection rule on rows that exercise every branch of the kernel: the K largest values, ties
    broken towards the smaller column, output in descending score / ascending column order.  The
    expectation is a stable sort by the library routine."""
    from loongforge_amd import ops

    n, rows = 6001, 12                                    # odd width: row starts at every 4-byte alignment
    g = torch.Generator().manual_seed(5)
    x = torch.randn(rows, n, generator=g)
    if kind == "ties":
        x = torch.round(x * 8) / 8                        # a few dozen distinct values
    elif kind == "constant":
        x = torch.full((rows, n), 1.25)
    elif kind == "outlier":
        x[:, 17] = 1e30                                   # every other value lands in the last value bins
        x[:, 99] = -1e30
    elif kind == "holes":
        x[torch.rand(rows, n, generator=g) < 0.3] = float("-inf")
    elif kind == "two_values":
        x = (x > 0.5).float()
    elif kind == "plus_inf":
        x[:, 5] = float("inf")                            # +inf is the largest value, as for torch.topk
        x[::2, 4000] = float("inf")
    end = torch.full((rows,), n, dtype=torch.int32)
    if kind == "short":
        end = torch.tensor([1, 2, 63, 64, 255, 256, 257, 999, 1000, 1001, 2047, 2049], dtype=torch.int32)
    beg = torch.zeros(rows, dtype=torch.int32) if kind == "short" else (torch.arange(rows, dtype=torch.int32) % 5)
    sc, ids = ops.topk(x.to(gpu), K, beg.to(gpu), end.to(gpu), sorted=sorted_out)
    sc, ids = sc.cpu(), ids.cpu()
    for i in range(rows):
        row = x[i, : int(end[i])].clone()
        row[: int(beg[i])] = float("-inf")                  # columns before the window cannot be selected
        order = torch.sort(-row, stable=True).indices      # descending value, ascending column among equals
        fin = row[order] > float("-inf")                    # only -inf marks a column that cannot be selected
        exp_ids = order[fin][:K]
        kk = len(exp_ids)
        if sorted_out:
            assert torch.equal(ids[i, :kk].long(), exp_ids), (kind, K, i)
            assert torch.equal(sc[i, :kk], row[exp_ids])
        else:
            got = ids[i][ids[i] >= 0].long()
            assert torch.equal(torch.sort(got).values, torch.sort(exp_ids).values), (kind, K, i)
            assert torch.equal(sc[i][ids[i] >= 0], row[got])
        assert (ids[i, kk:] == -1).all() and torch.isinf(sc[i, kk:]).all() and (sc[i, kk:] < 0).all()


def test_topk_on_full_width_rows_at_every_alignment(gpu):
    """Rows of the widest size the register-resident path takes (8192), starting 0..3 elements past a
    16-byte boundary."""
    from loongforge_amd import ops

    g = torch.Generator().manual_seed(11)
    buf = torch.randn(4 * 8192 + 3, generator=g).to(gpu)
    for off in range(4):
        x = buf[off: off + 4 * 8192].view(4, 8192)
        assert x.data_ptr() % 16 == 4 * off
        sc, ids = ops.topk(x, 2048)
        ref = torch.sort(-x.cpu(), stable=True, dim=-1).indices[:, :2048]
        assert torch.equal(ids.cpu().long(), ref)
        assert torch.equal(sc.cpu(), torch.gather(x.cpu(), 1, ref))


def test_fused_rotation_and_quantiser(gpu):
    """rotate_quant_e4m3 against the unfused sequence rotate_activation -> quantiser: the rotated bf16
    values agree to one bf16 step (the fp32 sums are taken in a different order), payload and scale
    are exactly the quantisation of the kernel's own rotated values, and the rotation is an involution."""
    from loongforge_amd import ops
    from loongforge_amd.dsa_fused import rotate_activation

    g = torch.Generator().manual_seed(3)
    x = torch.randn(1000, 7, 128, generator=g).to(torch.bfloat16)
    x[5] = 0
    xd = x.to(gpu)
    x8, sinv, y = ops.rotate_quant_e4m3(xd, return_rotated=True)
    ref = rotate_activation(x)                                       # fp32 product with the Hadamard matrix on the CPU
    err = (y.cpu().float() - ref.float()).abs()
    assert (err <= 2.0 ** -7 * ref.float().abs() + 1e-30).all()      # at most one bf16 step
    assert (err == 0).float().mean().item() > 0.98
    r8, rs = O.quant_rowwise_e4m3(y.cpu())
    assert torch.equal(x8.cpu().view(torch.uint8), r8.view(torch.uint8)) and torch.equal(sinv.cpu(), rs)
    x8b, sinvb = ops.rotate_quant_e4m3(xd)
    assert torch.equal(x8b.view(torch.uint8), x8.view(torch.uint8)) and torch.equal(sinvb, sinv)
    assert torch.equal(ops.rotate_bf16(xd), y)
    back = ops.rotate_bf16(y).float().cpu()                          # H.H = 128 I: rotating twice returns x
    assert (back - x.float()).abs().max().item() <= 2.0 ** -6 * x.float().abs().max().item()


def test_quantiser_with_weight_scaling_equals_the_separate_operations(gpu):
    """The quantiser kernel that also emits weights * scale_inv * factor: payload and scales are those
    of the plain kernel, the scaled weights are bit-equal to the two torch multiplications."""
    from loongforge_amd import ops

    iq, _, w = O.make_indexer_inputs(300, 64, 128, seed=3)
    x, wd = iq.to(gpu), w.to(gpu)
    for rotate in (False, True):
        plain = ops.rotate_quant_e4m3(x) if rotate else ops.quant_rowwise_e4m3(x)
        x8, si, ws = ops.quant_rowwise_e4m3_weights(x, wd, 128 ** -0.5, rotate)
        assert torch.equal(x8.view(torch.uint8), plain[0].view(torch.uint8)) and torch.equal(si, plain[1])
        assert torch.equal(ws, wd * si * 128 ** -0.5)
    with pytest.raises(ValueError):
        ops.quant_rowwise_e4m3_weights(x, wd[:, :32], 1.0)


def test_indexer_kernel_with_fused_rotation_matches_rotating_first(gpu):
    """DSAIndexerKernel(rotate=True) == DSAIndexerKernel on pre-rotated inputs: same scores and ids, and
    gradients that agree with autograd through rotate_activation."""
    from loongforge_amd.dsa_fused import rotate_activation
    from loongforge_amd.dsa_fused_kernels import DSAIndexerKernel

    S, Hi, K = 512, 64, 128
    iq, ik, w = O.make_indexer_inputs(S, Hi, 128, seed=11)
    kern = DSAIndexerKernel()
    q1, k1, w1 = (t.to(gpu).requires_grad_(True) for t in (iq, ik, w))
    sc1, id1 = kern(q1, k1, w1, K, 0, None, rotate=True)
    q2, k2, w2 = (t.to(gpu).requires_grad_(True) for t in (iq, ik, w))
    sc2, id2 = kern(rotate_activation(q2), rotate_activation(k2), w2, K, 0, None)
    fin = torch.isfinite(sc2)
    assert torch.equal(torch.isfinite(sc1), fin)
    # a bf16 step in a few rotated values moves a logit by a few 1e-3 of the row's scale
    tol = 5e-3 * sc2[fin].abs().max().item()
    assert (sc1[fin] - sc2[fin]).abs().max().item() <= tol
    same = (torch.sort(id1, 1).values == torch.sort(id2, 1).values).float().mean().item()
    assert same > 0.99
    gsc = torch.randn(S, K, generator=torch.Generator().manual_seed(12)).to(gpu)
    torch.where(fin, sc1, torch.zeros_like(sc1)).mul(gsc).sum().backward()
    torch.where(fin, sc2, torch.zeros_like(sc2)).mul(gsc).sum().backward()
    for a, b in ((q1.grad, q2.grad), (k1.grad, k2.grad), (w1.grad, w2.grad)):
        scale = b.float().abs().max().item()
        assert (a.float() - b.float()).abs().max().item() <= 3e-2 * scale
