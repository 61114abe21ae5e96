"""Helpers shared by the GPU parity tests."""
import torch


def assert_close(got, ref, name, atol=2e-2, rtol=1e-2, scale_aware=False):
    """|got - ref| <= atol + rtol * |ref| elementwise (the tolerance the path is specified with:
    max-abs 2e-2, relative 1e-2 against an fp32 reference).  With ``scale_aware`` the absolute term
    grows to 5e-3 * max|ref|: gradients at tiny top-k are sums of a few large terms (peaky softmax
    rows), and the bf16 rounding of the P / dS operands of the MFMA - which the reference's kernels
    share - scales with those terms, not with the element it lands on."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    if scale_aware:
        atol = max(atol, 5e-3 * ref.abs().max().item())
    d = (got - ref).abs()
    lim = atol + rtol * ref.abs()
    worst = (d - lim).max().item()
    assert worst <= 0, "%s: max abs err %.4e (ref max %.3e), exceeds tolerance by %.3e" % (
        name, d.max().item(), ref.abs().max().item(), worst)


def valid_sets_equal_up_to_noise(ids, ref_ids, ref_logits, band):
    """Top-k parity rule: per row the sets of valid ids are equal, except for keys whose oracle
    score lies within ``band`` of the row's k-th score (fp32 accumulation noise of a 64-term signed
    sum; an exact tie is the band = 0 case).  Returns the number of offending rows."""
    bad = 0
    ids, ref_ids = ids.cpu(), ref_ids.cpu()
    for i in range(ids.shape[0]):
        a = set(ids[i][ids[i] >= 0].tolist())
        b = set(ref_ids[i][ref_ids[i] >= 0].tolist())
        if a == b:
            continue
        if len(a) != len(b):
            bad += 1
            continue
        kth = min(ref_logits[i, j].item() for j in b)
        if any(abs(ref_logits[i, j].item() - kth) > band for j in a ^ b):
            bad += 1
    return bad
