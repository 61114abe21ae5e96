"""Pins of oracle/front_oracle.py against library routines and closed forms (CPU)."""
import torch

from oracle import dsa_oracle as O
from oracle import front_oracle as F
from oracle import rope_oracle as R


def _rows(n, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, 128, generator=g) * scale).to(torch.bfloat16)


def test_layer_norm_rows_is_layer_norm():
    g = torch.Generator().manual_seed(1)
    x = _rows(300, 0, 3.0) + 1.5
    w, b = torch.randn(128, generator=g), torch.randn(128, generator=g)
    y = F.layer_norm_rows(x, w, b, 1e-5)
    ref = torch.nn.functional.layer_norm(x.double(), (128,), w.double(), b.double(), 1e-5)
    # one bf16 rounding of a value computed to fp32 accuracy
    assert y.dtype == torch.bfloat16
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5).all()
    assert (y.double() == ref.to(torch.bfloat16).double()).float().mean() > 0.995
    # a constant row has no variance: the output is the bias, whatever the weight
    const = torch.full((4, 128), 2.5).to(torch.bfloat16)
    assert torch.equal(F.layer_norm_rows(const, w, b, 1e-5), b.to(torch.bfloat16).expand(4, 128))
    # a dropped mean, a variance without the eps, or an unbiased variance would all fail this closed form
    x2 = torch.zeros(1, 128); x2[0, 0] = 128.0
    y2 = F.layer_norm_rows(x2.to(torch.bfloat16), torch.ones(128), torch.zeros(128), 0.0).float()
    var = (127.0 ** 2 + 127.0) / 128.0
    assert abs(y2[0, 0].item() - 127.0 / var ** 0.5) < 0.05 and abs(y2[0, 1].item() + 1.0 / var ** 0.5) < 1e-3


def test_hadamard_rows_is_the_scaled_sylvester_matrix():
    h = torch.ones(1, 1, dtype=torch.float64)
    while h.shape[0] < 128:
        h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
    x = _rows(500, 2)
    y = F.hadamard_rows(x)
    ref = (x.double() @ h) * 128 ** -0.5
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-30).all()          # one rounding to bf16
    e0 = torch.zeros(1, 128); e0[0, 5] = 1.0                                         # a unit vector gives a matrix row
    assert torch.equal(F.hadamard_rows(e0.to(torch.bfloat16)).double(), (h[5:6] * 128 ** -0.5).to(torch.bfloat16).double())
    back = F.hadamard_rows(y).float()                                               # H.H = 128 I
    assert (back - x.float()).abs().max() <= 2.0 ** -6 * x.float().abs().max()


def test_indexer_front_is_the_sequence_of_library_routines():
    g = torch.Generator().manual_seed(3)
    T, Hh = 40, 3
    x = (torch.randn(T, Hh, 128, generator=g) * 2).to(torch.bfloat16)
    w, b = torch.randn(128, generator=g), torch.randn(128, generator=g)
    cos, sin = R.rope_tables(64, 64, dtype=torch.bfloat16)
    pos = torch.randint(0, 64, (T,), generator=g)
    hw = torch.randn(T, Hh, generator=g)
    for pairing in (R.ADJACENT, R.SPLIT):
        x8, si, rows, ws = F.indexer_front(x, Hh, w, b, 1e-6, cos, sin, pairing, pos, 1, True, hw, 0.25)
        # the same pipeline in fp64 with library routines and a bf16 rounding after every stage
        v = torch.nn.functional.layer_norm(x.double(), (128,), w.double(), b.double(), 1e-6).to(torch.bfloat16)
        c, s = cos.reshape(-1, 64)[pos].unsqueeze(1).double(), sin.reshape(-1, 64)[pos].unsqueeze(1).double()
        pe = v[..., :64].double()
        if pairing == R.ADJACENT:
            x1, x2 = pe[..., 0::2], pe[..., 1::2]
            y = torch.stack([x1 * c[..., 0::2] - x2 * s[..., 0::2], x2 * c[..., 1::2] + x1 * s[..., 1::2]], -1).flatten(-2)
        else:
            x1, x2 = pe[..., :32], pe[..., 32:]
            y = torch.cat([x1 * c[..., :32] - x2 * s[..., :32], x2 * c[..., 32:] + x1 * s[..., 32:]], -1)
        v = torch.cat([y.to(torch.bfloat16), v[..., 64:]], -1)
        h = torch.ones(1, 1, dtype=torch.float64)
        while h.shape[0] < 128:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        ref_rows = ((v.double() @ h) * 128 ** -0.5)
        # a bf16 step at an earlier stage moves the rotated values by well under their own bf16 step
        assert ((rows.double() - ref_rows).abs() <= 2.0 ** -7 * ref_rows.abs() + 2.0 ** -9 * ref_rows.abs().amax(-1, keepdim=True)).all()
        r8, rs = O.quant_rowwise_e4m3(rows)
        assert torch.equal(x8.view(torch.uint8), r8.view(torch.uint8)) and torch.equal(si, rs)
        assert torch.equal(ws, hw * si * 0.25)
    # without any stage it is the plain quantiser
    x8, si, rows, ws = F.indexer_front(x, rotate=False)
    r8, rs = O.quant_rowwise_e4m3(x)
    assert torch.equal(rows, x) and torch.equal(x8.view(torch.uint8), r8.view(torch.uint8)) and ws is None
