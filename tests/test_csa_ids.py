"""Host logic of the compressed-sparse-attention callers: the id helpers against the loop oracle and
against an independent statement of the rule they encode (runs on the CPU)."""
import pytest
import torch

from oracle import csa_oracle as C
from loongforge_amd import csa_kernels as P


def _visible_sets(window, ratio, seg_len):
    """What a query at position p of a segment of seg_len tokens may see, stated directly: raw
    positions in (p - window, p], and compressed key c once its last raw position is <= p."""
    n_c = seg_len // ratio
    raw = [set(range(max(0, p - window + 1), p + 1)) for p in range(seg_len)]
    comp = [set(c for c in range(n_c) if c * ratio + ratio - 1 <= p) for p in range(seg_len)]
    return raw, comp


@pytest.mark.parametrize("window,seqlen", [(1, 5), (4, 11), (16, 9), (8, 64)])
def test_window_ids(window, seqlen):
    got = P.get_window_topk_idxs(window, 2, seqlen, "cpu")
    assert got.shape == (2, seqlen, window) and got.dtype == torch.int64
    assert torch.equal(got[0], C.window_ids(window, seqlen)) and torch.equal(got[1], got[0])
    raw, _ = _visible_sets(window, 1, seqlen)
    for i in range(seqlen):
        row = got[0, i].tolist()
        live = [v for v in row if v >= 0]
        assert set(live) == raw[i] and live == sorted(live) and row[:len(live)] == live   # ascending, left-aligned


@pytest.mark.parametrize("ratio,seqlen,offset", [(4, 19, 19), (1, 6, 0), (128, 300, 7), (3, 2, 5)])
def test_compress_ids(ratio, seqlen, offset):
    got = P.get_compress_topk_idxs(ratio, 1, seqlen, offset, "cpu")[0]
    assert got.shape == (seqlen, seqlen // ratio)
    assert torch.equal(got, C.compress_ids(ratio, seqlen, offset))
    _, comp = _visible_sets(1, ratio, seqlen)
    for i in range(seqlen):
        assert set(v - offset for v in got[i].tolist() if v >= 0) == comp[i]


def test_packed_ids_equal_the_per_segment_forms():
    ratio, window = 4, 6
    lens = [13, 0, 3, 22]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    cu_c = torch.tensor([0] + list(torch.tensor([n // ratio for n in lens]).cumsum(0)), dtype=torch.int32)
    total = int(cu[-1]) + 3                                   # three padding rows after the last segment
    max_c = max(n // ratio for n in lens)
    w = P.get_window_topk_idxs_thd(window, cu, total)
    c = P.get_compress_topk_idxs_thd(ratio, cu, cu, cu_c, total, max_c)
    assert w.dtype == torch.int32 and c.dtype == torch.int32
    assert torch.equal(w, C.window_ids_thd(window, cu, total))
    assert torch.equal(c, C.compress_ids_thd(ratio, cu, cu, cu_c, total, max_c))
    assert (w[int(cu[-1]):] == -1).all() and (c[int(cu[-1]):] == -1).all()
    for b, n in enumerate(lens):                              # each segment on its own
        s = int(cu[b])
        assert torch.equal(w[s:s + n].long(), P.get_window_topk_idxs(window, 1, n, "cpu")[0])
        solo = P.get_compress_topk_idxs(ratio, 1, n, n, "cpu")[0]          # offset = the segment's own length
        assert torch.equal(c[s:s + n, :n // ratio].long(), solo)
        assert (c[s:s + n, n // ratio:] == -1).all()
    # sizes read from the tensors when the caller does not pass them
    assert torch.equal(P.get_window_topk_idxs_thd(window, cu), w[:int(cu[-1])])
    assert torch.equal(P.get_compress_topk_idxs_thd(ratio, cu, cu, cu_c), c[:int(cu[-1])])
    none = P.get_compress_topk_idxs_thd(64, cu, cu, torch.zeros(5, dtype=torch.int32), total)
    assert none.shape == (total, 0)


def test_indexer_window_rule():
    ks, ke = C.csa_indexer_window(10, 4, 2, sq_offset=0)
    assert ks.tolist() == [0] * 10 and ke.tolist() == [1, 1, 1, 1, 1, 1, 1, 2, 2, 2]      # never empty, capped at sk
    ks, ke = C.csa_indexer_window(4, 4, 8, sq_offset=9)
    assert ke.tolist() == [2, 2, 3, 3]
    cu_q = torch.tensor([0, 9, 12]); cu_kv = torch.tensor([0, 2, 2])
    ks, ke = C.csa_indexer_window(12, 4, 2, cu_seqlens_q=cu_q, cu_seqlens_kv=cu_kv)
    assert ks.tolist() == [0] * 9 + [2] * 3
    assert (ke - ks).tolist() == [0, 0, 0, 1, 1, 1, 1, 2, 2, 0, 0, 0]                     # empty rows are allowed here
