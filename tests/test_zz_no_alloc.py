"""The entry point that allocates nothing (dsa_indexer_topk_fwd_static) against dsa_indexer_topk_fwd,
through the C ABI: two calls in a row on the library's own scratch array, the second one smaller."""
import pytest
import torch

from oracle import dsa_oracle as O

pytestmark = pytest.mark.gpu


def _both(lib, gpu, S, Hi, K, seed, cu=None):
    from loongforge_amd import ops

    iq, ik, w = O.make_indexer_inputs(S, Hi, 128, seed=seed)
    ks, ke = O.indexer_window(S, 0, cu)
    q8, qs = ops.quant_rowwise_e4m3(iq.to(gpu))
    k8, ksc = ops.quant_rowwise_e4m3(ik.to(gpu))
    ws = (w.to(gpu) * qs * 128 ** -0.5).contiguous()
    ksd, ked = ks.to(gpu), ke.to(gpu)
    nbytes = lib.dsa_indexer_topk_workspace_bytes(S, S, K)
    wsp = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    sc_a = torch.empty(S, K, dtype=torch.float32, device=gpu)
    id_a = torch.empty(S, K, dtype=torch.int32, device=gpu)
    sc_b, id_b = torch.empty_like(sc_a), torch.empty_like(id_a)
    args = (q8.data_ptr(), ws.data_ptr(), k8.data_ptr(), ksc.data_ptr(), ksd.data_ptr(), ked.data_ptr(), S, Hi, S, K, 1)
    rc = lib.dsa_indexer_topk_fwd(*args, sc_a.data_ptr(), id_a.data_ptr(), wsp.data_ptr(), nbytes, None)
    assert rc == 0, lib.dsa_last_error()
    torch.cuda.synchronize()
    # free device memory as the driver sees it (a hipMalloc by the library would show here; torch's own
    # counters only know torch's allocations), and torch's counter for torch's side
    free_before, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_allocated()
    rc = lib.dsa_indexer_topk_fwd_static(*args, sc_b.data_ptr(), id_b.data_ptr(), None)
    assert rc == 0, lib.dsa_last_error()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before and torch.cuda.memory_allocated() == before
    return sc_a, id_a, sc_b, id_b


def test_static_scratch_entry_point_matches_the_workspace_one_twice(gpu):
    from loongforge_amd import _lib

    lib = _lib.load()
    # first call: 3000 queries x 3000 keys, packed documents, top-k 512
    cu = torch.tensor([0, 700, 701, 3000], dtype=torch.int32)
    sc_a, id_a, sc_b, id_b = _both(lib, gpu, 3000, 64, 512, seed=21, cu=cu)
    assert torch.equal(sc_a, sc_b) and torch.equal(id_a, id_b)
    assert (id_b >= 0).any() and torch.isfinite(sc_b[id_b >= 0]).all()
    # second call on the same array, smaller input: nothing of the first call may leak into it
    sc_a, id_a, sc_b, id_b = _both(lib, gpu, 500, 32, 128, seed=22)
    assert torch.equal(sc_a, sc_b) and torch.equal(id_a, id_b)
    valid = id_b >= 0
    pos = torch.arange(500, device=gpu)[:, None]
    assert (valid.sum(-1) == torch.clamp(pos[:, 0] + 1, max=128)).all() and ((id_b <= pos) | ~valid).all()


def test_static_scratch_entry_point_refuses_what_does_not_fit(gpu):
    from loongforge_amd import _lib

    lib = _lib.load()
    z = torch.zeros(16, dtype=torch.uint8, device=gpu)
    rc = lib.dsa_indexer_topk_fwd_static(z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(),
                                         8, 64, 70000, 64, 1, z.data_ptr(), z.data_ptr(), None)
    assert rc == -1 and b"65536" in lib.dsa_last_error()
