"""GPU parity: sparse MLA forward / backward and the attention distribution."""
import pytest
import torch

from oracle import dsa_oracle as O
from tests.gpu_util import assert_close, assert_mla_grads

pytestmark = pytest.mark.gpu


def _run_fwd(inp, dev, q_start=0, p_out=False, p_dtype=torch.bfloat16):
    from loongforge_amd import ops

    return ops.sparse_mla_fwd(inp.q.to(dev), inp.kv.to(dev), inp.idx.to(dev), q_start, inp.sm_scale, 512, p_out, p_dtype)


@pytest.mark.parametrize("S,H,K,q_start,skv,seed", [
    (64, 128, 64, 0, None, 0),
    (300, 128, 128, 17, None, 1),
    (256, 64, 256, 0, None, 2),
    (130, 32, 192, 5, 400, 3),
])
def test_forward_against_oracle(gpu, S, H, K, q_start, skv, seed):
    inp = O.make_mla_inputs(S, H, K, seed=seed, skv=skv, q_start=q_start)
    out, lse, _ = _run_fwd(inp, gpu, q_start)
    ro, rl, _ = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, q_start, inp.sm_scale, 512)
    assert_close(out, ro, "out")
    assert (lse.cpu() - rl).abs().max().item() < 1e-4


@pytest.mark.parametrize("K", [4096, 8192])
def test_top_k_beyond_2048(gpu, K):
    """Wider slot lists: the forward runs them with a three-stage tile ring; the backward and the recomputed attention
    distribution take 2048 / 4096 slots per call and the host walks the list in parts (the gradients are sums over the
    slots once lse and out of the whole list are given)."""
    from loongforge_amd import ops

    skv = K + 1500
    inp = O.make_mla_inputs(48, 64, K, seed=11, skv=skv, q_start=skv - 48)
    out, lse, _ = _run_fwd(inp, gpu, skv - 48)
    ro, rl, _ = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, skv - 48, inp.sm_scale, 512)
    assert_close(out, ro, "out")
    assert (lse.cpu() - rl).abs().max().item() < 1e-4
    q, kv, ids, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
    dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, ids, lse, skv - 48, inp.sm_scale)
    rdq, rdkv = O.sparse_mla_bwd(inp.q, inp.kv, inp.idx, inp.dout, skv - 48, inp.sm_scale, 512)
    assert_close(dq, rdq, "dq")
    assert_close(dkv, rdkv, "dkv")             # 48 queries: few rows per key, the bf16 rows stay inside the bound
    dist = ops.attn_dist_qk(q, kv, ids, lse, skv - 48, inp.sm_scale, 64)
    ref = O.attn_dist_from_lse(inp.q, inp.kv, inp.idx, rl, skv - 48, inp.sm_scale, 64)
    assert (dist.cpu() - ref).abs().max().item() <= 2e-5


def test_forward_p_out_and_attn_dist(gpu):
    from loongforge_amd import ops
    from loongforge_amd.dsa_fused_kernels import triton_attn_dist

    inp = O.make_mla_inputs(200, 128, 128, seed=4)
    _, _, rp = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, 0, inp.sm_scale, 512)
    for dt in (torch.float32, torch.bfloat16):
        _, _, p = _run_fwd(inp, gpu, 0, True, dt)
        assert p.dtype == dt and p.shape == (200, 128, 128)
        fin = torch.isfinite(rp)
        assert torch.equal(torch.isfinite(p.float().cpu()), fin)          # -inf exactly on invalid slots
        tol = 2e-4 if dt == torch.float32 else 0.26                         # bf16 ulp of |logit| < 64
        assert (p.float().cpu()[fin] - rp[fin]).abs().max().item() < tol
        tgt = ops.attn_dist(p, inp.sm_scale)
        ref = O.attn_dist(rp, inp.sm_scale)
        assert (tgt.cpu() - ref).abs().max().item() < (1e-5 if dt == torch.float32 else 6e-3)
        assert (tgt.sum(-1).cpu() - 1).abs().max().item() < 1e-4
        # head-sliced view (what the attention module passes when it padded the heads)
        tgt16 = ops.attn_dist(p[:, :16], inp.sm_scale)
        ref16 = O.attn_dist(rp[:, :16], inp.sm_scale)
        assert (tgt16.cpu() - ref16).abs().max().item() < (1e-5 if dt == torch.float32 else 6e-3)
        assert triton_attn_dist(p, inp.sm_scale).dtype == dt
        # leaving out leading slots changes nothing but the width of p_out
        for skip in (32, 96):
            o_s, l_s, p_s = ops.sparse_mla_fwd(inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), 0, inp.sm_scale, 512, True, dt,
                                               p_out_skip=skip)
            assert p_s.shape == (200, 128, 128 - skip) and torch.equal(p_s, p[:, :, skip:])


def test_forward_invalid_ids_and_empty_rows(gpu):
    inp = O.make_mla_inputs(96, 128, 64, seed=5, skv=120, q_start=10)
    idx = inp.idx.clone()
    idx[5, 0] = -1
    idx[6, 1] = 120            # == s_kv
    idx[7, 2] = 119            # in range but in the future of query 7
    idx[8, :] = -1             # no valid slot at all
    idx[9] = idx[9][torch.randperm(64, generator=torch.Generator().manual_seed(1))]   # padding in the middle
    inp.idx = idx
    out, lse, p = _run_fwd(inp, gpu, 10, True, torch.float32)
    ro, rl, rp = O.sparse_mla_fwd(inp.q, inp.kv, idx, 10, inp.sm_scale, 512)
    assert_close(out, ro, "out")
    assert out[8].abs().max().item() == 0 and torch.isinf(lse[8]).all() and (lse[8] > 0).all()
    m = torch.isfinite(rl)
    assert (lse.cpu()[m] - rl[m]).abs().max().item() < 1e-4
    assert torch.equal(torch.isfinite(p.cpu()), torch.isfinite(rp))


def test_forward_survives_a_late_dominant_key(gpu):
    """A key whose logit exceeds everything before it by far more than 2^64 forces the exact-max
    pass; the result must still match the oracle."""
    inp = O.make_mla_inputs(80, 128, 64, seed=6)
    kv = inp.kv.clone().float()
    kv[70] = inp.q[79, 0].float() * 40.0          # q.k ~ 40 * |q|^2 for query 79, head 0
    inp.kv = kv.to(torch.bfloat16)
    inp.idx[79, 63] = 70                            # visited in the last tile position
    out, lse, _ = _run_fwd(inp, gpu)
    ro, rl, _ = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, 0, inp.sm_scale, 512)
    assert_close(out, ro, "out", atol=4e-2)         # |kv[70]| is ~40x larger than the other rows
    assert (lse.cpu() - rl).abs().max().item() < 2e-2 * rl.abs().max().item() * 1e-2 + 1e-2


def test_forward_slot_permutation_invariance(gpu):
    inp = O.make_mla_inputs(100, 128, 128, seed=7)
    out1, lse1, _ = _run_fwd(inp, gpu)
    perm = torch.randperm(128, generator=torch.Generator().manual_seed(2))
    inp.idx = inp.idx[:, perm].contiguous()
    out2, lse2, _ = _run_fwd(inp, gpu)
    assert (out1.float() - out2.float()).abs().max().item() < 2e-2
    assert (lse1 - lse2).abs().max().item() < 1e-4


@pytest.mark.parametrize("S,H,K,q_start,skv,seed", [
    (64, 128, 64, 0, None, 0),
    (200, 128, 128, 40, 300, 3),
    (160, 64, 64, 0, None, 5),
    (130, 32, 192, 5, 400, 7),           # two of pass A's eight 16-head waves hold real heads
    (90, 96, 320, 0, None, 9),           # six of them; ten tiles per query
])
def test_backward_against_oracle_and_deterministic(gpu, S, H, K, q_start, skv, seed):
    from loongforge_amd import ops

    inp = O.make_mla_inputs(S, H, K, seed=seed, skv=skv, q_start=q_start)
    q, kv, idx, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx, q_start, inp.sm_scale)
    dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, q_start, inp.sm_scale)
    assert_mla_grads(dq, dkv, inp.q, inp.kv, inp.idx, inp.dout, q_start, inp.sm_scale, out=out, lse=lse)
    dq2, dkv2 = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, q_start, inp.sm_scale)
    assert torch.equal(dq, dq2) and torch.equal(dkv, dkv2)          # bit-identical


def test_backward_does_not_depend_on_the_slot_order(gpu):
    """The backward walks each query's ids in ascending key order whatever order they arrive in, so
    permuting the slots (independently per query) and scattering unused slots between the used ones
    gives bit-identical gradients."""
    from loongforge_amd import ops

    S, K = 150, 128
    inp = O.make_mla_inputs(S, 128, 96, seed=9)                       # 96 used slots ...
    idx = torch.cat([inp.idx, torch.full((S, K - 96), -1, dtype=torch.int32)], dim=1)
    g = torch.Generator().manual_seed(3)
    shuffled = torch.stack([idx[i][torch.randperm(K, generator=g)] for i in range(S)])      # ... anywhere among 128
    q, kv, do = inp.q.to(gpu), inp.kv.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx.to(gpu), 0, inp.sm_scale)
    dq1, dkv1 = ops.sparse_mla_bwd(q, kv, out, do, idx.to(gpu), lse, 0, inp.sm_scale)
    dq2, dkv2 = ops.sparse_mla_bwd(q, kv, out, do, shuffled.to(gpu), lse, 0, inp.sm_scale)
    assert torch.equal(dq1, dq2) and torch.equal(dkv1, dkv2)
    assert_mla_grads(dq2, dkv2, inp.q, inp.kv, inp.idx, inp.dout, 0, inp.sm_scale, out=out, lse=lse)


def test_backward_with_more_keys_than_the_key_bitmap_in_lds_holds(gpu):
    """Beyond about 600 000 keys the per-query key bitmap (and with it the key-sorted id list) no longer
    fits LDS and the passes walk the caller's slot order; results must not care.  The oracle runs on the
    selected keys only (compacted), everything else must get a zero gradient."""
    from loongforge_amd import ops

    S, H, K, skv = 64, 128, 64, 620_000
    g = torch.Generator().manual_seed(17)
    q = torch.randn(S, H, 576, generator=g).to(torch.bfloat16)
    dout = torch.randn(S, H, 512, generator=g).to(torch.bfloat16)
    picked = torch.randperm(skv, generator=g)[:1500]                       # the keys any query may select
    kv_small = torch.randn(1500, 576, generator=g).to(torch.bfloat16)
    idx_small = torch.stack([torch.randperm(1500, generator=g)[:K] for _ in range(S)]).to(torch.int32)
    idx_small[3, 10:] = -1
    idx = torch.where(idx_small >= 0, picked[idx_small.clamp(min=0).long()].to(torch.int32), idx_small)
    kv = torch.zeros(skv, 576, dtype=torch.bfloat16)
    kv[picked] = kv_small
    sm = 192 ** -0.5
    qd, kd, dd, ids = q.to(gpu), kv.to(gpu), dout.to(gpu), idx.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(qd, kd, ids, skv, sm)                 # q_start = skv: no causal test
    dq, dkv = ops.sparse_mla_bwd(qd, kd, out, dd, ids, lse, skv, sm)
    ro, _, _ = O.sparse_mla_fwd(q, kv_small, idx_small, 1500, sm, 512)
    assert_close(out, ro, "out")
    assert_mla_grads(dq, dkv, q, kv_small, idx_small, dout, 1500, sm, out=out, lse=lse, dkv_rows=picked)
    rest = torch.ones(skv, dtype=torch.bool)
    rest[picked] = False
    assert (dkv.cpu()[rest] == 0).all()


def test_backward_with_a_repeated_id_returns_nan_not_a_wrong_sum(gpu):
    """The backward keeps one bit and one row per (query, key): a row of ids that names a key twice
    cannot be summed correctly, and the call says so by returning NaN everywhere."""
    from loongforge_amd import ops

    inp = O.make_mla_inputs(96, 128, 64, seed=4)
    idx = inp.idx.clone()
    idx[70, 5] = idx[70, 9]
    q, kv, do = inp.q.to(gpu), inp.kv.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx.to(gpu), 0, inp.sm_scale)
    dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, idx.to(gpu), lse, 0, inp.sm_scale)
    assert torch.isnan(dq.float()).all() and torch.isnan(dkv.float()).all()
    # the same workspace-free call with distinct ids is clean again (the flag is cleared per call)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, inp.idx.to(gpu), 0, inp.sm_scale)
    dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, inp.idx.to(gpu), lse, 0, inp.sm_scale)
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dkv.float()).all()
    # a repeated id that is not valid (in the future of the query) does not count
    idx = inp.idx.clone()
    idx[3, 5] = idx[3, 9] = 50
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx.to(gpu), 0, inp.sm_scale)
    dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, idx.to(gpu), lse, 0, inp.sm_scale)
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dkv.float()).all()


def test_forward_and_backward_with_attention_sink(gpu):
    from loongforge_amd import ops

    S, H, K, q_start = 200, 128, 128, 40
    inp = O.make_mla_inputs(S, H, K, seed=7, skv=300, q_start=q_start)
    idx = inp.idx.clone()
    idx[9, :] = -1                                                  # a row with only the sink
    g = torch.Generator().manual_seed(3)
    sink = torch.randn(H, generator=g) * 3.0
    sink[0], sink[1], sink[2] = 60.0, -60.0, 0.0                    # dominant, negligible, neutral
    q, kv, ids, do = inp.q.to(gpu), inp.kv.to(gpu), idx.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, ids, q_start, inp.sm_scale, attn_sink=sink.to(gpu))
    ro, rl, _ = O.sparse_mla_fwd(inp.q, inp.kv, idx, q_start, inp.sm_scale, 512, attn_sink=sink)
    assert_close(out, ro, "out")
    assert torch.isfinite(lse).all()
    assert (lse.cpu() - rl).abs().max().item() < 1e-4
    assert (lse[9].cpu() - sink).abs().max().item() < 1e-5 and out[9].abs().max().item() == 0
    # without a sink the same call is unchanged by the extra argument
    o0, l0, _ = ops.sparse_mla_fwd(q, kv, ids, q_start, inp.sm_scale)
    o1, l1, _ = ops.sparse_mla_fwd(q, kv, ids, q_start, inp.sm_scale, attn_sink=None)
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, ids, lse, q_start, inp.sm_scale)
    assert_mla_grads(dq, dkv, inp.q, inp.kv, idx, inp.dout, q_start, inp.sm_scale, attn_sink=sink, out=out, lse=lse)


def test_sink_survives_the_exact_pass(gpu):
    # a late dominant key sends the query through the second (exact-maximum) pass; the sink term
    # must be applied there as well
    from loongforge_amd import ops

    inp = O.make_mla_inputs(80, 128, 64, seed=6)
    kv = inp.kv.clone().float()
    kv[70] = inp.q[79, 0].float() * 40.0
    kv = kv.to(torch.bfloat16)
    idx = inp.idx.clone()
    idx[79, 63] = 70
    sink = torch.linspace(-4, 4, 128)
    sink[0] = 1567.0                                 # comparable with the dominant logit of head 0 (about 1568)
    out, lse, _ = ops.sparse_mla_fwd(inp.q.to(gpu), kv.to(gpu), idx.to(gpu), 0, inp.sm_scale, attn_sink=sink.to(gpu))
    ro, rl, _ = O.sparse_mla_fwd(inp.q, kv, idx, 0, inp.sm_scale, 512, attn_sink=sink)
    assert_close(out, ro, "out", atol=4e-2)
    assert ((lse.cpu() - rl).abs() / rl.abs().clamp_min(1)).max().item() < 1e-3


def test_backward_chunked_workspace_through_the_c_abi(gpu):
    """A workspace too small for all queries at once makes the library walk the queries in chunks;
    the result must not change."""
    from loongforge_amd import _lib, ops

    inp = O.make_mla_inputs(300, 128, 128, seed=7)
    q, kv, idx, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx, 0, inp.sm_scale)
    dq1, dkv1 = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, 0, inp.sm_scale)
    lib = _lib.load()
    small = lib.dsa_sparse_mla_bwd_workspace_bytes(100, 128, 300, 128)
    ws = torch.empty(small, dtype=torch.uint8, device=gpu)
    dq2, dkv2 = torch.empty_like(q), torch.empty_like(kv)
    rc = lib.dsa_sparse_mla_bwd(q.data_ptr(), kv.data_ptr(), out.data_ptr(), do.data_ptr(), idx.data_ptr(),
                                lse.data_ptr(), 300, 128, 300, 128, 0, inp.sm_scale, 512, dq2.data_ptr(),
                                dkv2.data_ptr(), ws.data_ptr(), small, None)
    assert rc == 0, lib.dsa_last_error()
    torch.cuda.synchronize()
    assert torch.equal(dq1, dq2)
    assert (dkv1.float() - dkv2.float()).abs().max().item() <= 2 * 2.0 ** -8 * dkv1.float().abs().max().item()
    # the smallest accepted workspace, and a repeated id in the last chunk: every chunk's dQ is NaN, not only the last's
    least = lib.dsa_sparse_mla_bwd_workspace_bytes_min(300, 128, 300, 128)
    assert 0 < least <= small
    idx_dup = inp.idx.clone()
    idx_dup[299, 5] = idx_dup[299, 9]
    idx_dup = idx_dup.to(gpu)
    wl = torch.empty(least, dtype=torch.uint8, device=gpu)
    rc = lib.dsa_sparse_mla_bwd(q.data_ptr(), kv.data_ptr(), out.data_ptr(), do.data_ptr(), idx_dup.data_ptr(),
                                lse.data_ptr(), 300, 128, 300, 128, 0, inp.sm_scale, 512, dq2.data_ptr(),
                                dkv2.data_ptr(), wl.data_ptr(), least, None)
    assert rc == 0, lib.dsa_last_error()
    torch.cuda.synchronize()
    assert torch.isnan(dq2.float()).all() and torch.isnan(dkv2.float()).all()
    tiny = torch.empty(1024, dtype=torch.uint8, device=gpu)
    rc = lib.dsa_sparse_mla_bwd(q.data_ptr(), kv.data_ptr(), out.data_ptr(), do.data_ptr(), idx.data_ptr(),
                                lse.data_ptr(), 300, 128, 300, 128, 0, inp.sm_scale, 512, dq2.data_ptr(),
                                dkv2.data_ptr(), tiny.data_ptr(), 1024, None)
    assert rc == -3 and b"workspace" in lib.dsa_last_error()


def test_backward_op_workspace_is_capped_and_kept(gpu, monkeypatch):
    """ops.sparse_mla_bwd keeps its workspace between calls (one allocation per device, not one per call) and
    honours DSA_BWD_WORKSPACE_GIB: a cap below the full size makes the library walk the queries in chunks."""
    from loongforge_amd import _lib, ops

    inp = O.make_mla_inputs(300, 128, 128, seed=8)
    q, kv, idx, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx, 0, inp.sm_scale)
    ops._BWD_WS.clear()
    dq1, dkv1 = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, 0, inp.sm_scale)
    kept = ops._BWD_WS[gpu.index or 0]
    full = _lib.load().dsa_sparse_mla_bwd_workspace_bytes(300, 128, 300, 128)
    assert kept.numel() == full
    ops.sparse_mla_bwd(q, kv, out, do, idx, lse, 0, inp.sm_scale)
    assert ops._BWD_WS[gpu.index or 0] is kept                      # reused, not reallocated
    ops._BWD_WS.clear()
    small = _lib.load().dsa_sparse_mla_bwd_workspace_bytes(100, 128, 300, 128)
    monkeypatch.setenv("DSA_BWD_WORKSPACE_GIB", repr(small / 2 ** 30))
    dq2, dkv2 = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, 0, inp.sm_scale)
    assert ops._BWD_WS[gpu.index or 0].numel() <= small + 256 < full
    assert torch.equal(dq1, dq2)
    assert (dkv1.float() - dkv2.float()).abs().max().item() <= 2 * 2.0 ** -8 * dkv1.float().abs().max().item()
    ops._BWD_WS.clear()


def test_argument_errors(gpu):
    from loongforge_amd import ops

    q = torch.zeros(8, 128, 576, dtype=torch.bfloat16, device=gpu)
    kv = torch.zeros(8, 576, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError, match="multiple of 64"):
        ops.sparse_mla_fwd(q, kv, torch.zeros(8, 48, dtype=torch.int32, device=gpu))
    with pytest.raises(ValueError, match="576"):
        ops.sparse_mla_fwd(q[..., :512].contiguous(), kv, torch.zeros(8, 64, dtype=torch.int32, device=gpu))
    with pytest.raises(ValueError, match="head count"):
        ops.sparse_mla_fwd(q[:, :16].contiguous(), kv, torch.zeros(8, 64, dtype=torch.int32, device=gpu))
    with pytest.raises(ValueError, match="d_v"):
        ops.sparse_mla_fwd(q, kv, torch.zeros(8, 64, dtype=torch.int32, device=gpu), d_v=256)
    # the backward keeps one bit per key in LDS: more than 1 228 800 keys are turned down with a message
    big = torch.zeros(1_300_000, 576, dtype=torch.bfloat16, device=gpu)
    ids = torch.zeros(8, 64, dtype=torch.int32, device=gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, big, ids, 1_300_000)
    with pytest.raises(ValueError, match="at most"):
        ops.sparse_mla_bwd(q, big, out, torch.zeros_like(out), ids, lse, 1_300_000)


@pytest.mark.parametrize("S,H,K,heads,q_start,skv,seed", [
    (200, 128, 128, 128, 40, 300, 3),
    (96, 128, 64, 16, 0, None, 5),          # 16 real heads padded to 128: only they count
    (70, 64, 192, 64, 0, None, 8),
])
def test_attn_dist_from_q_kv_lse_matches_oracle_and_the_logits_path(gpu, S, H, K, heads, q_start, skv, seed):
    from loongforge_amd import ops

    inp = O.make_mla_inputs(S, H, K, seed=seed, skv=skv, q_start=q_start)
    idx = inp.idx.clone()
    idx[5, 3] = -1
    q, kv, ids = inp.q.to(gpu), inp.kv.to(gpu), idx.to(gpu)
    out, lse, p_out = ops.sparse_mla_fwd(q, kv, ids, q_start, inp.sm_scale, 512, True, torch.float32)
    got = ops.attn_dist_qk(q, kv, ids, lse, q_start, inp.sm_scale, heads)
    _, rl, rp = O.sparse_mla_fwd(inp.q, inp.kv, idx, q_start, inp.sm_scale, 512)
    ref = O.attn_dist_from_lse(inp.q, inp.kv, idx, rl, q_start, inp.sm_scale, heads)
    assert (got.cpu() - ref).abs().max().item() <= 2e-5
    assert (got.cpu() - O.attn_dist(rp[:, :heads], inp.sm_scale)).abs().max().item() <= 2e-5
    # the route through the materialised logits gives the same distribution
    via_logits = ops.attn_dist(p_out[:, :heads], inp.sm_scale)
    assert (got - via_logits).abs().max().item() <= 2e-5
    assert ((got.sum(-1) - 1.0).abs() <= 1e-4).all() and (got[5, 3] == 0).all()


def test_attn_dist_from_q_kv_lse_with_sink_is_the_softmax_over_the_slots(gpu):
    from loongforge_amd import ops

    inp = O.make_mla_inputs(120, 128, 64, seed=12)
    sink = torch.linspace(-3, 3, 128)
    q, kv, ids = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu)
    out, lse, p_out = ops.sparse_mla_fwd(q, kv, ids, 0, inp.sm_scale, 512, True, torch.float32, attn_sink=sink.to(gpu))
    got = ops.attn_dist_qk(q, kv, ids, lse, 0, inp.sm_scale, 128, attn_sink=sink.to(gpu))
    _, _, rp = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, 0, inp.sm_scale, 512)
    assert (got.cpu() - O.attn_dist(rp, inp.sm_scale)).abs().max().item() <= 5e-5


def test_random_shapes_forward_backward_distribution(gpu):
    """Sixteen seeded random shapes (32 - 128 heads, 1 - 8 tiles per query, chunk offsets, longer key arrays, slot
    lists with holes): forward, backward by the parity rule, bit-equal reruns, recomputed attention distribution."""
    import random

    from loongforge_amd import ops

    rng = random.Random(1234)
    for case in range(16):
        H = rng.choice([32, 64, 96, 128])
        K = 64 * rng.randint(1, 8)
        S = rng.randint(1, 160)
        q_start = rng.choice([0, 0, rng.randint(1, 300)])
        skv = q_start + S + rng.choice([0, 0, rng.randint(1, 100)])
        seed = rng.randint(0, 10 ** 6)
        name = "case %d S=%d H=%d K=%d q_start=%d skv=%d seed=%d" % (case, S, H, K, q_start, skv, seed)
        print(name, flush=True)
        inp = O.make_mla_inputs(S, H, K, seed=seed, skv=skv, q_start=q_start)
        if rng.random() < 0.3:
            holes = torch.rand(inp.idx.shape, generator=torch.Generator().manual_seed(seed)) < 0.3
            inp.idx[holes] = -1
        q, kv, idx, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
        out, lse, _ = ops.sparse_mla_fwd(q, kv, idx, q_start, inp.sm_scale)
        ro, rl, _ = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, q_start, inp.sm_scale)
        assert_close(out, ro, name + " out", atol=2e-2, rtol=0)
        fin = torch.isfinite(rl)
        assert torch.equal(torch.isfinite(lse.cpu()), fin), name
        assert_close(lse.cpu()[fin], rl[fin], name + " lse", atol=1e-3, rtol=0)
        dq, dkv = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, q_start, inp.sm_scale)
        dq2, dkv2 = ops.sparse_mla_bwd(q, kv, out, do, idx, lse, q_start, inp.sm_scale)
        assert torch.equal(dq, dq2) and torch.equal(dkv, dkv2), name
        assert_mla_grads(dq, dkv, inp.q, inp.kv, inp.idx, inp.dout, q_start, inp.sm_scale, name=name, out=out, lse=lse)
        target = ops.attn_dist_qk(q, kv, idx, lse, q_start, inp.sm_scale, H)
        ref = O.attn_dist_from_lse(inp.q, inp.kv, inp.idx, lse.cpu(), q_start, inp.sm_scale, H)
        assert_close(target, ref, name + " attn_dist", atol=1e-3, rtol=1e-2)
