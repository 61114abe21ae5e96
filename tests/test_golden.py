"""The committed golden fixtures: the oracle must keep reproducing them (CPU), and the HIP kernels
must match them (GPU)."""
import importlib.util
import os

import numpy as np
import pytest
import torch

from oracle import dsa_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
G = importlib.util.module_from_spec(spec)
spec.loader.exec_module(G)


def _load(name):
    return np.load(os.path.join(HERE, "golden", name), allow_pickle=False)


def test_oracle_reproduces_mla_fixture():
    ref, now = _load("mla_small.npz"), G.mla_golden()
    for k in ref.files:
        np.testing.assert_allclose(now[k], ref[k], rtol=1e-9, atol=1e-12, err_msg=k)


def test_oracle_reproduces_indexer_fixture():
    ref, now = _load("indexer_packed.npz"), G.indexer_golden()
    for k in ref.files:
        if k == "ids":      # ReLU makes exact ties common; the scores pin the selection
            continue
        np.testing.assert_allclose(now[k], ref[k], rtol=1e-9, atol=1e-12, err_msg=k)


@pytest.mark.gpu
def test_kernels_match_mla_fixture(gpu):
    from loongforge_amd import ops

    c, ref = G.MLA_CASE, _load("mla_small.npz")
    inp = O.make_mla_inputs(c["S"], c["H"], c["K"], seed=c["seed"], skv=c["skv"], q_start=c["q_start"])
    q, kv, idx, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
    out, lse, p = ops.sparse_mla_fwd(q, kv, idx, c["q_start"], inp.sm_scale, 512, True, torch.float32)
    # the backward takes the forward's out and lse as inputs (Delta = rowsum(out * dO) feels every bf16
    # rounding of out): hand it the ones the fixture was made with, the oracle's
    o_ref, l_ref, _ = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, c["q_start"], inp.sm_scale, 512)
    dq, dkv = ops.sparse_mla_bwd(q, kv, o_ref.to(torch.bfloat16).to(gpu), do, idx, l_ref.to(gpu), c["q_start"], inp.sm_scale)
    tgt = ops.attn_dist(p, inp.sm_scale)

    def close(got, want, atol, rtol=1e-2):
        assert (np.abs(got - want) <= atol + rtol * np.abs(want)).all()

    close(G.sample(out.cpu(), 5, 3, 37), ref["out"], 2e-2)
    close(G.sample(lse.cpu(), 1, 1), ref["lse"], 1e-4, 0)
    close(G.sample(tgt.cpu(), 7, 5), ref["target"], 1e-5, 1e-3)
    close(G.sample(dq.cpu(), 5, 3, 41), ref["dq"], 2e-2)
    # dKV element by element against the oracle evaluated with the kernels' rounding points; the plain
    # fp64 gradient is out of reach of any bf16-operand backward by the margin recorded in gpu_util
    from tests.gpu_util import FP32_DKV_EXCESS_LIMIT
    close(G.sample(dkv.cpu(), 3, 29), ref["dkv_kernel_rounding"], 2e-2)
    close(G.sample(dkv.cpu(), 3, 29), ref["dkv"], 2e-2 + FP32_DKV_EXCESS_LIMIT)


@pytest.mark.gpu
def test_kernels_match_indexer_fixture(gpu):
    from loongforge_amd import ops

    c, ref = G.IDX_CASE, _load("indexer_packed.npz")
    iq, ik, w = O.make_indexer_inputs(c["S"], c["Hi"], 128, seed=c["seed"])
    cu = torch.tensor(c["cu"], dtype=torch.int32)
    ks, ke = O.indexer_window(c["S"], 0, cu)
    q8, qs = ops.quant_rowwise_e4m3(iq.to(gpu))
    k8, ksc = ops.quant_rowwise_e4m3(ik.to(gpu))
    assert np.array_equal(q8.view(torch.uint8).cpu()[::9, ::5, ::7].numpy(), ref["q8"])
    assert np.array_equal(qs.cpu().numpy(), ref["q_scale"]) and np.array_equal(ksc.cpu().numpy(), ref["k_scale"])
    ws = (w.to(gpu) * qs * 128 ** -0.5).contiguous()
    logits = ops.indexer_logits(q8, ws, k8, ksc, ks.to(gpu), ke.to(gpu)).cpu()
    fin = torch.isfinite(logits)
    assert np.array_equal(fin.sum(-1).numpy(), ref["finite_count"])
    noise = 1e-4 * np.abs(ref["logits_sample"]).max()
    assert np.abs(G.sample(logits.masked_fill(~fin, 0.0), 3, 3) - ref["logits_sample"]).max() <= noise
    sc, ids = ops.indexer_topk(q8, ws, k8, ksc, ks.to(gpu), ke.to(gpu), c["K"])
    got = sc.cpu().double().numpy()
    got = np.where(np.isfinite(got), got, -1e30)      # padded slots are stored as -1e30 in the fixture
    assert np.abs(got - ref["scores"]).max() <= noise
    assert np.array_equal(ids.cpu().numpy() >= 0, ref["ids"] >= 0)
