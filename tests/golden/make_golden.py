"""Writes the golden fixtures under tests/golden/ from the CPU oracle (oracle/dsa_oracle.py).

    python tests/golden/make_golden.py

The reference ships no golden vectors for this path and its implementation cannot be imported (its
arithmetic lives in wheels that are not in the tree), so these vectors come from this repository's
own oracle, whose functions are pinned independently in tests/test_oracle_*.py.  Inputs are
regenerated from their seeds by the tests (CPU torch.Generator); the fixtures hold strided samples
of the expected outputs plus whole-tensor sums, which keeps every file to a few kilobytes.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import dsa_oracle as O  # noqa: E402

MLA_CASE = dict(S=96, H=32, K=64, seed=11, q_start=7, skv=140)
IDX_CASE = dict(S=160, Hi=32, K=32, seed=13, cu=[0, 50, 51, 160])


def sample(t, *steps):
    sl = tuple(slice(None, None, s) for s in steps)
    return t[sl].double().numpy()


def mla_golden():
    c = MLA_CASE
    inp = O.make_mla_inputs(c["S"], c["H"], c["K"], seed=c["seed"], skv=c["skv"], q_start=c["q_start"])
    out, lse, p_out = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, c["q_start"], inp.sm_scale, 512, dtype=torch.float64)
    dq, dkv = O.sparse_mla_bwd(inp.q, inp.kv, inp.idx, inp.dout, c["q_start"], inp.sm_scale, 512, dtype=torch.float64)
    tgt = O.attn_dist(p_out.float(), inp.sm_scale)
    # dKV with the rounding points of the HIP backward (bf16 P / dS as in the reference kernel, bf16
    # per-pair rows), fp32 evaluation
    _, dkv_r = O.sparse_mla_bwd_kernel_rounding(inp.q, inp.kv, inp.idx, inp.dout, c["q_start"], inp.sm_scale, 512,
                                                round_rows_bf16=True, dtype=torch.float64)
    return dict(out=sample(out, 5, 3, 37), lse=sample(lse, 1, 1), dq=sample(dq, 5, 3, 41), dkv=sample(dkv, 3, 29),
                dkv_kernel_rounding=sample(dkv_r, 3, 29),
                target=sample(tgt, 7, 5), sums=np.array([out.sum().item(), lse.sum().item(), dq.abs().sum().item(),
                                                          dkv.abs().sum().item()]))


def indexer_golden():
    c = IDX_CASE
    iq, ik, w = O.make_indexer_inputs(c["S"], c["Hi"], 128, seed=c["seed"])
    cu = torch.tensor(c["cu"], dtype=torch.int32)
    sc, idx, aux = O.indexer_forward(iq, ik, w, c["K"], 0, cu, dtype=torch.float64)
    logits = aux["logits"]
    fin = torch.isfinite(logits)
    return dict(q8=aux["q8"].view(torch.uint8)[::9, ::5, ::7].numpy(), q_scale=aux["q_scale"].numpy(),
                k_scale=aux["k_scale"].numpy(), logits_sample=sample(logits.masked_fill(~fin, 0.0), 3, 3),
                finite_count=fin.sum(-1).numpy(), scores=sc.masked_fill(~torch.isfinite(sc), -1e30).double().numpy(),
                ids=idx.numpy())


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "mla_small.npz"), **mla_golden())
    np.savez_compressed(os.path.join(HERE, "indexer_packed.npz"), **indexer_golden())
    for f in ("mla_small.npz", "indexer_packed.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
