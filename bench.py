#!/usr/bin/env python3
"""Benchmark of the fused DSA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --config {1,3,5}      one timing row for another configuration of BASELINE.json

One step = one pass of the hot path at sequence length 8192 with all inputs resident in HBM:
  * lightning indexer (fp8, 64 heads x 128) + causal top-k 2048        (benchmark config 2)
  * sparse MLA forward + backward, 128 heads, d_qk 576, d_v 512, top-k 2048   (config 4)
Prints ONE JSON line.  `value` is the sparse-MLA forward+backward rate in TFLOP/s (algorithmic
flops: 2*H*(576+512) forward and 2*H*(3*576+2*512) backward per valid (query, key) pair, pairs =
sum_q min(prefix_q, 2048)); the indexer + top-k rate in tokens/s is reported next to it.
`roofline` describes the longest-running launch of the step, timed live with HIP events, against
the bf16 MFMA peak (its share of the algorithmic flops); the HBM bytes the design moves are beside it;
`cpu_baseline` is the CPU oracle (a PyTorch restatement of the reference's math) on a bounded
sample of the same workload, on this box's host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

S, H, K, HI = 8192, 128, 2048, 64
DQK, DV = 576, 512
PEAK_BF16 = 2500.0      # TFLOP/s, dense
PEAK_FP8 = 5000.0


def cpu_baseline(inp, iq, ik, w, n_queries=2048):
    """Oracle timed on an evenly spaced sample of queries (gather formulation, fp32)."""
    import torch

    from oracle import dsa_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    sel = torch.linspace(0, S - 1, n_queries).long()
    q, idx, do = inp.q[sel], inp.idx[sel], inp.dout[sel]
    pairs = int((idx >= 0).sum())
    t0 = time.time()
    # q_start = S disables the positional test (the ids are already causal for their own rows)
    O.sparse_mla_bwd(q, inp.kv, idx, do, S, inp.sm_scale, DV)       # forward + backward by autograd
    t_mla = time.time() - t0
    flops = 2.0 * H * (4 * DQK + 3 * DV) * pairs
    t0 = time.time()
    q8, qs = O.quant_rowwise_e4m3(iq[sel])
    k8, ks8 = O.quant_rowwise_e4m3(ik)
    wk, we = O.indexer_window(S, 0)
    logits = O.indexer_logits(q8, w[sel] * qs * 128 ** -0.5, k8, ks8, wk[sel], we[sel])
    O.topk_select(logits, K)
    t_idx = time.time() - t0
    return {
        "value": round(flops / t_mla / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": "%d evenly spaced queries of the seq-8192 workload: sparse-MLA fwd+bwd through the PyTorch oracle "
                  "(%.1f s); indexer+top-k on the same queries (%.1f s)" % (n_queries, t_mla, t_idx),
        "indexer_topk_tokens_per_s": round(n_queries / t_idx, 1),
    }


def kernel_sources_sha256():
    """Digest of the kernel sources: a committed counter profile counts only for the sources it was taken with."""
    import glob
    import hashlib

    h = hashlib.sha256()
    base = os.path.join(ROOT, "loongforge_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(base, "*.hip")) + glob.glob(os.path.join(base, "*.h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def timed_ms(torch, fn, reps=5):
    """Average time of `fn` over `reps` calls after one untimed call (events on the current stream)."""
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def config_row(n):
    """One JSON line for configuration n of BASELINE.json (1: tiny DSA forward, 3: sparse-MLA forward at
    4096 tokens, 5: the whole fused path forward + backward on 32768 packed tokens).  Timing rows beside the
    headline, not the headline: the parity of these configurations is the business of tests/."""
    import torch

    from loongforge_amd import ops
    from oracle import dsa_oracle as O

    dev = torch.device("cuda:0")
    row = {"n_gpus": 1, "data": "synthetic", "dtype": "bf16", "higher_is_better": True, "vs_baseline": None}
    if n == 3:
        S3 = 4096
        inp = O.make_mla_inputs(S3, H, K, seed=0)
        pairs = int((inp.idx >= 0).sum())
        q, kv, idx = inp.q.to(dev), inp.kv.to(dev), inp.idx.to(dev)
        t = timed_ms(torch, lambda: ops.sparse_mla_fwd(q, kv, idx, 0, inp.sm_scale), 10)
        fl = 2.0 * H * (DQK + DV) * pairs
        row.update(metric="sparse-MLA forward TFLOP/s, seq 4096, 128 heads, top-k 2048 (config 3)", unit="TFLOP/s",
                   value=round(fl / t / 1e9, 1), ms_per_step=round(t, 3), frac_of_bf16_mfma_peak=round(fl / t / 1e9 / PEAK_BF16, 4),
                   config={"workload": "config 3", "pairs": pairs})
    elif n == 1:
        S1, H1, K1 = 1024, 16, 256
        g = torch.Generator().manual_seed(0)
        q = torch.randn(S1, H1, DQK, generator=g).to(torch.bfloat16)
        kv = torch.randn(S1, DQK, generator=g).to(torch.bfloat16)
        iq = torch.randn(S1, 4, 64, generator=g).to(torch.bfloat16)
        ik = torch.randn(S1, 64, generator=g).to(torch.bfloat16)
        w = torch.rand(S1, 4, generator=g)
        sm = 192.0 ** -0.5
        t0 = time.time()
        O.dsa_forward(q, kv, iq, ik, w, K1, sm)
        t_cpu = time.time() - t0
        # the kernels take 128-wide indexer rows, 32 indexer heads and 128 query heads: zero padding is exact
        pad = torch.nn.functional.pad
        qd, kvd = pad(q, (0, 0, 0, 128 - H1)).to(dev), kv.to(dev)
        iqd, ikd, wd = pad(iq, (0, 64, 0, 28)).to(dev), pad(ik, (0, 64)).to(dev), pad(w, (0, 28)).to(dev)
        ks, ke = (x.to(dev) for x in O.indexer_window(S1, 0))

        def step():
            q8, qs, ws = ops.quant_rowwise_e4m3_weights(iqd, wd, 64 ** -0.5)
            k8, ksc = ops.quant_rowwise_e4m3(ikd)
            _, ids = ops.indexer_topk(q8, ws, k8, ksc, ks, ke, K1)
            return ops.sparse_mla_fwd(qd, kvd, ids, 0, sm)

        t = timed_ms(torch, step, 10)
        row.update(metric="tiny DSA forward tokens/s: indexer 4x64 + top-k 256 + sparse MLA 16 heads, seq 1024 (config 1)",
                   unit="tokens/s", value=round(S1 / (t * 1e-3), 1), ms_per_step=round(t, 3),
                   cpu_baseline={"value": round(S1 / t_cpu, 1), "unit": "tokens/s", "cores": os.cpu_count() or 1, "kind": "port",
                                 "sample": "the whole configuration through the PyTorch oracle (%.2f s)" % t_cpu},
                   config={"workload": "config 1"})
    elif n == 5:
        T = 32768
        os.environ.setdefault("DSA_BWD_WORKSPACE_GIB", "128")        # one sweep over all queries (105 GiB of workspace)
        cu = O.make_packed_cu_seqlens(T, 4, 2048, seed=7)
        iq, ik, w = O.make_indexer_inputs(T, HI, 128, seed=7)
        ks, ke = (x.to(dev) for x in O.indexer_window(T, 0, cu))
        iqd, ikd, wd = iq.to(dev), ik.to(dev), w.to(dev)
        g = torch.Generator(device=dev).manual_seed(7)
        q = torch.randn(T, H, DQK, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        kv = torch.randn(T, DQK, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        dout = torch.randn(T, H, DV, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        sm = 192.0 ** -0.5
        parts = {}

        def step():
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
            ev[0].record()
            q8, qs, ws = ops.quant_rowwise_e4m3_weights(iqd, wd, 128 ** -0.5)
            k8, ksc = ops.quant_rowwise_e4m3(ikd)
            sc, ids = ops.indexer_topk(q8, ws, k8, ksc, ks, ke, K)
            ev[1].record()
            # forward and head-averaged attention distribution, 12288 queries at a time: the logits of a block (6 GB)
            # are a passing buffer, the 17 GB of all of them never exist
            out, lse, target = ops.sparse_mla_fwd_dist(q, kv, ids, 0, sm, DV, H, 12288)
            ev[2].record()
            scg = sc.detach().requires_grad_(True)
            (ops.indexer_kl_loss(scg, target) * (1.0 / T)).backward()
            gs = torch.where(ids >= 0, scg.grad, torch.zeros_like(sc)).contiguous()
            ev[3].record()
            ops.indexer_bwd(gs, q8, k8, ksc, ws, ids)
            ev[4].record()
            ops.sparse_mla_bwd(q, kv, out, dout, ids, lse, 0, sm)
            ev[5].record()
            torch.cuda.synchronize()
            names = ["indexer_topk_ms", "mla_fwd_attn_dist_ms", "kl_loss_ms", "indexer_bwd_ms", "mla_bwd_ms"]
            for i, nm in enumerate(names):
                parts[nm] = round(ev[i].elapsed_time(ev[i + 1]), 3)
            return int((ids >= 0).sum())

        step()
        pairs = step()
        t = sum(parts.values())
        row.update(metric="fused DSA forward + backward tokens/s, 32768 packed tokens in 4 documents (config 5)", unit="tokens/s",
                   value=round(T / (t * 1e-3), 1), ms_per_step=round(t, 3), config={"workload": "config 5", "pairs": pairs,
                                                                                    "cu_seqlens": cu.tolist(),
                                                                                    "bwd_workspace_cap_gib": float(os.environ["DSA_BWD_WORKSPACE_GIB"])},
                   mla_fwd_bwd_tflops=round(2.0 * H * (4 * DQK + 3 * DV) * pairs / ((parts["mla_fwd_attn_dist_ms"] + parts["mla_bwd_ms"]) * 1e-3) / 1e12, 1),
                   **parts)
    else:
        raise SystemExit("bench.py --config takes 1, 3 or 5 (2 and 4 are the default run)")
    print(json.dumps(row))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device copy (reference kernel for scaling the HBM counters)")
    ap.add_argument("--config", type=int, default=0, help="print one timing row for configuration 1, 3 or 5 instead")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    from loongforge_amd import _lib, ops
    from oracle import dsa_oracle as O

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)
    if args.config:
        config_row(args.config)
        return
    lib = _lib.load()
    blib = _lib.load_bench()         # measurement aids: the backward with per-launch timing, plain movers, an MFMA loop
    dev = torch.device("cuda:0")

    # ---- synthetic inputs (CPU RNG, then resident in HBM) ------------------------------------
    inp = O.make_mla_inputs(S, H, K, seed=0)
    iq, ik, w = O.make_indexer_inputs(S, HI, 128, seed=42)
    pairs = int((inp.idx >= 0).sum())
    vis = S * (S + 1) // 2
    q, kv, idx, do = inp.q.to(dev), inp.kv.to(dev), inp.idx.to(dev), inp.dout.to(dev)
    iq_d, ik_d, w_d = iq.to(dev), ik.to(dev), w.to(dev)
    ks, ke = (t.to(dev) for t in O.indexer_window(S, 0))
    flops_fwd = 2.0 * H * (DQK + DV) * pairs
    flops_bwd = 2.0 * H * (3 * DQK + 2 * DV) * pairs
    flops_idx = 2.0 * HI * 128 * vis

    wsb = lib.dsa_sparse_mla_bwd_workspace_bytes(S, H, S, K)
    ws = torch.empty(wsb, dtype=torch.uint8, device=dev)
    dq, dkv = torch.empty_like(q), torch.empty_like(kv)
    out = torch.empty(S, H, DV, dtype=torch.bfloat16, device=dev)
    lse = torch.empty(S, H, dtype=torch.float32, device=dev)
    pass_ms = (ctypes.c_float * 5)()
    q8 = torch.empty(S, HI, 128, dtype=torch.uint8, device=dev)
    k8 = torch.empty(S, 128, dtype=torch.uint8, device=dev)
    qs = torch.empty(S, HI, dtype=torch.float32, device=dev)
    ksc = torch.empty(S, dtype=torch.float32, device=dev)
    wsd = torch.empty(S, HI, dtype=torch.float32, device=dev)
    sc = torch.empty(S, K, dtype=torch.float32, device=dev)
    ids = torch.empty(S, K, dtype=torch.int32, device=dev)
    iwsb = lib.dsa_indexer_topk_workspace_bytes(S, S, K)
    iws = torch.empty(iwsb, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def ev():
        return torch.cuda.Event(enable_timing=True)

    def indexer_calls(st):
        # straight through the C ABI on preallocated buffers, like the attention calls of the timed step
        _lib.check(lib.dsa_quant_rowwise_e4m3_weights(iq_d.data_ptr(), S * HI, 128, q8.data_ptr(), qs.data_ptr(), 1e-12, 1,
                                                      0, w_d.data_ptr(), 128 ** -0.5, wsd.data_ptr(), st), "quant q")
        _lib.check(lib.dsa_quant_rowwise_e4m3(ik_d.data_ptr(), S, 128, k8.data_ptr(), ksc.data_ptr(), 1e-12, 1, st), "quant k")
        _lib.check(lib.dsa_indexer_topk_fwd(q8.data_ptr(), wsd.data_ptr(), k8.data_ptr(), ksc.data_ptr(), ks.data_ptr(),
                                            ke.data_ptr(), S, HI, S, K, 1, sc.data_ptr(), ids.data_ptr(),
                                            iws.data_ptr(), iwsb, st), "indexer + top-k")

    indexer_calls(stream)                        # once eagerly (loads the kernels), then recorded
    torch.cuda.synchronize()
    idx_graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(idx_graph):
        indexer_calls(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    t_idx = t_fwd = t_bwd = 0.0
    t_pass = [0.0] * 5           # launch groups of the backward: order, pass A, pass C, passes B | D
    t_logits = t_topk = 0.0
    wall = 0.0
    for step in range(args.warmup + args.steps):
        timed = step >= args.warmup
        torch.cuda.synchronize()
        t0 = time.time()
        e = [ev() for _ in range(6)]
        e[0].record()
        # quantise q and k, fold the query scales into the head weights, logits + top-k: the four launches
        # recorded once into a HIP graph (below) - the kernels are short enough for the host's launch latency to
        # show between them otherwise (0.42 ms of kernels measured as 0.43 - 0.52 ms depending on the host)
        idx_graph.replay()
        e[2].record()
        _lib.check(lib.dsa_sparse_mla_fwd(q.data_ptr(), kv.data_ptr(), idx.data_ptr(), S, H, S, K, 0, inp.sm_scale, DV,
                                          out.data_ptr(), lse.data_ptr(), None, 0, stream), "fwd")
        e[3].record()
        _lib.check(lib.dsa_sparse_mla_bwd(q.data_ptr(), kv.data_ptr(), out.data_ptr(), do.data_ptr(),
                                          idx.data_ptr(), lse.data_ptr(), S, H, S, K, 0, inp.sm_scale, DV,
                                          dq.data_ptr(), dkv.data_ptr(), ws.data_ptr(), wsb, stream), "bwd")
        e[4].record()
        torch.cuda.synchronize()
        if timed:
            wall += time.time() - t0
            t_idx += e[0].elapsed_time(e[2])
            t_fwd += e[2].elapsed_time(e[3])
            t_bwd += e[3].elapsed_time(e[4])
    n = args.steps
    t_idx, t_fwd, t_bwd = t_idx / n, t_fwd / n, t_bwd / n
    # the backward's launch groups, timed by the benchmark library's copy of the same kernels (events
    # between the launches and a host wait per sweep: not part of the timed steps above)
    n_prof = 3
    for _ in range(n_prof):
        _lib.check(blib.dsa_sparse_mla_bwd_profile(q.data_ptr(), kv.data_ptr(), out.data_ptr(), do.data_ptr(),
                                                   idx.data_ptr(), lse.data_ptr(), S, H, S, K, 0, inp.sm_scale, DV,
                                                   dq.data_ptr(), dkv.data_ptr(), ws.data_ptr(), wsb, stream, pass_ms),
                   "bwd", blib)
        torch.cuda.synchronize()
        for i in range(5):
            t_pass[i] += pass_ms[i]
    t_pass = [x / n_prof for x in t_pass]
    # the indexer part alone, twenty replays in a row: inside a step it starts on caches and clocks the backward
    # of the previous step left behind, here on its own
    e0, e1 = ev(), ev()
    idx_graph.replay()
    e0.record()
    for _ in range(20):
        idx_graph.replay()
    e1.record()
    torch.cuda.synchronize()
    t_idx_alone = e0.elapsed_time(e1) / 20
    # separate timing of the two indexer kernels (logits with dense layout + top-k on it)
    lg = ops.indexer_logits(q8, wsd, k8, ksc, ks, ke)          # untimed first call
    ops.topk(lg, K, ks, ke)
    torch.cuda.synchronize()
    del lg                                                     # the timed call reuses this block: no allocation inside the timing
    e0, e1, e2 = ev(), ev(), ev()
    e0.record()
    lg = ops.indexer_logits(q8, wsd, k8, ksc, ks, ke)
    e1.record()
    ops.topk(lg, K, ks, ke)
    e2.record()
    torch.cuda.synchronize()
    t_logits, t_topk = e0.elapsed_time(e1), e1.elapsed_time(e2)
    # the remaining kernels of the path, once each after an untimed call: indexer backward on the
    # selected logits, and the head-averaged attention distribution over the forward's raw logits
    def timed(fn):
        fn()
        torch.cuda.synchronize()
        a, b = ev(), ev()
        a.record()
        r = fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b), r
    g_sel = torch.empty(S, K, dtype=torch.float32, device=dev).normal_()
    t_ibwd, _ = timed(lambda: ops.indexer_bwd(g_sel, q8, k8, ksc, wsd, ids))
    _, _, p_raw = ops.sparse_mla_fwd(q, kv, idx, 0, inp.sm_scale, DV, True)
    t_dist, _ = timed(lambda: ops.attn_dist(p_raw, inp.sm_scale))
    del p_raw, g_sel
    # the same distribution without the [S, H, K] logits: recomputed from q, kv and lse
    t_dist_qk, _ = timed(lambda: ops.attn_dist_qk(q, kv, idx, lse, 0, inp.sm_scale, H))
    # one forward with cold caches (a 1 GiB fill evicts L2 and the memory-side cache first)
    flush = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    flush.fill_(1)
    e0, e1 = ev(), ev()
    e0.record()
    _lib.check(lib.dsa_sparse_mla_fwd(q.data_ptr(), kv.data_ptr(), idx.data_ptr(), S, H, S, K, 0, inp.sm_scale, DV,
                                      out.data_ptr(), lse.data_ptr(), None, 0, stream), "fwd")
    e1.record()
    torch.cuda.synchronize()
    t_fwd_cold = e0.elapsed_time(e1)
    del flush
    # neighbouring step of the path: q_content permute + rotary embedding + concatenation at the same shape
    from loongforge_amd.dsa_fused_kernels import fused_rope_permute_cat
    qc = torch.empty(H, S, DV, dtype=torch.bfloat16, device=dev).normal_()
    qpe = torch.empty(S, 1, H, DQK - DV, dtype=torch.bfloat16, device=dev).normal_()
    ang = torch.arange(S, device=dev, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(0, 64, 2, device=dev) / 64.0))
    cos_t = torch.cat([ang.cos(), ang.cos()], -1).view(S, 1, 1, 64).contiguous()
    sin_t = torch.cat([ang.sin(), ang.sin()], -1).view(S, 1, 1, 64).contiguous()
    fused_rope_permute_cat(qc, qpe, cos_t, sin_t)
    torch.cuda.synchronize()
    e0, e1 = ev(), ev()
    e0.record()
    for _ in range(5):
        fused_rope_permute_cat(qc, qpe, cos_t, sin_t)
    e1.record()
    torch.cuda.synchronize()
    t_rope = e0.elapsed_time(e1) / 5
    del qc, qpe

    # the "next" rows either side of the path: the indexer front end behind its projections (RoPE + Hadamard rotation +
    # quantiser [+ key LayerNorm]) as one kernel per side against the separate kernels, and the MLA weight
    # absorption written straight into the attention layouts against torch.einsum + permute / concatenate
    from loongforge_amd.dsa_fused_kernels import absorb_attention_output, fused_absorb_rope_query
    cos2, sin2 = cos_t.view(S, 64).to(torch.bfloat16), sin_t.view(S, 64).to(torch.bfloat16)
    lnw, lnb = torch.ones(128, device=dev), torch.zeros(128, device=dev)

    def front_fused():
        ops.indexer_front_e4m3(iq_d, HI, None, None, 0.0, cos2, sin2, ops.ROPE_SPLIT, None, 1, True, w_d, 128 ** -0.5)
        ops.indexer_front_e4m3(ik_d, 1, lnw, lnb, 1e-5, cos2, sin2, ops.ROPE_SPLIT, None, 1, True)

    iq_s = iq_d * 1                          # the staged rotary kernel works in place: it gets its own copy

    def front_staged():
        pe = iq_s[:, :, :64]
        ops.rope_rows(pe, pe, cos2, sin2, ops.ROPE_SPLIT, ops.ROPE_SPLIT, False, None, 1)
        ops.quant_rowwise_e4m3_weights(iq_s, w_d, 128 ** -0.5, True)
        kn = torch.nn.functional.layer_norm(ik_d.float(), (128,), lnw, lnb, 1e-5).to(torch.bfloat16).unsqueeze(1)
        pk = kn[:, :, :64]
        ops.rope_rows(pk, pk, cos2, sin2, ops.ROPE_SPLIT, ops.ROPE_SPLIT, False, None, 1)
        ops.rotate_quant_e4m3(kn)

    t_front = timed_ms(torch, front_fused)
    t_front_staged = timed_ms(torch, front_staged)
    del iq_s
    q_up = torch.empty(S, H, 192, dtype=torch.bfloat16, device=dev).normal_()
    w_uk = (torch.empty(H, 128, 512, dtype=torch.bfloat16, device=dev).normal_() * 0.05)
    w_uv = (torch.empty(H, 128, 512, dtype=torch.bfloat16, device=dev).normal_() * 0.05)
    w_uk_t = w_uk.transpose(1, 2).contiguous()
    t_absorb_q = timed_ms(torch, lambda: fused_absorb_rope_query(q_up, w_uk_t, cos_t, sin_t))
    t_absorb_q_torch = timed_ms(torch, lambda: fused_rope_permute_cat(
        torch.einsum("shd,hdk->shk", q_up[:, :, :128], w_uk).permute(1, 0, 2).contiguous(), q_up[:, :, 128:], cos_t, sin_t))
    t_absorb_o = timed_ms(torch, lambda: absorb_attention_output(out, w_uv))
    t_absorb_o_torch = timed_ms(torch, lambda: torch.einsum("shk,hdk->shd", out, w_uv).flatten(-2, -1).contiguous())
    del q_up, w_uk, w_uv, w_uk_t

    # what plain data movers with the traffic shape of the two bandwidth-bound backward passes reach:
    # as many 1152-byte rows as the dKV pass writes, at scattered positions, beside a streaming read
    # of 0.6 x that size (P, dS, Q, dO); and a streaming read of the rows (the ordered sum).  Source
    # and destination are carved out of the backward's workspace, which is scratch between calls.
    rows_per_wg = int(pairs // S) // 4 * 4
    row_bytes = S * rows_per_wg * 1152
    steps4 = rows_per_wg // 4
    src_bytes = S * (steps4 // 5 * 3 + min(steps4 % 5, 3)) * 4608
    mover = None
    if row_bytes + src_bytes + 256 <= wsb:
        src_ptr = ws.data_ptr() + (row_bytes + 255) // 256 * 256
        sink = torch.zeros(16, dtype=torch.uint8, device=dev)
        t_rows, _ = timed(lambda: _lib.check(blib.dsa_probe_hbm_rows(src_ptr, ws.data_ptr(), S, rows_per_wg, 3, 1, stream),
                                             "probe rows", blib))
        t_read, _ = timed(lambda: _lib.check(blib.dsa_probe_hbm_read(ws.data_ptr(), row_bytes, sink.data_ptr(), stream),
                                             "probe read", blib))
        mover = {"rows_written_scattered_plus_stream_read_gbps": round((row_bytes + src_bytes) / (t_rows * 1e-3) / 1e9, 1),
                 "stream_read_gbps": round(row_bytes / (t_read * 1e-3) / 1e9, 1),
                 "note": "plain movers with the byte counts and access shape of bwd_dkv_kernel and bwd_reduce_kernel"}

    # what the matrix pipes sustain when a kernel issues nothing but bf16 MFMAs (about 20 ms of them)
    probe_flops = ctypes.c_double(0.0)
    sink4 = torch.zeros(4, dtype=torch.float32, device=dev)
    t_mfma, _ = timed(lambda: _lib.check(blib.dsa_probe_mfma_bf16(2048, 10000, sink4.data_ptr(), ctypes.byref(probe_flops),
                                                                  stream), "probe mfma", blib))
    mfma_sustained = probe_flops.value / (t_mfma * 1e-3) / 1e12

    mla_tflops = (flops_fwd + flops_bwd) / ((t_fwd + t_bwd) * 1e-3) / 1e12
    # ---- roofline of the longest-running launch of the step ----------------------------------------
    # Every sparse-MLA kernel is priced against the bf16 MFMA peak with its share of the algorithmic
    # flops (2*H*d per (query, key) pair and product).  Next to it: the HBM bytes this build's
    # design moves in that launch (its intermediates included), the bytes an ideal backward would
    # move, and - when a counter profile of exactly these sources is committed - the measured traffic.
    nq = float(S)
    b_q, b_do, b_o = nq * H * DQK * 2, nq * H * DV * 2, nq * H * DV * 2
    b_pds = 512.0 * pairs                     # bf16 P and dS, 128 heads, per pair
    b_rows = 1152.0 * pairs                   # one bf16 row of 576 per pair
    b_dq, b_dkv = nq * H * DQK * 2, float(S) * DQK * 2
    pass_names = ["order", "bwd_pds_kernel (S, dP -> P, dS)", "bwd_dkv_kernel (dKV rows)",
                  "bwd_dq_reduce_kernel (dQ beside the ordered dKV sum)"]
    pass_flops = [0.0, 2.0 * H * (DQK + DV) * pairs, 2.0 * H * (DQK + DV) * pairs, 2.0 * H * DQK * pairs]
    pass_bytes = [8.0 * pairs, b_q + b_do + b_o + b_pds, b_pds + b_rows + b_q + b_do,
                  0.5 * b_pds + b_dq + b_rows + S * DQK * 4.0]
    kernels = [("mla_fwd_kernel", t_fwd, flops_fwd, b_q + b_o)]
    kernels += [(pass_names[i], t_pass[i], pass_flops[i], pass_bytes[i]) for i in range(4)]
    name, t_dom, f_dom, b_dom = max(kernels, key=lambda k: k[1])
    traffic, traffic_note = None, "no counter profile committed for these kernel sources"
    tpath = os.path.join(ROOT, "profiles", "traffic.json")   # HBM bytes per launch from rocprofv3 counter runs
    if os.path.exists(tpath):
        with open(tpath) as fh:
            tj = json.load(fh)
        if tj.get("sources_sha256") == kernel_sources_sha256():
            traffic = tj.get("kernels", {}).get(name.split(" ")[0], {}).get("hbm_bytes_per_launch")
            traffic_note = "rocprofv3 FETCH_SIZE + WRITE_SIZE of profiles/traffic.json, taken with these kernel sources"
        else:
            traffic_note = "profiles/traffic.json was taken with other kernel sources: dropped"
    # The roof that binds that launch is the one it sits closer to: HBM (8 TB/s) when its bytes over its time are
    # the larger fraction of peak, else the bf16 MFMA peak; the other figure stays beside it.
    gbps_dom = b_dom / (t_dom * 1e-3) / 1e9
    tflops_dom = f_dom / (t_dom * 1e-3) / 1e12
    hbm_bound = gbps_dom / 8000.0 > tflops_dom / PEAK_BF16
    if hbm_bound:
        roofline = {"kernel": name, "bound": "hbm", "achieved": round(gbps_dom, 1), "peak": 8000.0, "unit": "GB/s"}
        roofline["mfma"] = {"achieved": round(tflops_dom, 1), "peak": PEAK_BF16, "unit": "TFLOP/s",
                            "frac": round(tflops_dom / PEAK_BF16, 4)}
    else:
        roofline = {"kernel": name, "bound": "mfma", "achieved": round(tflops_dom, 1), "peak": PEAK_BF16, "unit": "TFLOP/s"}
        roofline["hbm"] = {"achieved": round(gbps_dom, 1), "peak": 8000.0, "unit": "GB/s", "frac": round(gbps_dom / 8000.0, 4)}
    roofline["traffic"] = traffic
    roofline["traffic_note"] = traffic_note
    roofline["frac"] = round(roofline["achieved"] / roofline["peak"], 4)
    roofline["avg_launch_ms"] = round(t_dom, 3)
    roofline["algorithmic_flops"] = f_dom
    roofline["design_hbm_bytes"] = b_dom          # what this build's passes move in that launch, intermediates included
    # the whole backward: bytes an ideal implementation moves (Q, dO, O in; dQ, dKV out) against this design's
    ideal_bwd = b_q + b_do + b_o + b_dq + b_dkv
    design_bwd = sum(pass_bytes)
    roofline["backward_hbm_bytes"] = {"ideal": ideal_bwd, "design": design_bwd, "ratio": round(design_bwd / ideal_bwd, 2)}
    roofline["path_frac_of_bf16_mfma_peak"] = round(mla_tflops / PEAK_BF16, 4)
    if mover is not None:
        roofline["plain_mover_gbps"] = mover
    if args.copy_calibration:
        # a plain 1 GiB device copy: the known-size kernel the HBM counters are scaled by
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    result = {
        "metric": "sparse-MLA fwd+bwd TFLOP/s + indexer/top-k tokens/s, seq 8K, 1 GPU",
        "value": round(mla_tflops, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(t_idx + t_fwd + t_bwd, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "sparse MLA fwd+bwd seq 8192, 128 heads, d_qk 576, d_v 512, top-k 2048 (config 4) "
                               "+ fp8 lightning indexer 64x128 with causal top-k 2048 (config 2)",
                   "pairs": pairs, "visible_pairs": vis},
        "frac_of_bf16_mfma_peak": round(mla_tflops / PEAK_BF16, 4),
        "mla_fwd_ms": round(t_fwd, 3), "mla_bwd_ms": round(t_bwd, 3),
        "mla_fwd_tflops": round(flops_fwd / (t_fwd * 1e-3) / 1e12, 1),
        "mla_bwd_tflops": round(flops_bwd / (t_bwd * 1e-3) / 1e12, 1),
        "mla_bwd_pass_ms": {pass_names[i]: round(t_pass[i], 3) for i in range(4)},
        "indexer_topk_ms": round(t_idx, 3), "indexer_topk_launch": "one HIP graph of the four launches (quantise q, quantise k, logits, top-k)",
        "indexer_topk_tokens_per_s": round(S / (t_idx * 1e-3), 1),
        "indexer_topk_ms_back_to_back": round(t_idx_alone, 3),
        "indexer_topk_tokens_per_s_back_to_back": round(S / (t_idx_alone * 1e-3), 1),
        "indexer_topk_fp8_tflops": round(flops_idx / (t_idx * 1e-3) / 1e12, 1),
        "indexer_topk_frac_of_fp8_peak": round(flops_idx / (t_idx * 1e-3) / 1e12 / PEAK_FP8, 4),
        "indexer_logits_ms": round(t_logits, 3), "topk_ms": round(t_topk, 3),
        "topk_hbm_gbps": round((4.0 * vis + 8.0 * S * K) / (t_topk * 1e-3) / 1e9, 1),
        "indexer_bwd_ms": round(t_ibwd, 3),
        "attn_dist_ms": round(t_dist, 3),
        "attn_dist_gbps": round((2.0 * S * H * K + 4.0 * S * K) / (t_dist * 1e-3) / 1e9, 1),
        "attn_dist_from_q_kv_lse_ms": round(t_dist_qk, 3),
        "mla_fwd_ms_cold_caches": round(t_fwd_cold, 3),
        "mla_fwd_gather_gbps": round(2.0 * DQK * pairs / (t_fwd * 1e-3) / 1e9, 1),
        "nominal": {"note": "the same times priced on S*K pairs and S*S logits, as the reference's own print-outs do",
                    "mla_fwd_bwd_tflops": round(2.0 * H * (4 * DQK + 3 * DV) * S * K / ((t_fwd + t_bwd) * 1e-3) / 1e12, 1),
                    "indexer_topk_fp8_tflops": round(2.0 * HI * 128 * S * S / (t_idx * 1e-3) / 1e12, 1)},
        "indexer_front_end_ms": {"one_kernel_per_side": round(t_front, 3), "separate_kernels": round(t_front_staged, 3),
                                 "gbps": round((3.0 * S * HI * 128 + 3.0 * S * 128) / (t_front * 1e-3) / 1e9, 1)},
        "mla_absorb_ms": {"query_absorb_rope_in_place": round(t_absorb_q, 3), "query_einsum_permute_rope_cat": round(t_absorb_q_torch, 3),
                          "output_absorb_in_place": round(t_absorb_o, 3), "output_einsum": round(t_absorb_o_torch, 3),
                          "output_gbps": round(2.0 * S * H * (512 + 128) / (t_absorb_o * 1e-3) / 1e9, 1)},
        "rope_permute_cat_ms": round(t_rope, 3),
        "rope_permute_cat_gbps": round(4.0 * S * H * DQK / (t_rope * 1e-3) / 1e9, 1),
        "wall_s_per_step": round(wall / n, 4),
        "mfma_bf16_sustained_tflops": round(mfma_sustained, 1),
        "frac_of_sustained_bf16_mfma": round(mla_tflops / mfma_sustained, 4),
        "hbm_plain_mover": mover,
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(inp, iq, ik, w)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
