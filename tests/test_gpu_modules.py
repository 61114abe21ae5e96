"""GPU parity of the module-level drop-in interface: DSADotProductAttention layouts, the
sparse_mla_bwd_interface function and the fused attention module with the KL indexer loss."""
from types import SimpleNamespace

import pytest
import torch

from oracle import dsa_oracle as O
from tests.gpu_util import assert_close, assert_mla_grads

pytestmark = pytest.mark.gpu


def _cfg(**kw):
    base = dict(qk_pos_emb_head_dim=64, v_head_dim=128, kv_lora_rank=512, apply_rope_fusion=False,
                num_attention_heads=128, kv_channels=192, num_layers=2)
    base.update(kw)
    return SimpleNamespace(**base)


def test_dot_product_attention_layouts_and_autograd(gpu):
    from loongforge_amd.dsa_fused_kernels import DSADotProductAttention
    from loongforge_amd.megatron_compat import AttnMaskType, PackedSeqParams

    inp = O.make_mla_inputs(150, 128, 100, seed=1)               # top-k 100 is padded to 128 inside
    attn = DSADotProductAttention(_cfg(), softmax_scale=inp.sm_scale)
    q = inp.q.to(gpu).requires_grad_(True)
    kv = inp.kv.to(gpu).requires_grad_(True)
    ids = inp.idx.to(gpu)
    # sbhd: query [sq, b=1, h, d], kv [skv, b=1, d], ids [b=1, sq, topk]
    out, p_out = attn(q.unsqueeze(1), kv.unsqueeze(1), ids.unsqueeze(0), 0, AttnMaskType.causal, return_p_out=True)
    assert out.shape == (1, 150, 128, 512) and p_out.shape == (150, 128, 128)
    ro, _, rp = O.sparse_mla_fwd(inp.q, inp.kv, inp.idx, 0, inp.sm_scale, 512)
    assert_close(out[0], ro, "out")
    assert torch.isinf(p_out[:, :, 100:]).all()
    out.backward(inp.dout.to(gpu).unsqueeze(0))
    assert_mla_grads(q.grad, kv.grad, inp.q, inp.kv, inp.idx, inp.dout, 0, inp.sm_scale, out=out[0])
    # thd: query [t, h, d], kv [t, d], ids handed as [1, t, topk]
    psp = PackedSeqParams(qkv_format="thd")
    out2 = attn(inp.q.to(gpu), inp.kv.to(gpu), ids.unsqueeze(0), 0, None, packed_seq_params=psp)
    assert out2.shape == (150, 128, 512)
    assert torch.equal(out2, out[0].detach())
    with pytest.raises(AssertionError):
        attn(q.unsqueeze(1), kv.unsqueeze(1), ids.unsqueeze(0), 0, AttnMaskType.no_mask)
    with pytest.raises(NotImplementedError):
        attn(q.unsqueeze(1), kv.unsqueeze(1), ids.unsqueeze(0), 0, None, window_size=4, return_p_out=True)
    with pytest.raises(ValueError):
        attn(q.unsqueeze(1), kv.unsqueeze(1), ids.unsqueeze(0), 0, None, window_size=64)
    # window_size: p_out leaves out the leading (window) slots, the output is unchanged
    out4, p4 = attn(q.unsqueeze(1), kv.unsqueeze(1), ids.unsqueeze(0), 0, None, window_size=64, return_p_out=True)
    assert p4.shape == (150, 128, 64) and torch.equal(p4, p_out[:, :, 64:]) and torch.equal(out4, out)
    # topk_length keeps a prefix of each query's slots; attn_sink ([h] or a divisor of it) joins the denominator
    tl = torch.randint(0, 101, (150,), generator=torch.Generator().manual_seed(4), dtype=torch.int32)
    sink = torch.linspace(-2, 2, 64)
    q.grad = kv.grad = None
    out3 = attn(q.unsqueeze(1), kv.unsqueeze(1), ids.unsqueeze(0), 0, None, topk_length=tl.to(gpu), attn_sink=sink.to(gpu))
    cut = torch.where(torch.arange(inp.idx.shape[1])[None, :] < tl[:, None], inp.idx, torch.full_like(inp.idx, -1))
    sink_h = sink.repeat_interleave(2)
    ro3, _, _ = O.sparse_mla_fwd(inp.q, inp.kv, cut, 0, inp.sm_scale, 512, attn_sink=sink_h)
    assert_close(out3[0], ro3, "out with topk_length and sink")
    out3.backward(inp.dout.to(gpu).unsqueeze(0))
    from loongforge_amd import ops
    cut_pad = torch.nn.functional.pad(cut, (0, 28), value=-1).to(gpu)          # the module pads top-k 100 to 128
    _, lse3, _ = ops.sparse_mla_fwd(q.detach(), kv.detach(), cut_pad, 0, inp.sm_scale, attn_sink=sink_h.to(gpu))
    assert_mla_grads(q.grad, kv.grad, inp.q, inp.kv, cut, inp.dout, 0, inp.sm_scale, "topk_length and sink:", attn_sink=sink_h,
                     out=out3[0], lse=lse3)


def test_sparse_mla_bwd_interface_signature(gpu):
    from loongforge_amd import ops
    from loongforge_amd.sparse_mla_bwd import sparse_mla_bwd_interface

    inp = O.make_mla_inputs(128, 128, 64, seed=2, q_start=30, skv=200)
    q, kv, idx, do = inp.q.to(gpu), inp.kv.to(gpu), inp.idx.to(gpu), inp.dout.to(gpu)
    out, lse, _ = ops.sparse_mla_fwd(q, kv, idx, 30, inp.sm_scale)
    offsets = torch.tensor([0, 128], dtype=torch.int32, device=gpu)
    dq, dkv = sparse_mla_bwd_interface(q, kv.unsqueeze(1), out, do, idx.unsqueeze(1), lse, offsets, chunk_offset=30,
                                       sm_scale=inp.sm_scale)
    assert dq.shape == q.shape and dkv.shape == (200, 1, 576)
    assert_mla_grads(dq, dkv[:, 0], inp.q, inp.kv, inp.idx, inp.dout, 30, inp.sm_scale, out=out, lse=lse)


class _Linear(torch.nn.Module):
    """Column-parallel-linear stand-in: returns (output, bias) like the Megatron layers."""

    def __init__(self, n_in, n_out, **_):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty(n_out, n_in))

    def forward(self, x):
        return torch.nn.functional.linear(x, self.weight.to(x.dtype)), None


class _Norm(torch.nn.LayerNorm):
    def __init__(self, config=None, hidden_size=None, eps=1e-5):
        super().__init__(hidden_size, eps=eps)

    def forward(self, x):
        return super().forward(x.float()).to(x.dtype)


def test_fused_attention_module_matches_oracle_pipeline(gpu):
    """The reference's tiny configuration (16 query heads, indexer 4 x 64, top-k 256, uniform head
    weights) through DSAttentionFused: indexer -> top-k -> sparse attention -> KL loss -> backward."""
    from loongforge_amd import dsa_fused
    from loongforge_amd.megatron_compat import AttnMaskType, ModuleSpec

    S, H, Hi, Di, K, hid, qlr = 512, 16, 4, 64, 256, 96, 48
    cfg = _cfg(num_attention_heads=H, hidden_size=hid, q_lora_rank=qlr, dsa_indexer_n_heads=Hi,
               dsa_indexer_head_dim=Di, dsa_indexer_topk=K, dsa_indexer_loss_coeff=1.0, rope_type="rope",
               rotary_percent=1.0, rotary_base=10000, init_method=None, layernorm_epsilon=1e-5,
               dsa_indexer_rotate_activation=True, enable_chunkpipe=False)
    sub = dsa_fused.DSAttentionFusedSubmodules(indexer=ModuleSpec(
        module=dsa_fused.DSAIndexerFused,
        submodules=dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm,
                                                       linear_weights_proj=_Linear)))
    torch.manual_seed(0)
    mod = dsa_fused.DSAttentionFused(cfg, sub, layer_number=1, attn_mask_type=AttnMaskType.causal,
                                     attention_type="self", k_channels=192)
    for p in mod.parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    mod = mod.to(gpu).train()
    g = torch.Generator().manual_seed(0)
    query = torch.randn(S, 1, H, 576, generator=g).to(torch.bfloat16).to(gpu).requires_grad_(True)
    key = torch.randn(S, 1, 576, generator=g).to(torch.bfloat16).to(gpu).requires_grad_(True)
    x = torch.randn(S, 1, hid, generator=g).to(torch.bfloat16).to(gpu)
    qr = torch.randn(S, 1, qlr, generator=g).to(torch.bfloat16).to(gpu)
    out = mod(query, key, None, None, x=x, qr=qr, attn_mask_type=AttnMaskType.causal)
    assert out.shape == (1, S, H, 512)
    loss_logged = dsa_fused.DSAIndexerLossLoggingHelperFused.tracker[1]

    # oracle pipeline on the module's own indexer output (the selection itself is checked against
    # the oracle in test_gpu_indexer.py; re-using the ids keeps this test free of boundary noise)
    with torch.no_grad():
        sc_gpu, ids_gpu = mod.indexer(x, qr)
    ids_c, sc_c = ids_gpu.cpu(), sc_gpu.cpu()
    ro, _, rp = O.sparse_mla_fwd(query.detach().cpu()[:, 0], key.detach().cpu()[:, 0], ids_c, 0, mod.softmax_scale, 512)
    target = O.attn_dist(rp[:, :H], mod.softmax_scale)
    ref = dict(out=ro, idx=ids_c, loss=O.indexer_kl_loss(sc_c, target, 1.0, S))
    assert_close(out[0], ref["out"], "out")
    assert abs(loss_logged.item() - ref["loss"].item()) <= 2e-2 * abs(ref["loss"].item()) + 1e-3

    dout = torch.randn(1, S, H, 512, generator=g).to(torch.bfloat16).to(gpu)
    out.backward(dout)
    assert_mla_grads(query.grad[:, 0], key.grad[:, 0], query.detach().cpu()[:, 0], key.detach().cpu()[:, 0], ref["idx"],
                     dout[0].cpu(), 0, mod.softmax_scale, out=out[0])
    # the indexer loss reached the indexer's weights and only those
    grads = {n: p.grad for n, p in mod.named_parameters()}
    assert all(gv is not None and torch.isfinite(gv).all() and gv.abs().max() > 0 for n, gv in grads.items()
               if "indexer" in n and "k_norm.bias" not in n)


def test_indexer_front_end_with_fused_rope_matches_the_torch_rope(gpu):
    """config.apply_rope_fusion routes the indexer's RoPE through the in-place HIP kernel
    (dsa_fused.py:435-451 of the reference); q and k must agree with the torch-op path to bf16 rounding,
    for one sequence and for a packed batch, and gradients must reach the projection weights."""
    import copy

    from loongforge_amd import dsa_fused
    from loongforge_amd.megatron_compat import PackedSeqParams

    S, Hi, Di, hid, qlr = 300, 4, 128, 96, 48
    cfg = _cfg(num_attention_heads=16, hidden_size=hid, q_lora_rank=qlr, dsa_indexer_n_heads=Hi, dsa_indexer_head_dim=Di,
               dsa_indexer_topk=64, dsa_indexer_loss_coeff=1.0, rope_type="rope", rotary_percent=1.0, rotary_base=10000,
               init_method=None, layernorm_epsilon=1e-5, dsa_indexer_rotate_activation=True, enable_chunkpipe=False)
    sub = dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm, linear_weights_proj=_Linear)
    torch.manual_seed(1)
    plain = dsa_fused.DSAIndexerFused(cfg, sub)
    for p in plain.parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    plain = plain.to(gpu)
    fused = copy.deepcopy(plain)
    fused.config = copy.copy(cfg)
    fused.config.apply_rope_fusion = True
    g = torch.Generator().manual_seed(2)
    for packed in (False, True):
        shape = (S, hid) if packed else (S, 1, hid)
        x = torch.randn(*shape, generator=g).to(torch.bfloat16).to(gpu)
        qr = torch.randn(*shape[:-1], qlr, generator=g).to(torch.bfloat16).to(gpu)
        psp = None
        if packed:
            cu = torch.tensor([0, 100, 101, 300], dtype=torch.int32, device=gpu)
            psp = PackedSeqParams(qkv_format="thd", cu_seqlens_q=cu, cu_seqlens_kv=cu, max_seqlen_q=199, max_seqlen_kv=199)
        q0, k0, w0 = plain.get_query_key_weight_tensors(x, qr, psp, defer_rotation=True)
        q1, k1, w1 = fused.get_query_key_weight_tensors(x, qr, psp, defer_rotation=True)
        assert q1.shape == q0.shape and k1.shape == k0.shape and torch.equal(w0, w1)
        for a, b in ((q1, q0), (k1, k0)):
            err = (a.float() - b.float()).abs()
            # the torch path rounds every product and the sum to bf16, the kernel once: a few units in the last
            # place of the larger of the result and its two terms (inputs here stay below 8 in magnitude)
            assert (err <= 2.0 ** -6 * (b.float().abs() + 2.0)).all()
            assert torch.equal(a[..., 64:], b[..., 64:])                      # the non-rotary half is untouched
        (q1.float().square().sum() + k1.float().square().sum()).backward()
        assert all(p.grad is not None and torch.isfinite(p.grad).all() and p.grad.abs().max() > 0
                   for n, p in fused.named_parameters() if "weights_proj" not in n and "k_norm.bias" not in n)
        fused.zero_grad()


def test_index_share_second_layer_reuses_the_first_layers_topk(gpu):
    """dsa_indexer_topk_freq = 2 (dsa_fused.py:752-778, :839-878 of the reference): layer 1 owns an indexer
    and publishes its top-k ids in the carrier, layer 2 owns none and attends over layer 1's ids; only
    the computing layer contributes an indexer loss."""
    from loongforge_amd import dsa_fused, ops
    from loongforge_amd.megatron_compat import AttnMaskType, ModuleSpec

    S, H, Hi, Di, K, hid, qlr = 320, 16, 4, 64, 64, 96, 48
    cfg = _cfg(num_attention_heads=H, hidden_size=hid, q_lora_rank=qlr, dsa_indexer_n_heads=Hi,
               dsa_indexer_head_dim=Di, dsa_indexer_topk=K, dsa_indexer_loss_coeff=1.0, rope_type="rope",
               rotary_percent=1.0, rotary_base=10000, init_method=None, layernorm_epsilon=1e-5,
               dsa_indexer_rotate_activation=True, enable_chunkpipe=False, dsa_indexer_topk_freq=2,
               dsa_indexer_skip_topk_offset=0, num_layers=2)
    sub = dsa_fused.DSAttentionFusedSubmodules(indexer=ModuleSpec(
        module=dsa_fused.DSAIndexerFused,
        submodules=dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm,
                                                       linear_weights_proj=_Linear)))
    torch.manual_seed(3)
    layers = [dsa_fused.DSAttentionFused(cfg, sub, layer_number=n, attn_mask_type=AttnMaskType.causal,
                                         attention_type="self", k_channels=192) for n in (1, 2)]
    assert layers[0].indexer is not None and not layers[0].skip_topk
    assert layers[1].indexer is None and layers[1].skip_topk and layers[1].source_layer == 1
    for p in layers[0].parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    layers = [m.to(gpu).train() for m in layers]
    g = torch.Generator().manual_seed(4)

    def rnd(*shape):
        return torch.randn(*shape, generator=g).to(torch.bfloat16).to(gpu)

    x, qr = rnd(S, 1, hid), rnd(S, 1, qlr)
    carrier = SimpleNamespace()
    dsa_fused.DSAIndexerLossLoggingHelperFused.tracker.clear()
    # the skipping layer cannot run before its source layer has
    with pytest.raises(RuntimeError, match="did not run before"):
        layers[1](rnd(S, 1, H, 576), rnd(S, 1, 576), None, None, x=x, qr=qr, attn_mask_type=AttnMaskType.causal,
                  index_share_carrier=SimpleNamespace())
    q1, k1 = rnd(S, 1, H, 576).requires_grad_(True), rnd(S, 1, 576).requires_grad_(True)
    out1 = layers[0](q1, k1, None, None, x=x, qr=qr, attn_mask_type=AttnMaskType.causal, index_share_carrier=carrier)
    ids = carrier.dsa_topk_holder[1]
    assert ids.shape == (S, K) and set(carrier.dsa_topk_holder) == {1}
    q2, k2 = rnd(S, 1, H, 576).requires_grad_(True), rnd(S, 1, 576).requires_grad_(True)
    out2 = layers[1](q2, k2, None, None, x=x, qr=qr, attn_mask_type=AttnMaskType.causal, index_share_carrier=carrier)
    assert set(carrier.dsa_topk_holder) == {1}                       # the skipping layer publishes nothing
    assert set(dsa_fused.DSAIndexerLossLoggingHelperFused.tracker) == {1}      # ... and adds no indexer loss
    # layer 2 attended over layer 1's ids: the same kernel on the same ids gives the same bits
    qp = torch.nn.functional.pad(q2.detach()[:, 0], (0, 0, 0, 128 - H))
    ref2, _, _ = ops.sparse_mla_fwd(qp, k2.detach()[:, 0], ids.int(), 0, layers[1].softmax_scale)
    assert torch.equal(out2[0], ref2[:, :H])
    ro, _, _ = O.sparse_mla_fwd(q2.detach().cpu()[:, 0], k2.detach().cpu()[:, 0], ids.cpu(), 0, layers[1].softmax_scale, 512)
    assert_close(out2[0], ro, "out of the sharing layer")
    dout = rnd(1, S, H, 512)
    (out1 * dout).sum().backward()
    (out2 * dout).sum().backward()
    assert_mla_grads(q2.grad[:, 0], k2.grad[:, 0], q2.detach().cpu()[:, 0], k2.detach().cpu()[:, 0], ids.cpu(),
                     dout[0].cpu(), 0, layers[1].softmax_scale, "sharing layer:", out=out2[0])
    assert all(p.grad is not None for n, p in layers[0].named_parameters() if "indexer" in n and "k_norm.bias" not in n)


def test_chunkpipe_chunks_through_the_kernels_match_the_whole_sequence(gpu):
    """Chunkpipe (dsa_fused.py:234-421, :674-690, :897-901 of the reference) on the HIP path: every chunk of
    a sequence, given the latent keys of the sequence so far, selects the same keys as the whole sequence in
    one call (the indexer scores chunk queries against [cached keys | own keys] at their global positions) and
    produces the same attention rows bit for bit; the indexer's weight gradients, with the chunks' backward
    passes run last chunk first, agree with the whole-sequence ones."""
    import copy

    from loongforge_amd import dsa_fused
    from loongforge_amd.megatron_compat import AttnMaskType, ModuleSpec

    C, cs, H, Hi, Di, K, hid, qlr = 3, 128, 16, 4, 128, 64, 96, 48
    S = C * cs
    base = dict(num_attention_heads=H, hidden_size=hid, q_lora_rank=qlr, dsa_indexer_n_heads=Hi,
                dsa_indexer_head_dim=Di, dsa_indexer_topk=K, dsa_indexer_loss_coeff=1.0, rope_type="rope",
                rotary_percent=1.0, rotary_base=10000, init_method=None, layernorm_epsilon=1e-5,
                dsa_indexer_rotate_activation=True)
    cfg_w = _cfg(enable_chunkpipe=False, **base)
    cfg_c = _cfg(enable_chunkpipe=True, chunk_num_per_seq=C, chunksize=cs, micro_batch_size=1, chunkpipe_forward=True,
                 chunkpipe_forward_microbatch=0, chunkpipe_backward_microbatch=0, keep_activations_chunks=C,
                 virtual_pipeline_model_parallel_size=None, **base)
    sub = dsa_fused.DSAttentionFusedSubmodules(indexer=ModuleSpec(
        module=dsa_fused.DSAIndexerFused,
        submodules=dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm,
                                                       linear_weights_proj=_Linear)))
    torch.manual_seed(7)
    whole = dsa_fused.DSAttentionFused(cfg_w, sub, layer_number=1, attn_mask_type=AttnMaskType.causal,
                                       attention_type="self", k_channels=192)
    for p in whole.parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    whole = whole.to(gpu).train()
    chunked = dsa_fused.DSAttentionFused(cfg_c, sub, layer_number=1, attn_mask_type=AttnMaskType.causal,
                                         attention_type="self", k_channels=192).to(gpu).train()
    chunked.load_state_dict(whole.state_dict())
    g = torch.Generator().manual_seed(8)

    def rnd(*shape):
        return torch.randn(*shape, generator=g).to(torch.bfloat16).to(gpu)

    query, key, x, qr, dout = rnd(S, 1, H, 576), rnd(S, 1, 576), rnd(S, 1, hid), rnd(S, 1, qlr), rnd(1, S, H, 512)
    out_w = whole(query, key, None, None, x=x, qr=qr, attn_mask_type=AttnMaskType.causal)
    with torch.no_grad():
        _, ids_w = whole.indexer(x, qr)
    (out_w * dout).sum().backward()

    outs = []
    for c in range(C):
        cfg_c.chunkpipe_forward_microbatch = c
        rows = slice(c * cs, (c + 1) * cs)
        outs.append(chunked(query[rows], key[: (c + 1) * cs], None, None, x=x[rows], qr=qr[rows],
                            attn_mask_type=AttnMaskType.causal))
        assert torch.equal(outs[-1], out_w[:, rows])
    for c in reversed(range(C)):
        (outs[c] * dout[:, c * cs:(c + 1) * cs]).sum().backward()
    assert not chunked.indexer.indexer_key_cache_grad
    for (n, pw), pc in zip(whole.named_parameters(), chunked.parameters()):
        if "k_norm.bias" in n and pw.grad is None:
            continue
        # each chunk's loss is normalised by the chunk's length (loss / sq, dsa_fused.py:940), the whole
        # sequence's by S: C times the gradient.  The key gradient reaches the projections as a sum of bf16
        # pieces, one per chunk, instead of one bf16 value.
        scale = pw.grad.abs().max().item()
        err = (pc.grad / C - pw.grad).abs().max().item()
        assert err <= 2e-2 * scale, "%s: %.3e against %.3e" % (n, err, scale)
