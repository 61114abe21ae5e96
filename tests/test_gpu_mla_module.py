"""GPU parity of the MLA weight-absorption kernel and of MLASelfAttentionFused (absorbed data flow through the
HIP kernels) against the textbook dense multi-latent attention of oracle/mla_module_oracle.py."""
from types import SimpleNamespace

import pytest
import torch

from oracle import mla_module_oracle as M

pytestmark = pytest.mark.gpu


def test_absorb_kernel_in_place_views_and_gradients(gpu):
    """c[s, h, :] = a[s, h, :] @ w[h].T for both shapes, reading and writing views inside larger tensors, ragged
    row counts, bit-equal to itself under re-runs and equal to the fp32 product rounded once to bf16."""
    from loongforge_amd import ops

    g = torch.Generator().manual_seed(0)
    for (k, n), S, H in (((128, 512), 333, 16), ((512, 128), 130, 128), ((128, 512), 1, 3), ((512, 128), 1000, 5)):
        big_a = torch.randn(S, H, k + 64, generator=g).to(torch.bfloat16).to(gpu)
        w = (torch.randn(H, n, k, generator=g) * k ** -0.5).to(torch.bfloat16).to(gpu)
        big_c = torch.full((S, H, n + 64), 7.0, dtype=torch.bfloat16, device=gpu)
        a, c = big_a[:, :, :k], big_c[:, :, :n]
        ops.mla_absorb_into(a, w, c)
        ref = torch.einsum("shk,hnk->shn", a.float(), w.float())
        # fp32 accumulation in a different order, one rounding: one bf16 step at most
        assert ((c.float() - ref).abs() <= 2.0 ** -7 * ref.abs() + 1e-6).all()
        assert (c == ref.to(torch.bfloat16)).float().mean().item() > 0.98
        assert (big_c[:, :, n:] == 7.0).all()                       # the neighbouring columns are untouched
        c2 = torch.empty(S, H, n, dtype=torch.bfloat16, device=gpu)
        ops.mla_absorb_into(a, w, c2)
        assert torch.equal(c2, c)
    # autograd: the two gradient products against fp32 einsum autograd
    a = torch.randn(200, 8, 128, generator=g).to(torch.bfloat16).to(gpu).requires_grad_(True)
    w = (torch.randn(8, 512, 128, generator=g) * 0.1).to(torch.bfloat16).to(gpu).requires_grad_(True)
    go = torch.randn(200, 8, 512, generator=g).to(torch.bfloat16).to(gpu)
    ops.mla_absorb(a, w).backward(go)
    a2, w2 = a.detach().float().requires_grad_(True), w.detach().float().requires_grad_(True)
    torch.einsum("shk,hnk->shn", a2, w2).backward(go.float())
    for got, ref in ((a.grad, a2.grad), (w.grad, w2.grad)):
        assert ((got.float() - ref).abs() <= 2.0 ** -6 * ref.abs() + 2.0 ** -8 * ref.abs().max()).all()
    with pytest.raises(ValueError):
        ops.mla_absorb_into(a.detach(), w.detach()[:, :100], torch.empty(200, 8, 100, dtype=torch.bfloat16, device=gpu))


class _Linear(torch.nn.Module):
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


def _module(gpu, fusion, S, H, hid, qlr, topk):
    from loongforge_amd import dsa_fused
    from loongforge_amd.megatron_compat import AttnMaskType, ModuleSpec
    from loongforge_amd.multi_latent_attention import MLASelfAttentionFused, MLASelfAttentionSubmodules

    cfg = SimpleNamespace(hidden_size=hid, num_attention_heads=H, q_lora_rank=qlr, kv_lora_rank=512, qk_head_dim=128,
                          qk_pos_emb_head_dim=64, v_head_dim=128, kv_channels=192, num_layers=1, rope_type="rope",
                          rotary_percent=1.0, rotary_base=10000, init_method=None, layernorm_epsilon=1e-5,
                          apply_rope_fusion=fusion, dsa_indexer_n_heads=4, dsa_indexer_head_dim=128, dsa_indexer_topk=topk,
                          dsa_indexer_loss_coeff=0.0, dsa_indexer_rotate_activation=True, enable_chunkpipe=False)
    indexer = ModuleSpec(module=dsa_fused.DSAIndexerFused, submodules=dsa_fused.DSAIndexerFusedSubmodules(
        linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm, linear_weights_proj=_Linear))
    core = ModuleSpec(module=dsa_fused.DSAttentionFused, submodules=dsa_fused.DSAttentionFusedSubmodules(indexer=indexer))
    sub = MLASelfAttentionSubmodules(linear_q_down_proj=_Linear, linear_q_up_proj=_Linear, linear_kv_down_proj=_Linear,
                                     linear_kv_up_proj=_Linear, core_attention=core, linear_proj=_Linear,
                                     q_layernorm=_Norm, kv_layernorm=_Norm)
    torch.manual_seed(21)
    mod = MLASelfAttentionFused(cfg, sub, layer_number=1, attn_mask_type=AttnMaskType.causal)
    for p in mod.parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    with torch.no_grad():
        for ln in (mod.q_layernorm, mod.kv_layernorm):
            ln.weight.add_(0.1 * torch.randn_like(ln.weight))
            ln.bias.add_(0.1 * torch.randn_like(ln.bias))
    return mod.to(gpu)


def _weights(mod):
    f = lambda t: t.detach().float().cpu()     # noqa: E731
    return dict(q_down=f(mod.linear_q_down_proj.weight), q_ln_w=f(mod.q_layernorm.weight), q_ln_b=f(mod.q_layernorm.bias),
                q_up=f(mod.linear_q_up_proj.weight), kv_down=f(mod.linear_kv_down_proj.weight),
                kv_ln_w=f(mod.kv_layernorm.weight), kv_ln_b=f(mod.kv_layernorm.bias), kv_up=f(mod.linear_kv_up_proj.weight),
                proj=f(mod.linear_proj.weight))


@pytest.mark.parametrize("fusion", [True, False])
def test_absorbed_mla_module_equals_dense_multi_latent_attention(gpu, fusion):
    """top-k >= sequence length makes the sparse attention dense and causal, whatever the indexer scores: the whole
    module (absorbed query, shared latent key / value, absorbed output) must then equal textbook MLA, forward and
    in the gradients of its projections.  With and without the fused rotary / absorption kernels."""
    S, H, hid, qlr = 192, 16, 128, 96
    mod = _module(gpu, fusion, S, H, hid, qlr, topk=256).train()
    g = torch.Generator().manual_seed(22)
    x = torch.randn(S, 1, hid, generator=g).to(torch.bfloat16).to(gpu)
    y, bias = mod(x, None)
    assert y.shape == (S, 1, hid) and bias is None
    p = _weights(mod)
    pr = {k: v.double().requires_grad_(True) for k, v in p.items()}
    ref = M.mla_dense(x[:, 0].double().cpu(), pr, H)
    scale = ref.abs().max().item()
    assert (y[:, 0].double().cpu() - ref).abs().max().item() <= 2e-2 * scale
    gy = torch.randn(S, 1, hid, generator=g).to(torch.bfloat16)
    y.backward(gy.to(gpu))
    ref.backward(gy[:, 0].double())
    got = dict(q_down=mod.linear_q_down_proj.weight.grad, q_up=mod.linear_q_up_proj.weight.grad,
               kv_down=mod.linear_kv_down_proj.weight.grad, kv_up=mod.linear_kv_up_proj.weight.grad,
               proj=mod.linear_proj.weight.grad, kv_ln_w=mod.kv_layernorm.weight.grad, q_ln_b=mod.q_layernorm.bias.grad)
    for name, gv in got.items():
        r = pr[name].grad
        assert gv is not None, name
        err, sc = (gv.double().cpu() - r).abs().max().item(), r.abs().max().item()
        assert err <= 4e-2 * sc, "%s: %.3e against %.3e" % (name, err, sc)


def test_absorbed_mla_module_packed_and_fused_equals_unfused(gpu):
    """Packed documents through the module; the fused-kernel data flow against the torch-operation one on the
    same weights.  top-k covers the longer document, so both attend to every key of a token's own document and
    a difference in selection between two indexers a bf16 step apart cannot hide or cause a mismatch; the second
    document must not see the first (checked against the dense oracle on the second document alone)."""
    import copy

    from loongforge_amd.megatron_compat import PackedSeqParams

    S, H, hid, qlr = 300, 16, 128, 96
    fused = _module(gpu, True, S, H, hid, qlr, topk=256).eval()
    plain = copy.deepcopy(fused)
    plain.config = copy.copy(fused.config)
    plain.config.apply_rope_fusion = False
    plain.core_attention.config = plain.config
    plain.core_attention.indexer.config = plain.config
    g = torch.Generator().manual_seed(23)
    x = torch.randn(S, 1, hid, generator=g).to(torch.bfloat16).to(gpu)
    cu = torch.tensor([0, 100, 300], dtype=torch.int32, device=gpu)
    psp = PackedSeqParams(qkv_format="thd", cu_seqlens_q=cu, cu_seqlens_kv=cu, max_seqlen_q=200, max_seqlen_kv=200)
    with torch.no_grad():
        q1, k1, _, _, _ = fused.get_query_key_value_tensors(x, packed_seq_params=psp)
        q2, k2, _, _, _ = plain.get_query_key_value_tensors(x, packed_seq_params=psp)
        assert q1.shape == (S, H, 576) and k1.shape == (S, 576)
        for a, b in ((q1, q2), (k1, k2)):
            assert ((a.float() - b.float()).abs() <= 2.0 ** -6 * (b.float().abs() + 1.0)).all()
        y1, _ = fused(x, None, packed_seq_params=psp)
        y2, _ = plain(x, None, packed_seq_params=psp)
    assert y1.shape == (S, 1, hid)
    assert (y1.float() - y2.float()).abs().max().item() <= 2e-2 * y2.float().abs().max().item()
    ref = M.mla_dense(x[100:, 0].double().cpu(), {k: v.double() for k, v in _weights(fused).items()}, H)
    assert (y1[100:, 0].double().cpu() - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()


@pytest.mark.parametrize("fusion", [False, True])
def test_chunkpipe_through_the_mla_module_matches_the_whole_sequence(gpu, fusion):
    """Chunkpipe at the level of the attention module (multi_latent_attention.py:468-555, :921-922, :1058-1064,
    :1274-1298 of the reference): the sequence arrives in chunks; every chunk caches its normalised latent and its
    rotated key position channels, attends to [cached | own] keys at their positions in the whole sequence, and the
    gradient it sends to cached keys reaches the producing chunk's backward (run last chunk first).  Outputs and
    weight gradients must agree with the same module run on the whole sequence; top-k covers the sequence, so the
    selection cannot differ."""
    import copy

    C, cs, H, hid, qlr = 3, 64, 16, 128, 96
    S = C * cs
    whole = _module(gpu, fusion, S, H, hid, qlr, topk=256).train()
    chunked = copy.deepcopy(whole)
    cfg = copy.copy(whole.config)
    cfg.__dict__.update(enable_chunkpipe=True, chunk_num_per_seq=C, chunksize=cs, micro_batch_size=1, chunkpipe_forward=True,
                        chunkpipe_forward_microbatch=0, chunkpipe_backward_microbatch=0, keep_activations_chunks=C,
                        virtual_pipeline_model_parallel_size=None)
    chunked.config = chunked.core_attention.config = chunked.core_attention.indexer.config = cfg
    chunked.init_chunk_key_value_cache_mla()
    chunked.core_attention.indexer.setup_chunkpipe_indexer_cache_config()
    chunked.core_attention.indexer.init_chunk_indexer_key_cache()
    chunked = chunked.to(gpu)
    g = torch.Generator().manual_seed(31)
    x = torch.randn(S, 1, hid, generator=g).to(torch.bfloat16).to(gpu)
    gy = torch.randn(S, 1, hid, generator=g).to(torch.bfloat16).to(gpu)
    y_w, _ = whole(x, None)
    y_w.backward(gy)
    outs = []
    for c in range(C):
        cfg.chunkpipe_forward_microbatch = c
        assert chunked.is_enable_grad_chunkpipe()
        y_c, _ = chunked(x[c * cs:(c + 1) * cs], None)
        outs.append(y_c)
        ref = y_w[c * cs:(c + 1) * cs].float()
        assert (y_c.float() - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()
    assert len(chunked.micro_batch_to_cache_chunk_map) == C - 1           # the last chunk is not cached
    for c in reversed(range(C)):
        outs[c].backward(gy[c * cs:(c + 1) * cs])
    assert not chunked.kv_compressed_cache_grad and not chunked.key_pos_emb_cache_grad
    for (n, pw), pc in zip(whole.named_parameters(), chunked.parameters()):
        if pw.grad is None:
            assert pc.grad is None or "indexer" in n, n
            continue
        scale = pw.grad.abs().max().item()
        err = (pc.grad - pw.grad).abs().max().item()
        assert err <= 4e-2 * scale, "%s: %.3e against %.3e" % (n, err, scale)
    # the schedule's calls and their guards
    chunked.delete_chunk_key_value_cache(0)
    assert len(chunked.micro_batch_to_cache_chunk_map) == C - 2
    chunked.clear_chunk_key_value_cache()
    assert not chunked.micro_batch_to_cache_chunk_map
    with pytest.raises(RuntimeError):
        whole.concat_cached_chunk_key_value_dsa(x)
