"""Constructor-wiring checks of the fused indexer module: the same two behaviours the reference's
tests/test_dsa_fused.py pins (order of the four build_module calls with the k-norm epsilon routed
only to k_norm, falling back to layernorm_epsilon; dense indexer loss rejected before anything is
built), run against this repository's dsa_fused module.

Provenance: the first two tests follow the reference's tests/test_dsa_fused.py (Apache-2.0,
Copyright Baidu; same monkeypatched names, configuration and expected error text), because that
test is the definition of "drop-in" for this module; the remaining tests are this repository's."""
from types import SimpleNamespace

import pytest
import torch

from loongforge_amd import dsa_fused


def test_fused_indexer_uses_configured_k_norm_epsilon(monkeypatch):
    recorded = []

    def init_module(self, config):
        torch.nn.Module.__init__(self)
        self.config = config

    monkeypatch.setattr(dsa_fused.MegatronModule, "__init__", init_module)
    monkeypatch.setattr(dsa_fused, "RotaryEmbedding", lambda *args, **kwargs: None)
    monkeypatch.setattr(dsa_fused, "DSAIndexerKernel", lambda: None)

    def build_module(*args, **kwargs):
        recorded.append(kwargs.get("eps"))
        return torch.nn.Identity()

    monkeypatch.setattr(dsa_fused, "build_module", build_module)

    config = SimpleNamespace(
        hidden_size=16,
        qk_pos_emb_head_dim=4,
        q_lora_rank=8,
        dsa_indexer_n_heads=2,
        dsa_indexer_head_dim=4,
        dsa_indexer_topk=8,
        rope_type="rope",
        rotary_percent=1.0,
        rotary_base=10000,
        init_method=lambda tensor: tensor,
        layernorm_epsilon=1e-5,
        dsa_indexer_k_norm_epsilon=1e-6,
        enable_chunkpipe=False,
    )
    submodules = dsa_fused.DSAIndexerFusedSubmodules(
        linear_wq_b=object(), linear_wk=object(), k_norm=object(), linear_weights_proj=object(),
    )
    dsa_fused.DSAIndexerFused(config=config, submodules=submodules, pg_collection=SimpleNamespace(cp=None))
    assert recorded == [None, None, 1e-6, None]

    config.dsa_indexer_k_norm_epsilon = None
    dsa_fused.DSAIndexerFused(config=config, submodules=submodules, pg_collection=SimpleNamespace(cp=None))
    assert recorded[-4:] == [None, None, 1e-5, None]


def test_fused_indexer_rejects_dense_indexer_loss():
    with pytest.raises(ValueError, match="only supports .*sparse_loss=True"):
        dsa_fused.DSAIndexerFused(
            config=SimpleNamespace(dsa_indexer_use_sparse_loss=False),
            submodules=None,
        )


def test_module_exposes_the_patchable_names():
    for name in ["MegatronModule", "RotaryEmbedding", "DSAIndexerKernel", "build_module",
                 "DSAIndexerFusedSubmodules", "DSAIndexerFused", "DSAttentionFusedSubmodules", "DSAttentionFused"]:
        assert hasattr(dsa_fused, name)


def test_unscale_indexer_grad_zeroes_eps_floor_rows():
    from loongforge_amd.dsa_fused_kernels import _unscale_indexer_grad

    g = torch.ones(3, 4)
    s = torch.tensor([2.0 ** -48, 2.0 ** -6, float("inf")])
    out = _unscale_indexer_grad(g, s)
    assert out[0].abs().max() == 0 and out[2].abs().max() == 0
    assert torch.equal(out[1], torch.full((4,), 64.0))


def test_rotate_activation_is_an_orthogonal_hadamard():
    x = torch.randn(5, 128).to(torch.bfloat16)
    y = dsa_fused.rotate_activation(x).float()
    assert torch.allclose(y.norm(dim=-1), x.float().norm(dim=-1), rtol=2e-2)
    h = dsa_fused._hadamard(8, "cpu", torch.float32)
    assert torch.equal(h @ h.T, 8 * torch.eye(8))


# ---- chunkpipe: the sequence arrives in chunks, the indexer keys of the earlier chunks are cached ----
class _Lin(torch.nn.Module):
    def __init__(self, n_in, n_out, **_):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty(n_out, n_in))

    def forward(self, x):
        return torch.nn.functional.linear(x, self.weight.to(x.dtype)), None


class _LN(torch.nn.LayerNorm):
    def __init__(self, config=None, hidden_size=None, eps=1e-5):
        super().__init__(hidden_size, eps=eps)


class _TorchIndexerKernel(torch.nn.Module):
    """Dense torch stand-in with the indexer kernel's calling contract (causal at global positions, top-k sorted
    by score, short rows padded with -inf / -1), differentiable, so that the host plumbing can be run without a
    GPU.  softplus takes the place of the ReLU so that no two scores tie and slot orders are comparable."""

    def forward(self, q, k, w, topk, chunk_offset=0, packed_seq_params=None):
        sq, sk = q.shape[0], k.shape[0]
        logits = (torch.nn.functional.softplus(torch.einsum("shd,td->sht", q.float(), k.float())) * w.float().unsqueeze(-1)).sum(1)
        future = torch.arange(sk)[None, :] > (torch.arange(sq) + chunk_offset)[:, None]
        sc, ids = logits.masked_fill(future, float("-inf")).topk(min(topk, sk), dim=-1)
        ids = torch.where(torch.isinf(sc), torch.full_like(ids, -1), ids)
        pad = topk - sc.shape[1]
        return torch.nn.functional.pad(sc, (0, pad), value=float("-inf")), torch.nn.functional.pad(ids, (0, pad), value=-1)


def _chunkpipe_indexer(monkeypatch, chunks, chunksize, **extra):
    monkeypatch.setattr(dsa_fused, "DSAIndexerKernel", _TorchIndexerKernel)
    cfg = SimpleNamespace(
        hidden_size=24, qk_pos_emb_head_dim=8, q_lora_rank=12, dsa_indexer_n_heads=3, dsa_indexer_head_dim=16,
        dsa_indexer_topk=20, rope_type="rope", rotary_percent=1.0, rotary_base=10000, init_method=None,
        layernorm_epsilon=1e-5, dsa_indexer_rotate_activation=False, apply_rope_fusion=False,
        enable_chunkpipe=chunks > 1, chunk_num_per_seq=chunks, chunksize=chunksize, micro_batch_size=1,
        chunkpipe_forward=True, chunkpipe_forward_microbatch=0, chunkpipe_backward_microbatch=0,
        keep_activations_chunks=chunks, virtual_pipeline_model_parallel_size=None, **extra)
    sub = dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Lin, linear_wk=_Lin, k_norm=_LN, linear_weights_proj=_Lin)
    torch.manual_seed(5)
    mod = dsa_fused.DSAIndexerFused(cfg, sub)
    for p in mod.parameters():
        if p.ndim == 2:
            torch.nn.init.normal_(p, std=p.shape[1] ** -0.5)
    return mod, cfg


def _score_loss(sc, g):
    return (torch.where(torch.isinf(sc), torch.zeros_like(sc), sc) * g).sum()


@pytest.mark.parametrize("recompute", [False, True])
def test_chunkpipe_chunks_reproduce_the_whole_sequence(monkeypatch, recompute):
    """Four chunks of one sequence through DSAIndexerFused with chunkpipe (dsa_fused.py:234-421, :524-531,
    :606-622, :674-690 of the reference) select the same keys with the same scores as the whole sequence in
    one call, and, with the backward passes run last chunk first, leave the same gradients in the weights:
    what a later chunk's scores send to an earlier chunk's keys reaches that chunk's projection.  Both
    schedules: activations kept from the forward, and every chunk recomputed before its backward."""
    C, cs = 4, 16
    S = C * cs
    whole, _ = _chunkpipe_indexer(monkeypatch, 1, S)
    chunked, cfg = _chunkpipe_indexer(monkeypatch, C, cs)
    chunked.load_state_dict(whole.state_dict())
    gen = torch.Generator().manual_seed(6)
    x, qr = torch.randn(S, 1, 24, generator=gen), torch.randn(S, 1, 12, generator=gen)
    g = torch.randn(S, 20, generator=gen)

    sc_w, ids_w = whole(x, qr)
    _score_loss(sc_w, g).backward()

    if recompute:
        cfg.keep_activations_chunks = 0
    outs = []
    for c in range(C):
        cfg.chunkpipe_forward, cfg.chunkpipe_forward_microbatch = True, c
        assert chunked.is_enable_grad_chunkpipe() == (not recompute)
        with torch.set_grad_enabled(not recompute):
            outs.append(chunked(x[c * cs:(c + 1) * cs], qr[c * cs:(c + 1) * cs]))
    assert sorted(chunked.micro_batch_to_cache_chunk_map) == [0, 1, 2]        # the last chunk is not cached
    for c, (sc, ids) in enumerate(outs):
        assert torch.equal(ids, ids_w[c * cs:(c + 1) * cs])
        assert torch.allclose(sc, sc_w[c * cs:(c + 1) * cs], rtol=1e-5, atol=1e-5)
    for c in reversed(range(C)):
        if recompute:
            cfg.chunkpipe_forward, cfg.chunkpipe_backward_microbatch = False, c
            assert chunked.is_enable_grad_chunkpipe()
            sc, _ = chunked(x[c * cs:(c + 1) * cs], qr[c * cs:(c + 1) * cs])
        else:
            sc = outs[c][0]
        _score_loss(sc, g[c * cs:(c + 1) * cs]).backward()
    assert not chunked.indexer_key_cache_grad                                 # every cached gradient was handed on
    for (n, pw), pc in zip(whole.named_parameters(), chunked.parameters()):
        assert pw.grad is not None and pc.grad is not None, n
        assert torch.allclose(pc.grad, pw.grad, rtol=1e-4, atol=1e-5), n

    # slots go back to the pool when the schedule releases a micro-batch, and run out if it never does
    for mb in range(3):
        chunked.delete_chunk_indexer_key_cache(mb)
    assert sorted(chunked.empty_chunk_indices) == list(range(C)) and not chunked.micro_batch_to_cache_chunk_map
    cfg.chunkpipe_forward = True
    with torch.no_grad():
        for mb in (0, 1, 2, 4, 5):                 # chunks 0-2 of one sequence, 0-1 of the next: a fifth slot is needed
            cfg.chunkpipe_forward_microbatch = mb
            if mb == 5:
                with pytest.raises(RuntimeError, match="No available cache chunks"):
                    chunked(x[:cs], qr[:cs])
            else:
                chunked(x[(mb % C) * cs:(mb % C + 1) * cs], qr[(mb % C) * cs:(mb % C + 1) * cs])
    chunked.clear_chunk_indexer_key_cache()
    assert len(chunked.empty_chunk_indices) == C


def test_chunkpipe_cache_calls_need_chunkpipe(monkeypatch):
    mod, _ = _chunkpipe_indexer(monkeypatch, 1, 8)
    for call in (mod.clear_chunk_indexer_key_cache, lambda: mod.delete_chunk_indexer_key_cache(0), mod.is_enable_grad_chunkpipe):
        with pytest.raises(RuntimeError):
            call()
