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
