"""Checkpoint names of the indexer weights (configs/models/deepseek3/ckpt_convert/deepseek_v3_2_convert.yaml:40-43, 99-112)."""
import torch

from loongforge_amd import checkpoint_keys as C


def test_names_follow_the_converter_table():
    assert C.hf_to_mcore_key("model.layers.7.self_attn.indexer.wq_b.weight") == \
        "decoder.layers.7.self_attention.core_attention.indexer.linear_wq_b.weight"
    assert C.hf_to_mcore_key("model.layers.0.self_attn.indexer.k_norm.bias") == \
        "decoder.layers.0.self_attention.core_attention.indexer.k_norm.bias"
    assert C.mcore_to_hf_key("decoder.layers.60.self_attention.core_attention.indexer.linear_weights_proj.weight") == \
        "model.layers.60.self_attn.indexer.weights_proj.weight"
    assert C.hf_to_mcore_key("model.layers.3.self_attn.o_proj.weight") is None
    assert C.mcore_to_hf_key("decoder.layers.3.self_attention.linear_proj.weight") is None


def test_round_trip_and_loading_into_the_indexer_module():
    from types import SimpleNamespace

    from loongforge_amd import dsa_fused

    class _Linear(torch.nn.Module):
        def __init__(self, n_in, n_out, **_):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.empty(n_out, n_in))

        def forward(self, x):
            return torch.nn.functional.linear(x, self.weight.to(x.dtype)), None

    class _Norm(torch.nn.LayerNorm):
        def __init__(self, config=None, hidden_size=None, eps=1e-5):
            super().__init__(hidden_size, eps=eps)

    hf = {}
    for n in range(2):
        p = "model.layers.%d.self_attn.indexer." % n
        hf[p + "wq_b.weight"] = torch.randn(4 * 64, 48)
        hf[p + "wk.weight"] = torch.randn(64, 96)
        hf[p + "k_norm.weight"] = torch.randn(64)
        hf[p + "k_norm.bias"] = torch.randn(64)
        hf[p + "weights_proj.weight"] = torch.randn(4, 96)
    hf["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(1)
    mc = C.rename_indexer_entries(hf, "mcore")
    assert set(C.rename_indexer_entries(mc, "hf")) == set(hf)
    assert "model.layers.0.self_attn.o_proj.weight" in mc                      # untouched
    cfg = SimpleNamespace(qk_pos_emb_head_dim=32, hidden_size=96, q_lora_rank=48, dsa_indexer_n_heads=4,
                          dsa_indexer_head_dim=64, dsa_indexer_topk=16, rope_type="rope", rotary_percent=1.0,
                          rotary_base=10000, init_method=None, layernorm_epsilon=1e-5, enable_chunkpipe=False,
                          apply_rope_fusion=False)
    sub = dsa_fused.DSAIndexerFusedSubmodules(linear_wq_b=_Linear, linear_wk=_Linear, k_norm=_Norm, linear_weights_proj=_Linear)
    mod = dsa_fused.DSAIndexerFused(cfg, sub)
    state = C.indexer_module_state(mc, 1)
    missing, unexpected = mod.load_state_dict(state, strict=False)
    assert not unexpected and not [m for m in missing if "rotary" not in m]
    assert torch.equal(mod.linear_wk.weight, hf["model.layers.1.self_attn.indexer.wk.weight"])
