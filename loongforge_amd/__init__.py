"""MI355X-native fused DeepSeek-Sparse-Attention path (lightning indexer, top-k, sparse MLA
forward/backward) behind the reference's Python call signatures.

    from loongforge_amd import ops                      # tensor-level kernel entry points
    from loongforge_amd.dsa_fused_kernels import DSAIndexerKernel, DSADotProductAttention, triton_attn_dist
    from loongforge_amd.dsa_fused import DSAIndexerFused, DSAttentionFused
"""
__all__ = ["ops", "dsa_fused", "dsa_fused_kernels", "sparse_mla_bwd", "megatron_compat"]
