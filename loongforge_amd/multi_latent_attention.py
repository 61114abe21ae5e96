"""Multi-latent self-attention in the absorbed form that feeds the fused sparse attention.

Counterpart, for one GPU, of ``MLASelfAttentionFused`` in
loongforge/models/common/experimental_attention_variant/multi_latent_attention.py (:66-178 constructor,
:870-1026 forward, :1028-1338 query / key preparation).  The reference class derives from Megatron's
``MLASelfAttention`` (not part of the reference tree) and adds the absorbed data flow:

    q_up  = up(q_layernorm(down(x)))                      [s, b, h, 128 + 64]
    query = [ q_up[..., :128] @ W_UK[h]  |  rope(q_up[..., 128:]) ]          [s, b, h, 512 + 64]
    key   = [ kv_layernorm(kv_down(x)[..., :512])  |  rope(kv_down(x)[..., 512:]) ]   [s, b, 512 + 64]
    out   = core_attention(query, key)                    [b, s, h, 512]     (DSAttentionFused)
    y     = linear_proj( out @ W_UV[h]^T flattened over heads )

with W_UK / W_UV the two slices of ``linear_kv_up_proj.weight`` viewed as ``[h, 128 + 128, 512]``
(:839-868).  Here the two per-head products and the rotary embedding run through HIP kernels that read
and write the attention kernel's own layouts (``fused_absorb_rope_query``, ``absorb_attention_output``,
``fused_apply_mla_rope_for_absorb_kv``); on CPU tensors, or with ``apply_rope_fusion`` off, the same
data flow runs as torch operations (the reference's ``absorb_backend == "torch"`` branch, :1304-1318).
Sequence-chunked pipelining ("chunkpipe", :468-555, :921-922, :1058-1064, :1274-1298): the compressed latent and the
rotated key position channels of every chunk are cached, a later chunk attends to ``[cached | own]`` keys, and what it
sends back to the cached keys reaches the producing chunk's own backward.  The cache itself and its method names
live in Megatron's ``MLASelfAttention`` (not in the reference tree): those names are kept where the reference calls
them (``append_chunk_key_value_cache_mla``, ``kv_compressed_cache``, ``key_pos_emb_cache`` and their ``_grad``
dictionaries, ``micro_batch_to_cache_chunk_map``), the slot book-keeping is that of the indexer's key cache.
Tensor / sequence / context parallelism, inference caches, activation offloading and the checkpoint
conversion hooks of the reference are not part of this module.  Constructor arguments of the sub-layers
follow Megatron's MLA naming from memory: parity of those argument lists is unpinned.
"""
import math
from dataclasses import dataclass
from typing import Optional, Union

import torch

from .megatron_compat import (
    AttnMaskType,
    MegatronModule,
    ModuleSpec,
    PackedSeqParams,
    ProcessGroupCollection,
    RotaryEmbedding,
    apply_rotary_pos_emb,
    build_module,
)


@dataclass
class MLASelfAttentionSubmodules:
    """Sub-layers of multi-latent self-attention (Megatron's names)."""

    linear_q_proj: Union[ModuleSpec, type] = None
    linear_q_down_proj: Union[ModuleSpec, type] = None
    linear_q_up_proj: Union[ModuleSpec, type] = None
    linear_kv_down_proj: Union[ModuleSpec, type] = None
    linear_kv_up_proj: Union[ModuleSpec, type] = None
    core_attention: Union[ModuleSpec, type] = None
    linear_proj: Union[ModuleSpec, type] = None
    q_layernorm: Union[ModuleSpec, type] = None
    kv_layernorm: Union[ModuleSpec, type] = None


class MLASelfAttentionFused(MegatronModule):
    """Absorbed multi-latent attention around :class:`loongforge_amd.dsa_fused.DSAttentionFused`."""

    def __init__(self, config, submodules: MLASelfAttentionSubmodules, layer_number: int,
                 attn_mask_type: AttnMaskType = AttnMaskType.padding, cp_comm_type: Optional[str] = None,
                 pg_collection: ProcessGroupCollection = None, is_mtp_layer: bool = False) -> None:
        super().__init__(config=config)
        cfg = self.config
        self.layer_number = layer_number
        self.attn_mask_type = attn_mask_type
        if pg_collection is None:
            pg_collection = ProcessGroupCollection.use_mpu_process_groups(required_pgs=["tp", "cp", "pp"])
        self.pg_collection = pg_collection
        self.num_attention_heads_per_partition = cfg.num_attention_heads
        self.q_head_dim = cfg.qk_head_dim + cfg.qk_pos_emb_head_dim
        self.softmax_scale = 1.0 / math.sqrt(self.q_head_dim)
        self.absorb_backend = "torch"            # the only one here: linear_kv_up_proj stays the trainable weight
        self.use_dsa_sp_first = False
        self.rotary_pos_emb = RotaryEmbedding(cfg.qk_pos_emb_head_dim, rotary_percent=cfg.rotary_percent,
                                              rotary_base=cfg.rotary_base, cp_group=self.pg_collection.cp)

        def linear(spec, n_in, n_out, init):
            return build_module(spec, n_in, n_out, config=cfg, init_method=init, bias=False, skip_bias_add=False)

        heads = cfg.num_attention_heads
        if cfg.q_lora_rank is None:
            self.linear_q_proj = linear(submodules.linear_q_proj, cfg.hidden_size, heads * self.q_head_dim, cfg.init_method)
        else:
            self.linear_q_down_proj = linear(submodules.linear_q_down_proj, cfg.hidden_size, cfg.q_lora_rank, cfg.init_method)
            self.linear_q_up_proj = linear(submodules.linear_q_up_proj, cfg.q_lora_rank, heads * self.q_head_dim, cfg.init_method)
            self.q_layernorm = build_module(submodules.q_layernorm, hidden_size=cfg.q_lora_rank, config=cfg,
                                            eps=cfg.layernorm_epsilon)
        self.linear_kv_down_proj = linear(submodules.linear_kv_down_proj, cfg.hidden_size,
                                          cfg.kv_lora_rank + cfg.qk_pos_emb_head_dim, cfg.init_method)
        self.linear_kv_up_proj = linear(submodules.linear_kv_up_proj, cfg.kv_lora_rank,
                                        heads * (cfg.qk_head_dim + cfg.v_head_dim), cfg.init_method)
        self.kv_layernorm = build_module(submodules.kv_layernorm, hidden_size=cfg.kv_lora_rank, config=cfg,
                                         eps=cfg.layernorm_epsilon)
        # the latent is both key (with its rotary part: 576 channels) and value (512 channels) of the attention
        self.core_attention = build_module(
            submodules.core_attention, config=cfg, layer_number=layer_number, attn_mask_type=attn_mask_type,
            attention_type="self", softmax_scale=self.softmax_scale, k_channels=self.q_head_dim,
            v_channels=cfg.kv_lora_rank, cp_comm_type=cp_comm_type, pg_collection=self.pg_collection,
            is_mtp_layer=is_mtp_layer)
        self.linear_proj = linear(submodules.linear_proj, heads * cfg.v_head_dim, cfg.hidden_size,
                                  getattr(cfg, "output_layer_init_method", cfg.init_method))
        if getattr(cfg, "enable_chunkpipe", False):
            self.init_chunk_key_value_cache_mla()

    # ---- chunkpipe: latent keys of the earlier chunks of the sequences in flight --------------------------
    def init_chunk_key_value_cache_mla(self) -> None:
        """One slot per chunk of a sequence (times the virtual pipeline depth, plus two per later pipeline stage),
        as for the indexer's key cache (dsa_fused.py:240-256); the compressed latent and the rotated position
        channels are kept apart, as the reference reads them (multi_latent_attention.py:530-531)."""
        from .dsa_fused import _ChunkKeySlab

        cfg = self.config
        self.num_chunks_per_seq = cfg.chunk_num_per_seq
        later_stages = self.pg_collection.pp.size() - self.pg_collection.pp.rank() - 1
        vpp = getattr(cfg, "virtual_pipeline_model_parallel_size", None)
        slots = 2 * later_stages + self.num_chunks_per_seq * (vpp if vpp is not None else 1)
        self._chunk_slab = _ChunkKeySlab(slots, cfg.chunksize)
        par = next(self.parameters(), None)
        device = par.device if par is not None else torch.device("cpu")
        dtype = getattr(cfg, "params_dtype", None) or torch.bfloat16
        self.register_buffer("kv_compressed_cache",
                             torch.zeros(slots * cfg.chunksize, cfg.micro_batch_size, cfg.kv_lora_rank, device=device,
                                         dtype=dtype), persistent=False)
        self.register_buffer("key_pos_emb_cache",
                             torch.zeros(slots * cfg.chunksize, cfg.micro_batch_size, 1, cfg.qk_pos_emb_head_dim,
                                         device=device, dtype=dtype), persistent=False)
        self.kv_compressed_cache_grad = {}       # chunk position in its sequence -> gradient sent by later chunks
        self.key_pos_emb_cache_grad = {}

    @property
    def micro_batch_to_cache_chunk_map(self):
        return self._chunk_slab.slot_of

    def _require_chunkpipe(self, what="Chunk key value cache operations require chunkpipe to be enabled."):
        if not getattr(self.config, "enable_chunkpipe", False):
            raise RuntimeError(what)

    def clear_chunk_key_value_cache(self) -> None:
        self._require_chunkpipe()
        self._chunk_slab.reset()

    def delete_chunk_key_value_cache(self, micro_batch_index: int) -> None:
        self._require_chunkpipe()
        self._chunk_slab.release(micro_batch_index)

    def _chunk_position(self):
        """(micro-batch number, position of its chunk inside the sequence): the forward counter in a forward pass,
        the backward counter while a chunk is recomputed for its backward (multi_latent_attention.py:485-489)."""
        cfg = self.config
        mb = cfg.chunkpipe_forward_microbatch if cfg.chunkpipe_forward else cfg.chunkpipe_backward_microbatch
        return mb, mb % self.num_chunks_per_seq

    def is_enable_grad_chunkpipe(self) -> bool:
        """Whether this forward will be differentiated: always when it is the recomputation before a backward; in a
        plain forward only for the last ``keep_activations_chunks`` chunks of a sequence, and never in evaluation
        (the rule of dsa_fused.py:258-287)."""
        self._require_chunkpipe("This method is valid only for Chunkpipe, please check config.enable_chunkpipe=True")
        if not self.config.chunkpipe_forward:
            return True
        if not self.training:
            return False
        pos = self.config.chunkpipe_forward_microbatch % self.num_chunks_per_seq
        return pos + self.config.keep_activations_chunks >= self.num_chunks_per_seq

    def append_chunk_key_value_cache_mla(self, kv_compressed: torch.Tensor, k_pos_emb: torch.Tensor) -> None:
        """Keeps this chunk's normalised latent ``[chunksize, b, 512]`` and rotated position channels
        ``[chunksize, b, 1, 64]`` for the later chunks of its sequence; only in a forward pass and not for the last
        chunk (multi_latent_attention.py:1297)."""
        if not self.config.chunkpipe_forward:
            return
        mb = self.config.chunkpipe_forward_microbatch
        if (mb + 1) % self.num_chunks_per_seq == 0:
            return
        rows = self._chunk_slab.take(mb)
        self.kv_compressed_cache[rows] = kv_compressed.detach().to(self.kv_compressed_cache.dtype)
        self.key_pos_emb_cache[rows] = k_pos_emb.detach().to(self.key_pos_emb_cache.dtype)

    def concat_cached_chunk_key_value_dsa(self, curr_key: torch.Tensor):
        """``([keys of the earlier chunks of this sequence | curr_key], None)`` along the sequence, a cached key being
        ``[compressed latent | rotated position channels]``; when the pass is differentiated the two cached parts are
        leaves whose gradients are collected per chunk position (multi_latent_attention.py:468-555)."""
        self._require_chunkpipe("Chunk concatenation requires chunkpipe to be enabled.")
        mb, pos = self._chunk_position()
        slab, track = self._chunk_slab, self.is_enable_grad_chunkpipe()

        def collect(store, c):
            def hook(grad):
                store[c] = store[c] + grad if c in store else grad
                return grad
            return hook

        pieces = []
        for c in range(pos):
            rows = slab.rows(slab.slot_of[mb - pos + c])
            kv_c = self.kv_compressed_cache[rows].to(curr_key.dtype, copy=True)
            pe_c = self.key_pos_emb_cache[rows].to(curr_key.dtype, copy=True)
            if track:
                kv_c.requires_grad_(True)
                pe_c.requires_grad_(True)
                kv_c.register_hook(collect(self.kv_compressed_cache_grad, c))
                pe_c.register_hook(collect(self.key_pos_emb_cache_grad, c))
            pieces.append(torch.cat([kv_c, pe_c.squeeze(-2)], dim=-1))
        pieces.append(curr_key)
        return torch.cat(pieces, dim=0), None

    # ---- W_UK, W_UV --------------------------------------------------------------------------------
    def _get_kv_up_slices(self):
        """``(k_up [h, 128, 512], v_up [h, 128, 512])``, views of ``linear_kv_up_proj.weight``
        (multi_latent_attention.py:839-868)."""
        cfg = self.config
        w = self.linear_kv_up_proj.weight.view(self.num_attention_heads_per_partition,
                                               cfg.qk_head_dim + cfg.v_head_dim, cfg.kv_lora_rank)
        return torch.split(w, [cfg.qk_head_dim, cfg.v_head_dim], dim=1)

    def _rotary(self, hidden_states, packed_seq_params):
        packed = packed_seq_params is not None and packed_seq_params.qkv_format == "thd"
        seq_len = self.rotary_pos_emb.get_rotary_seq_len(None, None, hidden_states, self.config, packed_seq_params)
        cu_q = cu_kv = None
        if packed_seq_params is not None:
            cu_q = packed_seq_params.cu_seqlens_q_padded
            cu_q = packed_seq_params.cu_seqlens_q if cu_q is None else cu_q
            cu_kv = packed_seq_params.cu_seqlens_kv_padded
            cu_kv = packed_seq_params.cu_seqlens_kv if cu_kv is None else cu_kv
        return packed, seq_len, cu_q, cu_kv

    def get_query_key_value_tensors(self, hidden_states, key_value_states=None, position_ids=None,
                                    packed_seq_params: Optional[PackedSeqParams] = None, inference_context=None):
        """-> ``(query [s, b, h, 576], key [s, b, 576], None, q_compressed, kv_compressed)``; packed input drops
        the batch dimension (multi_latent_attention.py:1028-1338)."""
        assert hidden_states.ndim == 3, f"hidden_states should be 3D, [s, b, n*h], got {hidden_states.ndim}D"
        cfg = self.config
        heads = self.num_attention_heads_per_partition
        packed, seq_len, cu_q, cu_kv = self._rotary(hidden_states, packed_seq_params)
        if cfg.q_lora_rank is not None:
            q_compressed, _ = self.linear_q_down_proj(hidden_states)
        else:
            q_compressed = hidden_states
        kv_combined, _ = self.linear_kv_down_proj(hidden_states)
        kv_compressed, k_pos_emb = torch.split(kv_combined, [cfg.kv_lora_rank, cfg.qk_pos_emb_head_dim], dim=-1)
        if packed_seq_params is not None:
            q_compressed, kv_compressed, k_pos_emb = q_compressed.squeeze(1), kv_compressed.squeeze(1), k_pos_emb.squeeze(1)
        if cfg.q_lora_rank is not None:
            q_compressed = self.q_layernorm(q_compressed)
        kv_compressed = self.kv_layernorm(kv_compressed)

        q, _ = (self.linear_q_up_proj if cfg.q_lora_rank is not None else self.linear_q_proj)(q_compressed)
        q = q.view(*q.size()[:-1], heads, self.q_head_dim)
        k_up, _ = self._get_kv_up_slices()
        cp = self.pg_collection.cp
        chunkpipe = getattr(cfg, "enable_chunkpipe", False)
        if chunkpipe and packed:
            raise NotImplementedError("chunkpipe takes the [s, b, ...] layout (its cache holds chunks of equal length)")
        # a chunk's tokens sit at their positions in the whole sequence (multi_latent_attention.py:1058-1064)
        pos_emb_offset = self._chunk_position()[1] * cfg.chunksize if chunkpipe else 0
        if getattr(cfg, "apply_rope_fusion", False) and hidden_states.is_cuda:
            from .dsa_fused_kernels import fused_absorb_rope_query, fused_apply_mla_rope_for_absorb_kv

            # the fused kernels index their tables by the token's place in this call: a chunk reads the tables of the
            # sequence so far from its own first position on
            cos, sin = self.rotary_pos_emb.get_cached_cos_sin(pos_emb_offset + seq_len, dtype=hidden_states.dtype,
                                                              packed_seq=packed)
            cos, sin = cos[pos_emb_offset:].contiguous(), sin[pos_emb_offset:].contiguous()
            w_uk_t = k_up.transpose(1, 2).contiguous().to(q.dtype)                     # [h, 512, 128]
            query = fused_absorb_rope_query(q, w_uk_t, cos, sin, cu_q, cp.rank(), cp.size())
            key = fused_apply_mla_rope_for_absorb_kv(kv_compressed.unsqueeze(-2), k_pos_emb.unsqueeze(-2), cos, sin,
                                                     cfg.qk_pos_emb_head_dim, cfg.kv_lora_rank, cu_kv, cp.rank(),
                                                     cp.size()).squeeze(-2)
        else:
            rotary_pos_emb = self.rotary_pos_emb(seq_len, offset=pos_emb_offset, packed_seq=packed)
            q_no_pe, q_pos_emb = torch.split(q, [cfg.qk_head_dim, cfg.qk_pos_emb_head_dim], dim=-1)
            rope_cfg = _Interleaved()
            q_pos_emb = apply_rotary_pos_emb(q_pos_emb, rotary_pos_emb, config=rope_cfg, cu_seqlens=cu_q, cp_group=cp)
            k_pos_emb = apply_rotary_pos_emb(k_pos_emb.unsqueeze(-2), rotary_pos_emb, config=rope_cfg, cu_seqlens=cu_kv,
                                             cp_group=cp).squeeze(-2)
            q_content = torch.einsum("...hd,hdk->...hk", q_no_pe, k_up.to(q.dtype))
            query = torch.cat([q_content, q_pos_emb], dim=-1)
            key = torch.cat([kv_compressed, k_pos_emb], dim=-1)
        if chunkpipe:
            lat = cfg.kv_lora_rank
            if self.is_enable_grad_chunkpipe() and key.requires_grad:
                # what the later chunks of the sequence sent to this chunk's cached latent and position channels
                # (their backward ran first) joins this chunk's own key gradient (multi_latent_attention.py:1274-1296)
                pos, last = self._chunk_position()[1], self.num_chunks_per_seq - 1

                def add_later(g):
                    if pos == last:
                        return g
                    return g + torch.cat([self.kv_compressed_cache_grad.pop(pos),
                                          self.key_pos_emb_cache_grad.pop(pos).squeeze(-2)], dim=-1).to(g.dtype)
                key.register_hook(add_later)
            self.append_chunk_key_value_cache_mla(key[..., :lat], key[..., lat:].unsqueeze(-2))
        return query.contiguous(), key.contiguous(), None, q_compressed, kv_compressed

    def forward(self, hidden_states, attention_mask, key_value_states=None, inference_context=None, rotary_pos_emb=None,
                rotary_pos_cos=None, rotary_pos_sin=None, rotary_pos_cos_sin=None, attention_bias=None,
                packed_seq_params: Optional[PackedSeqParams] = None, position_ids=None, sequence_len_offset=None,
                index_share_carrier=None, *, inference_params=None):
        """``hidden_states [s, b, hidden]`` -> ``(output [s, b, hidden], bias)`` (multi_latent_attention.py:870-1026)."""
        assert rotary_pos_emb is None, "Rotary position embeddings should not be passed into MLA."
        assert attention_bias is None, "Attention bias should not be passed into MLA."
        assert rotary_pos_cos is None and rotary_pos_sin is None, "MLA does not support Flash Decoding"
        assert not rotary_pos_cos_sin, "Flash-infer rope has not been tested with MLA."
        assert inference_context is None and inference_params is None, "inference caches are not part of this module"
        query, key, value, q_compressed, _ = self.get_query_key_value_tensors(
            hidden_states, key_value_states, position_ids, packed_seq_params)
        if getattr(self.config, "enable_chunkpipe", False):
            key, value = self.concat_cached_chunk_key_value_dsa(key)       # [cached chunks | this chunk]
            key = key.contiguous()
        core_attn_out = self.core_attention(
            query, key, value, attention_mask, packed_seq_params=packed_seq_params, attn_mask_type=self.attn_mask_type,
            x=hidden_states, qr=q_compressed, index_share_carrier=index_share_carrier)
        _, v_up = self._get_kv_up_slices()
        if core_attn_out.is_cuda:
            from .dsa_fused_kernels import absorb_attention_output

            core_attn_out = absorb_attention_output(core_attn_out, v_up.contiguous().to(core_attn_out.dtype))
        else:
            core_attn_out = torch.einsum("...hk,hdk->...hd", core_attn_out, v_up.to(core_attn_out.dtype)).flatten(-2, -1)
        if packed_seq_params is not None and packed_seq_params.qkv_format == "thd":
            core_attn_out = core_attn_out.reshape(core_attn_out.size(0), 1, -1)
        else:
            core_attn_out = core_attn_out.transpose(0, 1)        # the attention returns [b, s, ...]; the projection takes [s, b, ...]
        return self.linear_proj(core_attn_out.contiguous())


class _Interleaved:
    """Rotary configuration of MLA: channel pairs are adjacent in the projection's output."""

    multi_latent_attention = True
