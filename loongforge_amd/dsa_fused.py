"""Fused DeepSeek-Sparse-Attention modules with the reference's class names and signatures.

Counterpart of loongforge/models/common/experimental_attention_variant/dsa_fused.py for one GPU:
``DSAIndexerFused`` (:111) computes indexer q / k / weights and calls ``DSAIndexerKernel``;
``DSAttentionFused`` (:718) runs indexer -> sparse attention -> sparse KL indexer loss.  The
tensor-parallel all-to-alls of the reference are identities at tensor-parallel size 1 and are not
present.  Sequence-chunked pipelining ("chunkpipe", dsa_fused.py:234-421) is supported for the
unpacked layout: the indexer keys of the earlier chunks of a sequence are kept in a slab, the
current chunk's queries score ``[cached keys | own keys]`` at their global positions, and the
gradient a later chunk sends to a cached key is handed to the chunk that produced it when that
chunk's backward runs.  The names
``MegatronModule``, ``RotaryEmbedding``, ``DSAIndexerKernel`` and ``build_module`` are module
attributes, as in the reference, so tests can patch them.

Provenance: the constructor argument lists, the order and keyword arguments of the four
``build_module`` calls, attribute names and error messages are the reference's (Apache-2.0,
Copyright Baidu), because its tests/test_dsa_fused.py and Megatron's ``build_module`` fix them; the
arithmetic behind the modules is this repository's HIP kernels.
"""
import copy
import math
from dataclasses import dataclass
from typing import Optional, Tuple, Union

import torch
import torch.nn.functional as F

from .dsa_fused_kernels import DSADotProductAttention, DSAIndexerKernel, triton_attn_dist
from .megatron_compat import (
    AttnMaskType,
    DSAIndexerLossAutoScaler,
    DSAIndexerLossLoggingHelper as DSAIndexerLossLoggingHelperFused,
    MegatronModule,
    ModuleSpec,
    PackedSeqParams,
    ProcessGroupCollection,
    RotaryEmbedding,
    apply_rotary_pos_emb,
    build_module,
    get_args,
    get_dsa_index_share_topk_holder,
    is_dsa_skip_topk_layer,
    source_dsa_compute_layer,
)

_HADAMARD_CACHE = {}


def _hadamard(n: int, device, dtype):
    key = (n, str(device), dtype)
    if key not in _HADAMARD_CACHE:
        assert n & (n - 1) == 0, "Hadamard size must be a power of two"
        h = torch.ones(1, 1, dtype=torch.float32)
        while h.shape[0] < n:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        _HADAMARD_CACHE[key] = h.to(device=device, dtype=dtype)
    return _HADAMARD_CACHE[key]


def rotate_activation(x: torch.Tensor) -> torch.Tensor:
    """Hadamard rotation of the last dimension scaled by ``dim ** -0.5`` (dsa_fused.py:74-90)."""
    assert x.dtype == torch.bfloat16, f"rotate_activation only support bf16 input, but got {x.dtype}"
    hidden_size = x.size(-1)
    h = _hadamard(hidden_size, x.device, torch.float32)
    return ((x.float() @ h) * hidden_size ** -0.5).to(x.dtype)


class _ChunkKeySlab:
    """Indexer keys of the chunks of the sequences in flight (dsa_fused.py:240-421).

    Book-keeping of a slab of ``slots * chunksize`` key rows (the rows themselves are a buffer of the
    module, so that they follow it between devices): a forward micro-batch (= one chunk of one
    sequence) takes a free slot, the schedule gives it back with ``release``.  ``grads`` collects, per
    chunk position inside the sequence, the gradient that later chunks' scores send to that chunk's keys.
    """

    def __init__(self, slots, chunksize):
        self.slots, self.chunksize = slots, chunksize
        self.free = list(range(slots))
        self.slot_of = {}              # forward micro-batch number -> slot
        self.grads = {}                # chunk position in its sequence -> accumulated gradient

    def rows(self, slot):
        return slice(slot * self.chunksize, (slot + 1) * self.chunksize)

    def reset(self):
        self.free = list(range(self.slots))
        self.slot_of.clear()

    def release(self, micro_batch):
        slot = self.slot_of.pop(micro_batch, None)
        if slot is not None:
            self.free.append(slot)

    def take(self, micro_batch):
        if not self.free:
            raise RuntimeError("No available cache chunks for indexer key.")
        slot = self.free.pop(0)
        self.slot_of[micro_batch] = slot
        return self.rows(slot)

    def add_grad(self, position, grad):
        if position in self.grads:
            self.grads[position] = self.grads[position] + grad
        else:
            self.grads[position] = grad


@dataclass
class DSAIndexerFusedSubmodules:
    """Submodules of the indexer: query expansion, key projection, key norm, head-weight projection."""

    linear_wq_b: Union[ModuleSpec, type] = None
    linear_wk: Union[ModuleSpec, type] = None
    k_norm: Union[ModuleSpec, type] = None
    linear_weights_proj: Union[ModuleSpec, type] = None


class DSAIndexerFused(MegatronModule):
    """Lightning indexer: scores keys per query and returns the top-k (dsa_fused.py:111-703)."""

    def __init__(self, config, submodules: DSAIndexerFusedSubmodules,
                 pg_collection: Optional[ProcessGroupCollection] = None) -> None:
        if not getattr(config, "dsa_indexer_use_sparse_loss", True):
            raise ValueError(
                "fused DSA only supports dsa_indexer_use_sparse_loss=True; "
                "use portable DSA for dense indexer loss"
            )
        super().__init__(config=config)
        self.hidden_size = self.config.hidden_size
        self.qk_pos_emb_head_dim = self.config.qk_pos_emb_head_dim
        self.q_lora_rank = (
            self.config.q_lora_rank if self.config.q_lora_rank is not None else self.config.hidden_size
        )
        self.index_n_heads = self.config.dsa_indexer_n_heads
        self.index_head_dim = self.config.dsa_indexer_head_dim
        self.index_topk = self.config.dsa_indexer_topk
        self.softmax_scale: float = self.index_head_dim ** -0.5

        if pg_collection is None:
            pg_collection = ProcessGroupCollection.use_mpu_process_groups(required_pgs=["tp", "cp", "pp"])
        self.pg_collection = pg_collection

        if self.config.rope_type == "rope":
            self.rotary_pos_emb = RotaryEmbedding(
                self.qk_pos_emb_head_dim,
                rotary_percent=self.config.rotary_percent,
                rotary_base=self.config.rotary_base,
                cp_group=self.pg_collection.cp,
            )
        else:
            raise ValueError(
                f'Unsupported RoPE type: {self.config.rope_type}, supported types are "rope" and '
                f'"yarn"'
            )

        self.linear_wq_b = build_module(
            submodules.linear_wq_b,
            self.q_lora_rank,
            self.index_n_heads * self.index_head_dim,
            config=self.config,
            init_method=self.config.init_method,
            bias=False,
            skip_bias_add=False,
            skip_weight_param_allocation=False,
            parallel_mode="duplicated",
        )
        self.linear_wk = build_module(
            submodules.linear_wk,
            self.hidden_size,
            self.index_head_dim,
            config=self.config,
            init_method=self.config.init_method,
            bias=False,
            skip_bias_add=False,
            skip_weight_param_allocation=False,
            parallel_mode="duplicated",
        )
        k_norm_config = copy.copy(self.config)
        k_norm_config.normalization = "LayerNorm"
        k_norm_eps = getattr(self.config, "dsa_indexer_k_norm_epsilon", None)
        if k_norm_eps is None:
            k_norm_eps = self.config.layernorm_epsilon
        self.k_norm = build_module(
            submodules.k_norm,
            config=k_norm_config,
            hidden_size=self.index_head_dim,
            eps=k_norm_eps,
        )
        self.linear_weights_proj = build_module(
            submodules.linear_weights_proj,
            self.hidden_size,
            self.index_n_heads,
            config=self.config,
            init_method=self.config.init_method,
            bias=False,
            skip_bias_add=False,
            skip_weight_param_allocation=False,
            parallel_mode="duplicated",
        )
        if getattr(self.config, "enable_chunkpipe", False):
            self.setup_chunkpipe_indexer_cache_config()
            self.init_chunk_indexer_key_cache()
        self.indexer_kernel = DSAIndexerKernel()

    # ---- chunkpipe: the reference's method names (its pipeline schedule calls them) over _ChunkKeySlab ----
    def setup_chunkpipe_indexer_cache_config(self) -> None:
        """Slot count of the key slab (dsa_fused.py:240-256): the chunks of one sequence, times the virtual
        pipeline depth, plus two per later pipeline stage still holding micro-batches in flight."""
        self.num_chunks_per_seq = self.config.chunk_num_per_seq
        later_stages = self.pg_collection.pp.size() - self.pg_collection.pp.rank() - 1
        vpp = getattr(self.config, "virtual_pipeline_model_parallel_size", None)
        self.indexer_key_cache_chunk_size = 2 * later_stages + self.num_chunks_per_seq * (vpp if vpp is not None else 1)

    def init_chunk_indexer_key_cache(self) -> None:
        """Allocates the slab next to the module's parameters (dsa_fused.py:289-300)."""
        par = next(self.parameters(), None)
        device = par.device if par is not None else torch.device("cpu")
        dtype = par.dtype if par is not None else torch.bfloat16
        # the reference sizes its slab by the chunks of one sequence (:293) although its slot numbers run up
        # to indexer_key_cache_chunk_size (:250-253); the slab here holds every slot
        self._chunk_slab = _ChunkKeySlab(self.indexer_key_cache_chunk_size, self.config.chunksize)
        self.register_buffer("indexer_key_cache",
                             torch.zeros(self.indexer_key_cache_chunk_size * self.config.chunksize,
                                         self.config.micro_batch_size, self.index_head_dim, device=device, dtype=dtype),
                             persistent=False)

    @property
    def indexer_key_cache_grad(self):
        return self._chunk_slab.grads

    @property
    def micro_batch_to_cache_chunk_map(self):
        return self._chunk_slab.slot_of

    @property
    def empty_chunk_indices(self):
        return self._chunk_slab.free

    def _require_chunkpipe(self, what):
        if not getattr(self.config, "enable_chunkpipe", False):
            raise RuntimeError(what)

    def clear_chunk_indexer_key_cache(self) -> None:
        self._require_chunkpipe("Chunk indexer key cache operations require chunkpipe to be enabled.")
        self._chunk_slab.reset()

    def delete_chunk_indexer_key_cache(self, micro_batch_index: int) -> None:
        self._require_chunkpipe("Chunk indexer key cache operations require chunkpipe to be enabled.")
        self._chunk_slab.release(micro_batch_index)

    def _chunk_position(self):
        """Position of the current chunk inside its sequence: the forward counter in a forward pass, the
        backward counter while a chunk is recomputed for its backward (dsa_fused.py:526-531)."""
        cfg = self.config
        mb = cfg.chunkpipe_forward_microbatch if cfg.chunkpipe_forward else cfg.chunkpipe_backward_microbatch
        return mb, mb % self.num_chunks_per_seq

    def is_enable_grad_chunkpipe(self) -> bool:
        """Whether this forward will be differentiated (dsa_fused.py:258-287): always when it is the
        recomputation before a backward; in a plain forward only for the last ``keep_activations_chunks``
        chunks of a sequence, whose activations are kept, and never in evaluation."""
        self._require_chunkpipe("This method is valid only for Chunkpipe, please check config.enable_chunkpipe=True")
        if not self.config.chunkpipe_forward:
            return True
        if not self.training:
            return False
        pos = self.config.chunkpipe_forward_microbatch % self.num_chunks_per_seq
        return pos + self.config.keep_activations_chunks >= self.num_chunks_per_seq

    def append_chunk_indexer_key_cache(self, indexer_key: torch.Tensor) -> None:
        """Keeps this chunk's keys ``[chunksize, b, d]`` for the later chunks of its sequence; only in a forward
        pass and not for the last chunk, which nobody follows (dsa_fused.py:329-361)."""
        if not getattr(self.config, "enable_chunkpipe", False) or not self.config.chunkpipe_forward:
            return
        mb = self.config.chunkpipe_forward_microbatch
        if (mb + 1) % self.num_chunks_per_seq == 0:
            return
        self.indexer_key_cache[self._chunk_slab.take(mb)] = indexer_key.detach().to(self.indexer_key_cache.dtype)

    def concat_cached_chunk_indexer_key(self, indexer_key: torch.Tensor) -> torch.Tensor:
        """``[keys of the earlier chunks of this sequence | indexer_key]`` along the sequence.  When the pass is
        differentiated every cached piece is a leaf whose gradient is collected per chunk position
        (dsa_fused.py:363-421); the producing chunk adds it to its own key gradient."""
        if not getattr(self.config, "enable_chunkpipe", False):
            return indexer_key
        mb, pos = self._chunk_position()
        slab, track = self._chunk_slab, self.is_enable_grad_chunkpipe()
        pieces = []
        for c in range(pos):
            piece = self.indexer_key_cache[slab.rows(slab.slot_of[mb - pos + c])].to(indexer_key.dtype, copy=True)
            if track:
                piece.requires_grad_(True)
                piece.register_hook(lambda g, c=c: (slab.add_grad(c, g), g)[1])
            pieces.append(piece)
        pieces.append(indexer_key)
        return torch.cat(pieces, dim=0)

    def _apply_rope(self, x, rotary_pos_emb, mscale, cu_seqlens, rotary_pos_cos=None, rotary_pos_sin=None):
        """RoPE on the leading ``qk_pos_emb_head_dim`` channels ("PE first", dsa_fused.py:423-487): the fused
        in-place kernel when ``config.apply_rope_fusion`` is set (:435-451), torch ops otherwise."""
        if getattr(self.config, "apply_rope_fusion", False) and x.is_cuda:
            from .dsa_fused_kernels import fused_apply_mla_rope

            x4 = x if (cu_seqlens is not None or x.ndim == 4) else x.unsqueeze(1)
            out = fused_apply_mla_rope(x4.contiguous(), rotary_pos_cos, rotary_pos_sin,
                                       self.index_head_dim - self.qk_pos_emb_head_dim, self.qk_pos_emb_head_dim,
                                       cu_seqlens, self.pg_collection.cp.rank(), self.pg_collection.cp.size(),
                                       pe_first=True, sp_offset=0)
            return out.view(x.shape)
        x_pe, x_nope = torch.split(
            x, [self.qk_pos_emb_head_dim, self.index_head_dim - self.qk_pos_emb_head_dim], dim=-1
        )
        indexer_rope_config = copy.copy(self.config)
        indexer_rope_config.multi_latent_attention = getattr(self.config, "dsa_indexer_rope_interleaved", False)
        x_pe = apply_rotary_pos_emb(x_pe, rotary_pos_emb, config=indexer_rope_config, cu_seqlens=cu_seqlens,
                                    mscale=mscale, cp_group=self.pg_collection.cp)
        return torch.cat([x_pe, x_nope], dim=-1)

    def get_query_key_weight_tensors(self, x, qr, packed_seq_params: Optional[PackedSeqParams] = None,
                                     defer_rotation: bool = False):
        """q ``[s, (b,) h, d]``, k ``[s, (b,) d]``, weights ``[s, (b,) h]`` (dsa_fused.py:490-638).
        ``defer_rotation`` leaves the Hadamard rotation to the caller (the indexer kernel fuses it)."""
        x = x.detach()
        qr = qr.detach()
        rotary_seq_len = self.rotary_pos_emb.get_rotary_seq_len(None, None, x, self.config, packed_seq_params)
        packed_seq = packed_seq_params is not None and packed_seq_params.qkv_format == "thd"
        chunkpipe = getattr(self.config, "enable_chunkpipe", False)
        pos_emb_offset = self._chunk_position()[1] * self.config.chunksize if chunkpipe else 0
        rotary_pos_emb = self.rotary_pos_emb(rotary_seq_len, offset=pos_emb_offset, packed_seq=packed_seq)
        mscale = 1.0
        cos = sin = None
        if getattr(self.config, "apply_rope_fusion", False):
            # the fused kernel indexes its tables by the token's place in this call: a chunk reads the tables of
            # the sequence so far from its own first position on
            cos, sin = self.rotary_pos_emb.get_cached_cos_sin(pos_emb_offset + rotary_seq_len, dtype=x.dtype,
                                                              packed_seq=packed_seq)
            cos, sin = cos[pos_emb_offset:].contiguous(), sin[pos_emb_offset:].contiguous()
        if packed_seq_params is not None:
            cu_seqlens_q = packed_seq_params.cu_seqlens_q_padded
            if cu_seqlens_q is None:
                cu_seqlens_q = packed_seq_params.cu_seqlens_q
            cu_seqlens_kv = packed_seq_params.cu_seqlens_kv_padded
            if cu_seqlens_kv is None:
                cu_seqlens_kv = packed_seq_params.cu_seqlens_kv
        else:
            cu_seqlens_q = cu_seqlens_kv = None

        q, _ = self.linear_wq_b(qr)
        q = q.view(*q.size()[:-1], self.index_n_heads, self.index_head_dim)
        q = self._apply_rope(q, rotary_pos_emb, mscale, cu_seqlens_q, cos, sin)

        k, _ = self.linear_wk(x)
        k = self.k_norm(k)
        if packed_seq_params is None:
            k = k.unsqueeze(-2)
            k = self._apply_rope(k, rotary_pos_emb, mscale, cu_seqlens_kv, cos, sin)
            k = k.squeeze(-2)
        else:
            k = self._apply_rope(k.unsqueeze(-2), rotary_pos_emb, mscale, cu_seqlens_kv, cos, sin).squeeze(-2)

        if getattr(self.config, "dsa_indexer_rotate_activation", True) and not defer_rotation:
            q = rotate_activation(q)
            k = rotate_activation(k)

        if chunkpipe and packed_seq_params is None and self.is_enable_grad_chunkpipe() and k.requires_grad:
            # what the later chunks of the sequence sent to this chunk's keys (their backward ran first) joins
            # this chunk's own key gradient (dsa_fused.py:606-622)
            pos, last = self._chunk_position()[1], self.num_chunks_per_seq - 1
            k.register_hook(lambda g: g if pos == last else g + self._chunk_slab.grads.pop(pos))

        weights, _ = self.linear_weights_proj(x)
        weights = weights * self.index_n_heads ** -0.5
        return q, k, weights

    def _fused_front_end(self, x, packed_seq_params):
        """An :class:`IndexerFrontEnd` when key LayerNorm, rotary embedding and rotation can run inside the indexer
        kernel's quantisers: fused rotary path configured, 128-channel heads with 64 rotary channels first, a k_norm
        that is a plain LayerNorm (weight, bias, eps), device tensors, no chunkpipe (its key cache holds finished keys)."""
        cfg, kern = self.config, self.indexer_kernel
        k_norm = self.k_norm
        if not (getattr(cfg, "apply_rope_fusion", False) and x.is_cuda and self.index_head_dim == 128
                and self.qk_pos_emb_head_dim == 64 and getattr(kern, "supports_fused_front_end", False)
                and not getattr(cfg, "enable_chunkpipe", False)
                and isinstance(getattr(k_norm, "weight", None), torch.Tensor)
                and isinstance(getattr(k_norm, "bias", None), torch.Tensor) and hasattr(k_norm, "eps")):
            return None
        from .dsa_fused_kernels import IndexerFrontEnd, _token_positions
        from . import ops

        packed_seq = packed_seq_params is not None and packed_seq_params.qkv_format == "thd"
        rotary_seq_len = self.rotary_pos_emb.get_rotary_seq_len(None, None, x, cfg, packed_seq_params)
        cos, sin = self.rotary_pos_emb.get_cached_cos_sin(rotary_seq_len, dtype=x.dtype, packed_seq=packed_seq)
        pos_q = pos_k = None
        if packed_seq_params is not None:
            cu_q = packed_seq_params.cu_seqlens_q_padded
            cu_q = packed_seq_params.cu_seqlens_q if cu_q is None else cu_q
            cu_k = packed_seq_params.cu_seqlens_kv_padded
            cu_k = packed_seq_params.cu_seqlens_kv if cu_k is None else cu_k
            cp = self.pg_collection.cp
            pos_q = _token_positions(cu_q, x.shape[0], cp.rank(), cp.size())
            pos_k = _token_positions(cu_k, x.shape[0], cp.rank(), cp.size())
        return IndexerFrontEnd(cos=cos.reshape(-1, 64), sin=sin.reshape(-1, 64), pairing=ops.ROPE_SPLIT, positions_q=pos_q,
                               positions_k=pos_k, batch=1 if packed_seq_params is not None else x.shape[1],
                               k_norm_eps=float(k_norm.eps))

    def forward(self, x, qr, packed_seq_params: Optional[PackedSeqParams] = None):
        """-> ``(index_score_topk [s, topk], topk_indices [s, topk])`` (dsa_fused.py:640-703)."""
        chunkpipe = getattr(self.config, "enable_chunkpipe", False)
        rotate = getattr(self.config, "dsa_indexer_rotate_activation", True)
        front = self._fused_front_end(x, packed_seq_params)
        if front is not None:
            # only the projections run here; k_norm, RoPE, rotation and quantisation are one kernel per side
            x, qr = x.detach(), qr.detach()
            q, _ = self.linear_wq_b(qr)
            q = q.view(*q.size()[:-1], self.index_n_heads, self.index_head_dim)
            k, _ = self.linear_wk(x)
            weights, _ = self.linear_weights_proj(x)
            weights = weights * self.index_n_heads ** -0.5
            if packed_seq_params is None:
                q = q.squeeze(1)
            return self.indexer_kernel(
                q.contiguous(), k.squeeze(1).contiguous(), weights.squeeze(1).contiguous(), self.index_topk,
                chunk_offset=self.pg_collection.tp.rank() * q.size(0), packed_seq_params=packed_seq_params,
                rotate=bool(rotate), front=front, k_norm_weight=self.k_norm.weight, k_norm_bias=self.k_norm.bias)
        # (with chunkpipe the cached keys are the rotated ones, so the rotation stays outside the kernel)
        fuse = (rotate and self.index_head_dim == 128
                and x.is_cuda and not chunkpipe and getattr(self.indexer_kernel, "supports_fused_rotate", False))
        indexer_query, indexer_key, indexer_weights = self.get_query_key_weight_tensors(x, qr, packed_seq_params,
                                                                                        defer_rotation=fuse)
        if packed_seq_params is None:
            indexer_query = indexer_query.squeeze(1).contiguous()
        indexer_key = indexer_key.squeeze(1).contiguous()
        indexer_weights = indexer_weights.squeeze(1).contiguous()
        if chunkpipe and packed_seq_params is None:
            self.append_chunk_indexer_key_cache(indexer_key.unsqueeze(1))
            indexer_key = self.concat_cached_chunk_indexer_key(indexer_key.unsqueeze(1)).squeeze(1)
        kv_offset = self.pg_collection.tp.rank() * indexer_query.size(0)
        if chunkpipe:
            kv_offset += self._chunk_position()[1] * self.config.chunksize
        return self.indexer_kernel(
            indexer_query,
            indexer_key,
            indexer_weights,
            self.index_topk,
            chunk_offset=kv_offset,
            packed_seq_params=packed_seq_params,
            **({"rotate": True} if fuse else {}),
        )


@dataclass
class DSAttentionFusedSubmodules:
    """Submodules of the sparse attention: the indexer."""

    indexer: Union[ModuleSpec, type] = None


class DSAttentionFused(MegatronModule):
    """Indexer -> top-k -> sparse MLA attention -> sparse KL indexer loss (dsa_fused.py:718-971)."""

    def __init__(self, config, submodules: DSAttentionFusedSubmodules, layer_number: int,
                 attn_mask_type: AttnMaskType, attention_type: str, attention_dropout: Optional[float] = None,
                 softmax_scale: Optional[float] = None, k_channels: Optional[int] = None,
                 v_channels: Optional[int] = None, cp_comm_type: str = "p2p",
                 pg_collection: ProcessGroupCollection = None, is_mtp_layer: bool = False):
        super().__init__(config=config)
        self.layer_number = layer_number
        if is_mtp_layer:
            self.layer_number = self.layer_number + self.config.num_layers
        if pg_collection is None:
            pg_collection = ProcessGroupCollection.use_mpu_process_groups(required_pgs=["tp", "cp", "pp"])
        self.pg_collection = pg_collection
        args = get_args()
        self.use_dsa_sp_first = getattr(args, "use_dsa_sp_first", False) if args is not None else False

        self.index_topk_freq = getattr(self.config, "dsa_indexer_topk_freq", 1)
        self.index_skip_topk_offset = getattr(self.config, "dsa_indexer_skip_topk_offset", 0)
        self.index_share = self.index_topk_freq > 1
        self.skip_topk = (
            self.index_share
            and not is_mtp_layer
            and is_dsa_skip_topk_layer(self.layer_number, self.index_skip_topk_offset, self.index_topk_freq)
        )
        self.source_layer = (
            source_dsa_compute_layer(self.layer_number, self.index_skip_topk_offset, self.index_topk_freq)
            if self.skip_topk
            else self.layer_number
        )
        self.indexer = None
        if not self.skip_topk:
            self.indexer = build_module(submodules.indexer, config=self.config, pg_collection=pg_collection)

        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(k_channels if k_channels is not None else config.kv_channels)
        self.softmax_scale = softmax_scale
        # the kernels behind this module take at most 2048 slots per query in the backward (the forward
        # takes 8192): say so here, not in the middle of loss.backward()
        topk = getattr(self.config, "dsa_indexer_topk", None)
        if topk is not None and int(topk) > 2048:
            raise ValueError("DSAttentionFused: dsa_indexer_topk=%d exceeds the 2048 slots per query the sparse "
                             "attention backward supports" % int(topk))
        self.sparse_attention = build_module(DSADotProductAttention, config=self.config,
                                             softmax_scale=self.softmax_scale)
        self.attn_sink = None
        _DSA_MIN_HEAD_DIM = 128  # head count the sparse attention kernel is tiled for
        self.num_attention_heads_padded = max(config.num_attention_heads, _DSA_MIN_HEAD_DIM)
        self.num_attention_heads = config.num_attention_heads

    def forward(self, query, key, value, attention_mask, x, qr, attn_mask_type: AttnMaskType = None,
                attention_bias=None, packed_seq_params: PackedSeqParams = None, index_share_carrier: object = None):
        """query ``[sq, b, h, 576]`` (or ``[t, h, 576]`` packed), key ``[skv, b, 576]`` -> ``[b, sq, h, 512]``
        (``[t, h, 512]`` packed), with the indexer loss attached in training mode."""
        sq = query.size(0)
        topk_holder = (
            get_dsa_index_share_topk_holder(packed_seq_params, index_share_carrier, self.skip_topk,
                                            self.layer_number, self.source_layer)
            if self.index_share
            else None
        )
        if self.skip_topk:
            if self.source_layer not in topk_holder:
                raise RuntimeError(
                    "DSA index-share skip layer "
                    f"(layer_number={self.layer_number}) needs top-k indices from source "
                    f"computing layer {self.source_layer}, but that layer did not run before it."
                )
            index_scores = None
            topk_indices = topk_holder[self.source_layer]
        else:
            x = x.detach()
            qr = qr.detach()
            index_scores, topk_indices = self.indexer(x, qr, packed_seq_params=packed_seq_params)
        if topk_holder is not None and not self.skip_topk:
            topk_holder[self.layer_number] = topk_indices

        chunk_query = query
        if self.num_attention_heads < self.num_attention_heads_padded:
            pad_size = self.num_attention_heads_padded - self.num_attention_heads
            chunk_query = F.pad(chunk_query, [0, 0, 0, pad_size])
        offset = self.pg_collection.tp.rank() * chunk_query.size(0)
        if getattr(self.config, "enable_chunkpipe", False):
            # the query chunk sits behind the earlier chunks of its sequence (dsa_fused.py:897-901)
            mb = (self.config.chunkpipe_forward_microbatch if self.config.chunkpipe_forward
                  else self.config.chunkpipe_backward_microbatch)
            offset += (mb % self.config.chunk_num_per_seq) * self.config.chunksize

        # The logits of the selected slots are needed for one thing only, the head-averaged attention
        # distribution the indexer is trained towards (dsa_fused.py:903-929 of the reference asks the
        # kernel for p_out [sq, n, topk] and reduces it with triton_attn_dist).  Here the attention call
        # returns that distribution itself, recomputed from q, kv and lse, and only when the loss will
        # be formed: no [sq, n, topk] tensor exists (4.3 GB at 8k tokens, 17 GB at 32k).
        need_loss = self.training and torch.is_grad_enabled() and not self.skip_topk
        res = self.sparse_attention(
            chunk_query,
            key,
            topk_indices.unsqueeze(0).int(),
            offset,
            attn_mask_type=attn_mask_type,
            packed_seq_params=packed_seq_params,
            attn_sink=self.attn_sink,
            return_attn_dist=self.num_attention_heads if need_loss else 0,
        )
        output, main_attn_probs = res if need_loss else (res, None)
        if self.num_attention_heads < self.num_attention_heads_padded:
            output = output[..., : self.num_attention_heads, :]

        if need_loss:
            indexer_loss_coeff = getattr(self.config, "dsa_indexer_loss_coeff", 0.0)
            main_attn_probs = main_attn_probs[:, : index_scores.shape[-1]]
            # softmax, F.kl_div(log(pred + 1e-10), target + 1e-10, "sum") and their backward in one kernel
            from . import ops
            loss = ops.indexer_kl_loss(index_scores, main_attn_probs, 1e-10)
            indexer_loss = indexer_loss_coeff * loss / sq
            if indexer_loss_coeff > 0:
                DSAIndexerLossLoggingHelperFused.save_loss_to_tracker(
                    loss=indexer_loss,
                    layer_number=self.layer_number,
                    num_layers=self.config.num_layers + getattr(self.config, "mtp_num_layers", 0),
                )
            output = DSAIndexerLossAutoScaler.apply(output, indexer_loss)
        return output
