"""Single-process stand-ins for the Megatron-core names the reference's DSA modules import.

The reference builds its attention modules on Megatron-core (``MegatronModule``, ``ModuleSpec`` /
``build_module``, ``PackedSeqParams``, ``AttnMaskType``, rotary embeddings, the indexer-loss
auto-scaler).  That package is not part of this repository; when it is importable the real classes
are used, otherwise the minimal equivalents below (one process, tensor-parallel size 1) are.
Reference import sites: loongforge/models/common/experimental_attention_variant/dsa_fused.py:30-51.
"""
import enum
from dataclasses import dataclass, field
from typing import Optional, Union

import torch

try:  # pragma: no cover - exercised only where Megatron-core is installed
    from megatron.core.packed_seq_params import PackedSeqParams
    from megatron.core.transformer.enums import AttnMaskType
    from megatron.core.transformer.module import MegatronModule
    from megatron.core.transformer.spec_utils import ModuleSpec, build_module
    HAVE_MEGATRON = True
except Exception:  # noqa: BLE001
    HAVE_MEGATRON = False

    class AttnMaskType(enum.Enum):
        padding = 1
        causal = 2
        no_mask = 3
        padding_causal = 4
        arbitrary = 5

    @dataclass
    class PackedSeqParams:
        qkv_format: str = None
        cu_seqlens_q: torch.Tensor = None
        cu_seqlens_kv: torch.Tensor = None
        cu_seqlens_q_padded: torch.Tensor = None
        cu_seqlens_kv_padded: torch.Tensor = None
        max_seqlen_q: int = None
        max_seqlen_kv: int = None

    class MegatronModule(torch.nn.Module):
        def __init__(self, config=None):
            super().__init__()
            self.config = config

    @dataclass
    class ModuleSpec:
        module: Union[type, tuple]
        params: dict = field(default_factory=dict)
        submodules: object = None

    def build_module(spec_or_module, *args, **kwargs):
        """Instantiates a class or ModuleSpec (a ready module instance is returned as is)."""
        if isinstance(spec_or_module, torch.nn.Module):
            return spec_or_module
        if isinstance(spec_or_module, ModuleSpec):
            params = dict(spec_or_module.params)
            params.update(kwargs)
            if spec_or_module.submodules is not None:
                params["submodules"] = spec_or_module.submodules
            return spec_or_module.module(*args, **params)
        if isinstance(spec_or_module, type):
            return spec_or_module(*args, **kwargs)
        raise TypeError("cannot build a module from %r" % (spec_or_module,))


class _SingleRankGroup:
    def rank(self):
        return 0

    def size(self):
        return 1


class ProcessGroupCollection:
    """tp / cp / pp groups of a one-process job."""

    def __init__(self):
        self.tp = _SingleRankGroup()
        self.cp = _SingleRankGroup()
        self.pp = _SingleRankGroup()

    @classmethod
    def use_mpu_process_groups(cls, required_pgs=None):
        return cls()


class RotaryEmbedding(torch.nn.Module):
    """Plain RoPE frequencies: ``forward(seq_len, offset)`` -> angles ``[seq, 1, 1, dim]``."""

    def __init__(self, kv_channels, rotary_percent=1.0, rotary_base=10000, cp_group=None, **_):
        super().__init__()
        dim = int(kv_channels * rotary_percent)
        self.dim = dim
        inv_freq = 1.0 / (rotary_base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    def get_rotary_seq_len(self, inference_context, transformer, x, config, packed_seq_params):
        if packed_seq_params is not None and packed_seq_params.max_seqlen_kv is not None:
            return max(int(packed_seq_params.max_seqlen_kv), 1)
        return x.size(0)

    def forward(self, max_seq_len, offset=0, packed_seq=False):
        seq = torch.arange(max_seq_len, device=self.inv_freq.device, dtype=torch.float32) + offset
        freqs = torch.outer(seq, self.inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)
        return emb[:, None, None, :]


    def get_cached_cos_sin(self, max_seq_len, dtype=torch.float32, packed_seq=False):
        """``(cos, sin)`` of the angles, each ``[seq, 1, 1, dim]`` in ``dtype`` (what the fused rotary kernels take)."""
        emb = self.forward(max_seq_len, packed_seq=packed_seq)
        return emb.cos().to(dtype).contiguous(), emb.sin().to(dtype).contiguous()


def _rotate_half(x, interleaved):
    if not interleaved:
        x1, x2 = torch.chunk(x, 2, dim=-1)
        return torch.cat((-x2, x1), dim=-1)
    x1, x2 = x[..., 0::2], x[..., 1::2]
    return torch.stack((-x2, x1), dim=-1).flatten(-2)


def apply_rotary_pos_emb(t, freqs, config=None, cu_seqlens=None, mscale=1.0, cp_group=None, offsets=None):
    """RoPE on ``t [s, (b,) h, d]`` with angles ``freqs [s_max, 1, 1, d]``.  With ``cu_seqlens`` the
    positions restart at every document (packed layout ``[t, h, d]``).  When
    ``config.multi_latent_attention`` is set the input is de-interleaved first, as Megatron does."""
    interleaved_in = bool(getattr(config, "multi_latent_attention", False))
    if interleaved_in:
        t = torch.cat((t[..., 0::2], t[..., 1::2]), dim=-1)
    if cu_seqlens is None:
        f = freqs[: t.shape[0]]
        while f.ndim < t.ndim:
            f = f.unsqueeze(1)
        f = f.reshape(f.shape[0], *([1] * (t.ndim - 2)), f.shape[-1])
    else:
        cu = cu_seqlens.to(torch.int64)
        lens = cu[1:] - cu[:-1]
        pos = torch.cat([torch.arange(int(n), device=t.device) for n in lens.tolist()])
        if pos.numel() < t.shape[0]:
            pos = torch.cat([pos, torch.arange(t.shape[0] - pos.numel(), device=t.device)])
        f = freqs[pos.to(freqs.device)]
        f = f.reshape(f.shape[0], *([1] * (t.ndim - 2)), f.shape[-1])
    cos, sin = (torch.cos(f) * mscale).to(t.dtype), (torch.sin(f) * mscale).to(t.dtype)
    return t * cos + _rotate_half(t, False) * sin


class DSAIndexerLossAutoScaler(torch.autograd.Function):
    """Attaches an auxiliary loss to an activation: forward returns the activation unchanged,
    backward feeds ``main_loss_backward_scale`` as the gradient of the loss (Megatron's auxiliary
    loss convention, used at dsa_fused.py:956)."""

    main_loss_backward_scale: torch.Tensor = None

    @staticmethod
    def forward(ctx, output, indexer_loss):
        ctx.save_for_backward(indexer_loss)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        (indexer_loss,) = ctx.saved_tensors
        scale = DSAIndexerLossAutoScaler.main_loss_backward_scale
        if scale is None:
            scale = torch.tensor(1.0, device=indexer_loss.device)
        return grad_output, torch.ones_like(indexer_loss) * scale.to(indexer_loss.device)

    @staticmethod
    def set_loss_scale(scale):
        DSAIndexerLossAutoScaler.main_loss_backward_scale = scale


class DSAIndexerLossLoggingHelper:
    """Keeps the last indexer loss per layer (dsa_fused.py:948-953)."""

    tracker = {}

    @staticmethod
    def save_loss_to_tracker(loss, layer_number, num_layers, **_):
        DSAIndexerLossLoggingHelper.tracker[layer_number] = loss.detach()


def get_dsa_index_share_topk_holder(packed_seq_params, index_share_carrier, skip_topk, layer_number, source_layer):
    """Per-forward dict layer -> top-k ids used for cross-layer index sharing."""
    if index_share_carrier is None:
        raise RuntimeError("index sharing needs an index_share_carrier object to hold the top-k ids")
    holder = getattr(index_share_carrier, "dsa_topk_holder", None)
    if holder is None:
        holder = {}
        setattr(index_share_carrier, "dsa_topk_holder", holder)
    return holder


def is_dsa_skip_topk_layer(layer_number, skip_offset, topk_freq):
    """Layers ``skip_offset + 1 + k * topk_freq`` compute the top-k; the others reuse it."""
    return topk_freq > 1 and (layer_number - 1 - skip_offset) % topk_freq != 0 and layer_number - 1 >= skip_offset


def source_dsa_compute_layer(layer_number, skip_offset, topk_freq):
    rel = layer_number - 1 - skip_offset
    return layer_number - (rel % topk_freq)


_ARGS = None


def get_args():
    """Global training arguments, if a trainer registered any (None otherwise)."""
    return _ARGS


def set_args(args):
    global _ARGS
    _ARGS = args
