"""On-disk names of the indexer weights in the two checkpoint layouts the reference converts between.

The reference's converter maps, per transformer layer, the Hugging Face names
``model.layers.<n>.self_attn.indexer.{wq_b, wk, k_norm, weights_proj}`` to the Megatron-core names
``decoder.layers.<n>.self_attention.core_attention.indexer.{linear_wq_b, linear_wk, k_norm,
linear_weights_proj}`` (configs/models/deepseek3/ckpt_convert/deepseek_v3_2_convert.yaml:40-43 and
:99-112, common names at tools/convert_checkpoint/common/common_checkpoint.py:35-38).  This module
holds that table and renames the entries of a state dict in either direction; it touches no tensor
data.  Only the indexer entries are handled: everything else in a checkpoint is outside this path.
"""
import re
from typing import Dict

# common name (converter) -> (Hugging Face suffix, Megatron-core suffix)
INDEXER_WEIGHT_NAMES = {
    "attention.indexer.wq_b": ("self_attn.indexer.wq_b", "self_attention.core_attention.indexer.linear_wq_b"),
    "attention.indexer.wk": ("self_attn.indexer.wk", "self_attention.core_attention.indexer.linear_wk"),
    "attention.indexer.k_norm": ("self_attn.indexer.k_norm", "self_attention.core_attention.indexer.k_norm"),
    "attention.indexer.weights_proj": ("self_attn.indexer.weights_proj",
                                       "self_attention.core_attention.indexer.linear_weights_proj"),
}
HF_LAYER_PREFIX = "model.layers."
MCORE_LAYER_PREFIX = "decoder.layers."

_HF = {hf: mc for hf, mc in INDEXER_WEIGHT_NAMES.values()}
_MC = {mc: hf for hf, mc in INDEXER_WEIGHT_NAMES.values()}


def _rename(key: str, src_prefix: str, dst_prefix: str, table: Dict[str, str]):
    m = re.match(re.escape(src_prefix) + r"(\d+)\.(.+)\.(weight|bias)$", key)
    if not m or m.group(2) not in table:
        return None
    return "%s%s.%s.%s" % (dst_prefix, m.group(1), table[m.group(2)], m.group(3))


def hf_to_mcore_key(key: str):
    """Megatron-core name of a Hugging Face indexer entry, or None when the key is not one."""
    return _rename(key, HF_LAYER_PREFIX, MCORE_LAYER_PREFIX, _HF)


def mcore_to_hf_key(key: str):
    """Hugging Face name of a Megatron-core indexer entry, or None when the key is not one."""
    return _rename(key, MCORE_LAYER_PREFIX, HF_LAYER_PREFIX, _MC)


def rename_indexer_entries(state_dict: Dict[str, object], to: str) -> Dict[str, object]:
    """Copy of ``state_dict`` with its indexer entries renamed ``to`` "mcore" or "hf"; other entries are kept."""
    if to not in ("mcore", "hf"):
        raise ValueError("to must be 'mcore' or 'hf'")
    fn = hf_to_mcore_key if to == "mcore" else mcore_to_hf_key
    out = {}
    for k, v in state_dict.items():
        nk = fn(k)
        out[nk if nk is not None else k] = v
    return out


def indexer_module_state(state_dict: Dict[str, object], layer: int) -> Dict[str, object]:
    """Entries of one layer's indexer from a Megatron-core state dict, keyed as the indexer module
    (``DSAIndexerFused``) names its own parameters: ``linear_wq_b.weight``, ``k_norm.bias``, ..."""
    prefix = "%s%d.self_attention.core_attention.indexer." % (MCORE_LAYER_PREFIX, layer)
    return {k[len(prefix):]: v for k, v in state_dict.items() if k.startswith(prefix)}
