"""Tensor-level entry points of the gfx950 DSA kernels.

Every function here checks its arguments, allocates outputs and workspaces with torch (the C
library allocates nothing), and calls libdsa_hip.so through ctypes on the current HIP stream.
The raw kernels are also registered as torch custom ops in the ``dsa::`` namespace so that they
can be used from compiled graphs and carry fake-tensor shape functions.

There is no CPU path and no fallback: tensors must live on a HIP device.
"""
import os
from typing import Optional, Tuple

import torch

from . import _lib

_FP8 = torch.float8_e4m3fn


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("DSA kernels need tensors on a HIP device; got a %s tensor" % t.device.type)


def _c(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


# --------------------------------------------------------------------------------------------
# quantiser
# --------------------------------------------------------------------------------------------
@torch.library.custom_op("dsa::quant_rowwise_e4m3", mutates_args=())
def _quant_op(x: torch.Tensor, eps: float, pow2: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    _need_gpu(x)
    if x.dtype != torch.bfloat16:
        raise ValueError("quant_rowwise_e4m3 expects bf16 input, got %s" % x.dtype)
    x = _c(x)
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    x8 = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scale_inv = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.dsa_quant_rowwise_e4m3(x.data_ptr(), rows, cols, x8.data_ptr(), scale_inv.data_ptr(),
                                              float(eps), int(pow2), _stream(x)), "dsa_quant_rowwise_e4m3")
    return x8, scale_inv


@_quant_op.register_fake
def _(x, eps, pow2):
    return x.new_empty(x.shape, dtype=torch.uint8), x.new_empty(x.shape[:-1], dtype=torch.float32)


def quant_rowwise_e4m3(x: torch.Tensor, eps: float = 1e-12, pow2: bool = True):
    """bf16 ``[..., 128]`` -> (float8_e4m3fn payload, fp32 ``scale_inv`` per row)."""
    x8, scale_inv = _quant_op(x, eps, pow2)
    return x8.view(_FP8), scale_inv


@torch.library.custom_op("dsa::rotate_quant_e4m3", mutates_args=())
def _rotate_quant_op(x: torch.Tensor, eps: float, pow2: bool, want_payload: bool,
                     want_rotated: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _need_gpu(x)
    if x.dtype != torch.bfloat16:
        raise ValueError("rotate_quant_e4m3 expects bf16 input, got %s" % x.dtype)
    if x.shape[-1] != 128:
        raise ValueError("rotate_quant_e4m3 rotates rows of 128 elements, got %d" % x.shape[-1])
    if not (want_payload or want_rotated):
        raise ValueError("rotate_quant_e4m3: no output requested")
    x = _c(x)
    rows = x.numel() // 128
    x8 = torch.empty(x.shape if want_payload else (0,), dtype=torch.uint8, device=x.device)
    scale_inv = torch.empty(x.shape[:-1] if want_payload else (0,), dtype=torch.float32, device=x.device)
    y = torch.empty(x.shape if want_rotated else (0,), dtype=torch.bfloat16, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.dsa_rotate_quant_e4m3(x.data_ptr(), rows, 128, x8.data_ptr() if want_payload else None,
                                             scale_inv.data_ptr() if want_payload else None,
                                             y.data_ptr() if want_rotated else None, float(eps), int(pow2), _stream(x)),
                   "dsa_rotate_quant_e4m3")
    return x8, scale_inv, y


@_rotate_quant_op.register_fake
def _(x, eps, pow2, want_payload, want_rotated):
    return (x.new_empty(x.shape if want_payload else (0,), dtype=torch.uint8),
            x.new_empty(x.shape[:-1] if want_payload else (0,), dtype=torch.float32),
            x.new_empty(x.shape if want_rotated else (0,), dtype=torch.bfloat16))


def rotate_quant_e4m3(x: torch.Tensor, eps: float = 1e-12, pow2: bool = True, return_rotated: bool = False):
    """Hadamard rotation (x 128^-0.5, rounded to bf16) fused with :func:`quant_rowwise_e4m3`:
    bf16 ``[..., 128]`` -> (fp8 payload, ``scale_inv``[, rotated bf16])."""
    x8, scale_inv, y = _rotate_quant_op(x, eps, pow2, True, return_rotated)
    return (x8.view(_FP8), scale_inv, y) if return_rotated else (x8.view(_FP8), scale_inv)


@torch.library.custom_op("dsa::indexer_front_e4m3", mutates_args=())
def _indexer_front_op(x: torch.Tensor, rows_per_token: int, ln_weight: Optional[torch.Tensor],
                      ln_bias: Optional[torch.Tensor], ln_eps: float, cos: Optional[torch.Tensor],
                      sin: Optional[torch.Tensor], pairing: int, positions: Optional[torch.Tensor], batch: int,
                      rotate: bool, weights: Optional[torch.Tensor], factor: float, want_payload: bool,
                      want_rows: bool, eps: float,
                      pow2: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    _need_gpu(x)
    if x.dtype != torch.bfloat16 or x.shape[-1] != 128:
        raise ValueError("indexer_front_e4m3 expects bf16 rows of 128 elements")
    x = _c(x)
    rows = x.numel() // 128
    if rows % rows_per_token:
        raise ValueError("indexer_front_e4m3: %d rows are not a multiple of %d rows per token" % (rows, rows_per_token))
    if (ln_weight is None) != (ln_bias is None):
        raise ValueError("indexer_front_e4m3: LayerNorm needs weight and bias")
    f32 = 0
    if pairing >= 0:
        if cos is None or sin is None or cos.dtype != sin.dtype or cos.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("indexer_front_e4m3: cos / sin must both be fp32 or bf16 tables")
        cos, sin = _c(cos.reshape(-1, cos.shape[-1])), _c(sin.reshape(-1, sin.shape[-1]))
        if cos.shape[-1] != 64 or sin.shape != cos.shape:
            raise ValueError("indexer_front_e4m3: cos / sin rows must have 64 entries")
        f32 = int(cos.dtype == torch.float32)
        if positions is not None:
            positions = _c(positions.to(torch.int32))
            if positions.numel() != rows // rows_per_token:
                raise ValueError("indexer_front_e4m3: one position per token expected")
        elif (rows // rows_per_token + batch - 1) // batch > cos.shape[0]:
            raise ValueError("indexer_front_e4m3: cos / sin tables are shorter than the sequence")
    if ln_weight is not None:
        ln_weight, ln_bias = _c(ln_weight.float()), _c(ln_bias.float())
        if ln_weight.numel() != 128 or ln_bias.numel() != 128:
            raise ValueError("indexer_front_e4m3: LayerNorm weight and bias must have 128 entries")
    if weights is not None:
        if not want_payload or weights.numel() != rows:
            raise ValueError("indexer_front_e4m3: one weight per row expected, together with the payload")
        weights = _c(weights.float())
    dev = x.device
    x8 = torch.empty(x.shape if want_payload else (0,), dtype=torch.uint8, device=dev)
    scale_inv = torch.empty(x.shape[:-1] if want_payload else (0,), dtype=torch.float32, device=dev)
    y = torch.empty(x.shape if want_rows else (0,), dtype=torch.bfloat16, device=dev)
    w_scaled = torch.empty(x.shape[:-1] if weights is not None else (0,), dtype=torch.float32, device=dev)
    ptr = lambda t: t.data_ptr() if t is not None and t.numel() else None   # noqa: E731
    lib = _lib.load()
    with torch.cuda.device(dev):
        _lib.check(lib.dsa_indexer_front_e4m3(
            x.data_ptr(), rows, 128, int(rows_per_token), ptr(ln_weight), ptr(ln_bias), float(ln_eps),
            ptr(cos) if pairing >= 0 else None, ptr(sin) if pairing >= 0 else None, f32, int(pairing), ptr(positions),
            int(batch), int(rotate), ptr(x8), ptr(scale_inv), ptr(y), float(eps), int(pow2), ptr(weights), float(factor),
            ptr(w_scaled), _stream(x)), "dsa_indexer_front_e4m3")
    return x8, scale_inv, y, w_scaled


@_indexer_front_op.register_fake
def _(x, rows_per_token, ln_weight, ln_bias, ln_eps, cos, sin, pairing, positions, batch, rotate, weights, factor,
      want_payload, want_rows, eps, pow2):
    return (x.new_empty(x.shape if want_payload else (0,), dtype=torch.uint8),
            x.new_empty(x.shape[:-1] if want_payload else (0,), dtype=torch.float32),
            x.new_empty(x.shape if want_rows else (0,), dtype=torch.bfloat16),
            x.new_empty(x.shape[:-1] if weights is not None else (0,), dtype=torch.float32))


def indexer_front_e4m3(x: torch.Tensor, rows_per_token: int = 1, ln_weight=None, ln_bias=None, ln_eps: float = 1e-5,
                       cos=None, sin=None, pairing: int = -1, positions=None, batch: int = 1, rotate: bool = True,
                       weights=None, factor: float = 1.0, return_payload: bool = True, return_rows: bool = False,
                       eps: float = 1e-12, pow2: bool = True):
    """The indexer front end behind its projections in one kernel: bf16 ``[..., 128]`` rows through
    [LayerNorm] -> [RoPE of the leading 64 elements, ``pairing`` ROPE_ADJACENT / ROPE_SPLIT, -1 none] ->
    [Hadamard rotation] -> quantiser.  Returns ``(x8, scale_inv, rows, weight_scaled)``; ``rows`` (the bf16
    values that were quantised) and ``weight_scaled`` (``weights * scale_inv * factor``) are ``None`` unless
    asked for."""
    x8, scale_inv, y, ws = _indexer_front_op(x, rows_per_token, ln_weight, ln_bias, ln_eps, cos, sin, pairing, positions,
                                             batch, rotate, weights, float(factor), return_payload, return_rows, eps, pow2)
    return (x8.view(_FP8) if return_payload else None, scale_inv if return_payload else None,
            y if return_rows else None, ws if weights is not None else None)


@torch.library.custom_op("dsa::quant_rowwise_e4m3_weights", mutates_args=())
def _quant_weights_op(x: torch.Tensor, weights: torch.Tensor, factor: float, rotate: bool, eps: float,
                      pow2: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _need_gpu(x, weights)
    if x.dtype != torch.bfloat16 or x.shape[-1] != 128:
        raise ValueError("quant_rowwise_e4m3_weights expects bf16 rows of 128 elements")
    if weights.shape != x.shape[:-1]:
        raise ValueError("quant_rowwise_e4m3_weights: one weight per row expected, got %s for rows %s"
                         % (tuple(weights.shape), tuple(x.shape[:-1])))
    x, weights = _c(x), _c(weights.float())
    rows = x.numel() // 128
    x8 = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scale_inv = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    w_scaled = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.dsa_quant_rowwise_e4m3_weights(x.data_ptr(), rows, 128, x8.data_ptr(), scale_inv.data_ptr(),
                                                      float(eps), int(pow2), int(rotate), weights.data_ptr(),
                                                      float(factor), w_scaled.data_ptr(), _stream(x)),
                   "dsa_quant_rowwise_e4m3_weights")
    return x8, scale_inv, w_scaled


@_quant_weights_op.register_fake
def _(x, weights, factor, rotate, eps, pow2):
    return (x.new_empty(x.shape, dtype=torch.uint8), x.new_empty(x.shape[:-1], dtype=torch.float32),
            x.new_empty(x.shape[:-1], dtype=torch.float32))


def quant_rowwise_e4m3_weights(x: torch.Tensor, weights: torch.Tensor, factor: float, rotate: bool = False,
                               eps: float = 1e-12, pow2: bool = True):
    """:func:`quant_rowwise_e4m3` (after the Hadamard rotation when ``rotate``) that also returns
    ``(weights * scale_inv) * factor`` per row: (fp8 payload, ``scale_inv``, scaled weights fp32)."""
    x8, scale_inv, w_scaled = _quant_weights_op(x, weights, float(factor), bool(rotate), eps, pow2)
    return x8.view(_FP8), scale_inv, w_scaled


def rotate_bf16(x: torch.Tensor):
    """Hadamard rotation of bf16 rows of 128 (x 128^-0.5), the kernel form of ``rotate_activation``."""
    return _rotate_quant_op(x, 1e-12, True, False, True)[2]


def _as_u8(t: torch.Tensor) -> torch.Tensor:
    if t.dtype == _FP8:
        return t.view(torch.uint8)
    if t.dtype != torch.uint8:
        raise ValueError("expected an fp8-e4m3 (or raw uint8) tensor, got %s" % t.dtype)
    return t


# --------------------------------------------------------------------------------------------
# indexer forward
# --------------------------------------------------------------------------------------------
def _check_indexer(q8, q_w, k8, k_scale, ks, ke):
    _need_gpu(q8, q_w, k8, k_scale, ks, ke)
    if q8.ndim != 3 or k8.ndim != 2 or q_w.ndim != 2:
        raise ValueError("indexer expects q8 [S,H,128], k8 [Sk,128], q_w [S,H]")
    S, Hi, D = q8.shape
    if D != 128 or k8.shape[1] != 128:
        raise ValueError("Only support dim with size 128.")
    if q_w.shape != (S, Hi) or k_scale.shape != (k8.shape[0],) or ks.shape != (S,) or ke.shape != (S,):
        raise ValueError("indexer: inconsistent shapes")
    return S, Hi, k8.shape[0]


@torch.library.custom_op("dsa::indexer_logits", mutates_args=())
def _indexer_logits_op(q8: torch.Tensor, q_w: torch.Tensor, k8: torch.Tensor, k_scale: torch.Tensor,
                       ks: torch.Tensor, ke: torch.Tensor, width: int, relative: bool) -> torch.Tensor:
    S, Hi, Sk = _check_indexer(q8, q_w, k8, k_scale, ks, ke)
    q8, k8 = _c(_as_u8(q8)), _c(_as_u8(k8))
    q_w, k_scale = _c(q_w.float()), _c(k_scale.float())
    ks, ke = _c(ks.int()), _c(ke.int())
    logits = torch.empty(S, width, dtype=torch.float32, device=q8.device)
    lib = _lib.load()
    with torch.cuda.device(q8.device):
        _lib.check(lib.dsa_indexer_logits(q8.data_ptr(), q_w.data_ptr(), k8.data_ptr(), k_scale.data_ptr(),
                                          ks.data_ptr(), ke.data_ptr(), S, Hi, Sk, logits.data_ptr(), width, width,
                                          int(relative), _stream(q8)), "dsa_indexer_logits")
    return logits


@_indexer_logits_op.register_fake
def _(q8, q_w, k8, k_scale, ks, ke, width, relative):
    return q_w.new_empty(q8.shape[0], width, dtype=torch.float32)


def indexer_logits(q8, q_w, k8, k_scale, ks, ke, width: Optional[int] = None, relative: bool = False):
    """Dense ``[S, width]`` fp32 logits, -inf outside ``[ks, ke)`` (column ``j - ks`` if relative)."""
    return _indexer_logits_op(q8, q_w, k8, k_scale, ks, ke, int(width if width is not None else k8.shape[0]),
                              bool(relative))


@torch.library.custom_op("dsa::topk", mutates_args=())
def _topk_op(logits: torch.Tensor, K: int, row_begin: Optional[torch.Tensor], row_end: Optional[torch.Tensor],
             id_base: Optional[torch.Tensor], sort: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    _need_gpu(logits, row_begin, row_end, id_base)
    if logits.ndim != 2 or logits.dtype != torch.float32:
        raise ValueError("topk expects a 2-D fp32 tensor")
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    S, width = logits.shape
    rb = _c(row_begin.int()) if row_begin is not None else None
    re = _c(row_end.int()) if row_end is not None else None
    ib = _c(id_base.int()) if id_base is not None else None
    scores = torch.empty(S, K, dtype=torch.float32, device=logits.device)
    ids = torch.empty(S, K, dtype=torch.int32, device=logits.device)
    lib = _lib.load()
    with torch.cuda.device(logits.device):
        _lib.check(lib.dsa_topk(logits.data_ptr(), S, logits.stride(0) if S > 0 else width,
                                rb.data_ptr() if rb is not None else None, re.data_ptr() if re is not None else None,
                                width, ib.data_ptr() if ib is not None else None, K, int(sort), scores.data_ptr(),
                                ids.data_ptr(), _stream(logits)), "dsa_topk")
    return scores, ids


@_topk_op.register_fake
def _(logits, K, row_begin, row_end, id_base, sort):
    return logits.new_empty(logits.shape[0], K), logits.new_empty(logits.shape[0], K, dtype=torch.int32)


def topk(logits, K: int, row_begin=None, row_end=None, id_base=None, sorted: bool = True):
    """Per-row top-K (scores, int32 ids); unused slots are (-inf, -1)."""
    return _topk_op(logits, int(K), row_begin, row_end, id_base, bool(sorted))


@torch.library.custom_op("dsa::indexer_topk", mutates_args=())
def _indexer_topk_op(q8: torch.Tensor, q_w: torch.Tensor, k8: torch.Tensor, k_scale: torch.Tensor, ks: torch.Tensor,
                     ke: torch.Tensor, K: int, sort: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    S, Hi, Sk = _check_indexer(q8, q_w, k8, k_scale, ks, ke)
    q8, k8 = _c(_as_u8(q8)), _c(_as_u8(k8))
    q_w, k_scale = _c(q_w.float()), _c(k_scale.float())
    ks, ke = _c(ks.int()), _c(ke.int())
    scores = torch.empty(S, K, dtype=torch.float32, device=q8.device)
    ids = torch.empty(S, K, dtype=torch.int32, device=q8.device)
    lib = _lib.load()
    nbytes = lib.dsa_indexer_topk_workspace_bytes(S, Sk, K)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=q8.device)
    with torch.cuda.device(q8.device):
        _lib.check(lib.dsa_indexer_topk_fwd(q8.data_ptr(), q_w.data_ptr(), k8.data_ptr(), k_scale.data_ptr(),
                                            ks.data_ptr(), ke.data_ptr(), S, Hi, Sk, K, int(sort), scores.data_ptr(),
                                            ids.data_ptr(), ws.data_ptr(), nbytes, _stream(q8)),
                   "dsa_indexer_topk_fwd")
    return scores, ids


@_indexer_topk_op.register_fake
def _(q8, q_w, k8, k_scale, ks, ke, K, sort):
    return q_w.new_empty(q8.shape[0], K, dtype=torch.float32), q_w.new_empty(q8.shape[0], K, dtype=torch.int32)


def indexer_topk(q8, q_w, k8, k_scale, ks, ke, K: int, sorted: bool = True):
    """Fused logits + top-K: (scores [S,K] fp32, global key ids [S,K] int32, -1 padded)."""
    return _indexer_topk_op(q8, q_w, k8, k_scale, ks, ke, int(K), bool(sorted))


@torch.library.custom_op("dsa::indexer_bwd", mutates_args=())
def _indexer_bwd_op(g: torch.Tensor, q8: torch.Tensor, k8: torch.Tensor, k_scale: torch.Tensor, q_w: torch.Tensor,
                    ids: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _need_gpu(g, q8, k8, k_scale, q_w, ids)
    S, Hi, D = q8.shape
    Sk = k8.shape[0]
    K = ids.shape[1]
    if g.shape != ids.shape or ids.shape[0] != S:
        raise ValueError("indexer_bwd: grad and ids must both be [S, K]")
    Kp = (K + 127) // 128 * 128
    g = g.float()
    ids = ids.int()
    if Kp != K:                       # slots are processed 128 at a time
        g = torch.nn.functional.pad(g, (0, Kp - K), value=0.0)
        ids = torch.nn.functional.pad(ids, (0, Kp - K), value=-1)
    g, ids = _c(g), _c(ids)
    q8, k8 = _c(_as_u8(q8)), _c(_as_u8(k8))
    q_w, k_scale = _c(q_w.float()), _c(k_scale.float())
    d_q8 = torch.empty(S, Hi, D, dtype=torch.float32, device=q8.device)
    d_k8 = torch.empty(Sk, D, dtype=torch.float32, device=q8.device)
    d_qw = torch.empty(S, Hi, dtype=torch.float32, device=q8.device)
    lib = _lib.load()
    nbytes = lib.dsa_indexer_bwd_workspace_bytes(S, Hi, Sk, Kp)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=q8.device)
    with torch.cuda.device(q8.device):
        _lib.check(lib.dsa_indexer_bwd(g.data_ptr(), q8.data_ptr(), k8.data_ptr(), k_scale.data_ptr(), q_w.data_ptr(),
                                       ids.data_ptr(), S, Hi, Sk, Kp, d_q8.data_ptr(), d_k8.data_ptr(), d_qw.data_ptr(),
                                       ws.data_ptr(), nbytes, _stream(q8)), "dsa_indexer_bwd")
    return d_q8, d_k8, d_qw


@_indexer_bwd_op.register_fake
def _(g, q8, k8, k_scale, q_w, ids):
    return (q_w.new_empty(q8.shape, dtype=torch.float32), q_w.new_empty(k8.shape, dtype=torch.float32),
            q_w.new_empty(q_w.shape, dtype=torch.float32))


def indexer_bwd(g, q8, k8, k_scale, q_w, ids):
    """Gradients of the selected logits w.r.t. the fp8 payloads and the scaled weights (fp32)."""
    return _indexer_bwd_op(g, q8, k8, k_scale, q_w, ids)


# --------------------------------------------------------------------------------------------
# sparse MLA
# --------------------------------------------------------------------------------------------
def _check_mla(q, kv, ids):
    _need_gpu(q, kv, ids)
    if q.ndim != 3 or kv.ndim != 2 or ids.ndim != 2:
        raise ValueError("sparse MLA expects q [S,H,576], kv [Skv,576], ids [S,K]")
    if q.dtype != torch.bfloat16 or kv.dtype != torch.bfloat16:
        raise ValueError("sparse MLA expects bf16 q and kv")
    if q.shape[-1] != 576 or kv.shape[-1] != 576:
        raise ValueError("you should assign dim otherwise: d_qk must be 576 (512 latent + 64 rope)")
    if ids.shape[0] != q.shape[0]:
        raise ValueError("ids and q disagree on the number of queries")
    if ids.shape[1] % 64 != 0:
        raise ValueError("top-k must be padded to a multiple of 64 (pad ids with -1)")


@torch.library.custom_op("dsa::sparse_mla_fwd", mutates_args=())
def _mla_fwd_op(q: torch.Tensor, kv: torch.Tensor, ids: torch.Tensor, q_start: int, sm_scale: float, d_v: int,
                p_out_mode: int, attn_sink: Optional[torch.Tensor] = None,
                p_out_skip: int = 0) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_mla(q, kv, ids)
    q, kv, ids = _c(q), _c(kv), _c(ids.int())
    S, H, _ = q.shape
    if attn_sink is not None:
        _need_gpu(attn_sink)
        if attn_sink.numel() != H:
            raise ValueError("attn_sink must hold one logit per head (%d), got %d" % (H, attn_sink.numel()))
        attn_sink = _c(attn_sink.float().reshape(H))
    K = ids.shape[1]
    out = torch.empty(S, H, d_v, dtype=torch.bfloat16, device=q.device)
    lse = torch.empty(S, H, dtype=torch.float32, device=q.device)
    if p_out_mode == 0:
        p_out = torch.empty(0, dtype=torch.bfloat16, device=q.device)
    else:
        if p_out_skip < 0 or p_out_skip >= K or p_out_skip % 32:
            raise ValueError("p_out_skip must be a multiple of 32 in [0, top-k), got %d" % p_out_skip)
        p_out = torch.empty(S, H, K - p_out_skip, dtype=torch.float32 if p_out_mode == 2 else torch.bfloat16,
                            device=q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        _lib.check(lib.dsa_sparse_mla_fwd_ex(q.data_ptr(), kv.data_ptr(), ids.data_ptr(), S, H, kv.shape[0], K,
                                             int(q_start), float(sm_scale), int(d_v), out.data_ptr(), lse.data_ptr(),
                                             p_out.data_ptr() if p_out_mode else None, int(p_out_mode == 2),
                                             attn_sink.data_ptr() if attn_sink is not None else None,
                                             int(p_out_skip), _stream(q)),
                   "dsa_sparse_mla_fwd")
    return out, lse, p_out


@_mla_fwd_op.register_fake
def _(q, kv, ids, q_start, sm_scale, d_v, p_out_mode, attn_sink=None, p_out_skip=0):
    S, H, _ = q.shape
    p = q.new_empty(0) if p_out_mode == 0 else q.new_empty(S, H, ids.shape[1] - p_out_skip, dtype=torch.float32 if p_out_mode == 2 else torch.bfloat16)
    return q.new_empty(S, H, d_v), q.new_empty(S, H, dtype=torch.float32), p


def sparse_mla_fwd(q, kv, ids, q_start: int = 0, sm_scale: Optional[float] = None, d_v: int = 512,
                   return_p_out: bool = False, p_out_dtype: torch.dtype = torch.bfloat16,
                   attn_sink: Optional[torch.Tensor] = None, p_out_skip: int = 0):
    """(out bf16 [S,H,d_v], natural-log lse fp32 [S,H], p_out or None).  ``attn_sink`` [H]: per-head
    sink logit added to the softmax denominator (and to lse).  ``p_out_skip``: p_out leaves out that
    many leading slots (a multiple of 32) and is [S,H,K - p_out_skip]."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    mode = 0 if not return_p_out else (2 if p_out_dtype == torch.float32 else 1)
    out, lse, p_out = _mla_fwd_op(q, kv, ids, int(q_start), float(sm_scale), int(d_v), mode, attn_sink,
                                   int(p_out_skip) if return_p_out else 0)
    return out, lse, (p_out if return_p_out else None)


@torch.library.custom_op("dsa::sparse_mla_fwd_dist", mutates_args=())
def _mla_fwd_dist_op(q: torch.Tensor, kv: torch.Tensor, ids: torch.Tensor, q_start: int, sm_scale: float, d_v: int,
                     dist_heads: int, block: int, attn_sink: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_mla(q, kv, ids)
    q, kv, ids = _c(q), _c(kv), _c(ids.int())
    S, H, _ = q.shape
    K = ids.shape[1]
    if attn_sink is not None:
        _need_gpu(attn_sink)
        attn_sink = _c(attn_sink.float().reshape(H))
    out = torch.empty(S, H, d_v, dtype=torch.bfloat16, device=q.device)
    lse = torch.empty(S, H, dtype=torch.float32, device=q.device)
    dist = torch.empty(S, K, dtype=torch.float32, device=q.device)
    block = max(1, min(int(block), S))
    p_out = torch.empty(block, H, K, dtype=torch.bfloat16, device=q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        st = _stream(q)
        for s0 in range(0, S, block):
            n = min(block, S - s0)
            _lib.check(lib.dsa_sparse_mla_fwd_ex(q[s0:].data_ptr(), kv.data_ptr(), ids[s0:].data_ptr(), n, H, kv.shape[0], K,
                                                 int(q_start) + s0, float(sm_scale), int(d_v), out[s0:].data_ptr(),
                                                 lse[s0:].data_ptr(), p_out.data_ptr(), 0,
                                                 attn_sink.data_ptr() if attn_sink is not None else None, 0, st),
                       "dsa_sparse_mla_fwd")
            _lib.check(lib.dsa_attn_dist(p_out.data_ptr(), 0, n, int(dist_heads), K, H * K, K, float(sm_scale),
                                         dist[s0:].data_ptr(), st), "dsa_attn_dist")
    return out, lse, dist


@_mla_fwd_dist_op.register_fake
def _(q, kv, ids, q_start, sm_scale, d_v, dist_heads, block, attn_sink=None):
    S, H, _ = q.shape
    return q.new_empty(S, H, d_v), q.new_empty(S, H, dtype=torch.float32), q.new_empty(S, ids.shape[1], dtype=torch.float32)


def sparse_mla_fwd_dist(q, kv, ids, q_start: int, sm_scale: float, d_v: int, dist_heads: int, block: int,
                        attn_sink: Optional[torch.Tensor] = None):
    """(out, lse, dist): the forward together with the head-averaged attention distribution over the first
    ``dist_heads`` heads (``attn_dist`` of the forward's raw logits), ``block`` queries at a time, so that the logits
    ``[block, H, K]`` are a passing buffer whatever the number of queries (a block's forward writes them, the
    reduction reads them back while they are still in the caches)."""
    return _mla_fwd_dist_op(q, kv, ids, int(q_start), float(sm_scale), int(d_v), int(dist_heads), int(block), attn_sink)


_BWD_WS = {}      # device index -> workspace kept between calls
BWD_MAX_SLOTS = 2048      # slots per query the backward kernels take in one call
ATTN_DIST_QK_MAX_SLOTS = 4096


def _bwd_workspace(full_bytes: int, device):
    """Workspace of the sparse-MLA backward: ``full_bytes`` lets it take all queries in one sweep (26 GiB at 8k
    tokens, top-k 2048; 105 GiB at 32k); given less, the library walks the queries in chunks.  The size handed to
    the library - and with it the chunking, on which the last bits of dKV depend - follows from the shapes and
    from ``DSA_BWD_WORKSPACE_GIB`` (default 48) alone, never from what happens to be free or from earlier calls.
    The buffer is kept per device and reused by later calls (held until :func:`release_bwd_workspace`; calls that
    overlap on one device - other streams - must not share it: set ``DSA_BWD_WORKSPACE_CACHE=0``).  Nothing is
    kept while a HIP graph is being captured."""
    want = max(int(full_bytes), 256)
    cap = os.environ.get("DSA_BWD_WORKSPACE_GIB", "48")
    want = min(want, max(int(float(cap) * 2 ** 30), 256))
    idx = device.index if device.index is not None else torch.cuda.current_device()
    kept = _BWD_WS.get(idx)
    if kept is not None and kept.numel() >= want:
        return kept, want
    _BWD_WS.pop(idx, None)
    del kept
    try:
        ws = torch.empty(want, dtype=torch.uint8, device=device)
    except torch.OutOfMemoryError as e:
        raise RuntimeError("sparse_mla_bwd: cannot allocate its %.1f GiB workspace; lower DSA_BWD_WORKSPACE_GIB "
                           "(the library then walks the queries in more chunks)" % (want / 2 ** 30)) from e
    if os.environ.get("DSA_BWD_WORKSPACE_CACHE", "1") != "0" and not torch.cuda.is_current_stream_capturing():
        _BWD_WS[idx] = ws
    return ws, want


def release_bwd_workspace(device=None):
    """Drops the backward workspace kept for ``device`` (all devices if None)."""
    if device is None:
        _BWD_WS.clear()
    else:
        d = torch.device(device)
        _BWD_WS.pop(d.index if d.index is not None else torch.cuda.current_device(), None)


@torch.library.custom_op("dsa::sparse_mla_bwd", mutates_args=())
def _mla_bwd_op(q: torch.Tensor, kv: torch.Tensor, out: torch.Tensor, dout: torch.Tensor, ids: torch.Tensor,
                lse: torch.Tensor, q_start: int, sm_scale: float, d_v: int) -> Tuple[torch.Tensor, torch.Tensor]:
    _check_mla(q, kv, ids)
    _need_gpu(out, dout, lse)
    q, kv, ids = _c(q), _c(kv), _c(ids.int())
    out, dout, lse = _c(out), _c(dout.to(torch.bfloat16)), _c(lse.float())
    S, H, _ = q.shape
    K = ids.shape[1]
    if out.shape != (S, H, d_v) or dout.shape != (S, H, d_v) or lse.shape != (S, H):
        raise ValueError("sparse_mla_bwd: out/dout must be [S,H,d_v] and lse [S,H]")
    dq = torch.empty_like(q)
    dkv = torch.empty_like(kv)
    lib = _lib.load()
    ws, nbytes = _bwd_workspace(lib.dsa_sparse_mla_bwd_workspace_bytes(S, H, kv.shape[0], K), q.device)
    with torch.cuda.device(q.device):
        _lib.check(lib.dsa_sparse_mla_bwd(q.data_ptr(), kv.data_ptr(), out.data_ptr(), dout.data_ptr(), ids.data_ptr(),
                                          lse.data_ptr(), S, H, kv.shape[0], K, int(q_start), float(sm_scale),
                                          int(d_v), dq.data_ptr(), dkv.data_ptr(), ws.data_ptr(), nbytes, _stream(q)),
                   "dsa_sparse_mla_bwd")
    return dq, dkv


@_mla_bwd_op.register_fake
def _(q, kv, out, dout, ids, lse, q_start, sm_scale, d_v):
    return torch.empty_like(q), torch.empty_like(kv)


def sparse_mla_bwd(q, kv, out, dout, ids, lse, q_start: int = 0, sm_scale: Optional[float] = None, d_v: int = 512):
    """(dq, dkv) in bf16; dkv is accumulated in a fixed order (bit-reproducible).

    The kernels take up to 2048 slots per query.  Longer lists are walked 2048 slots at a time: with the
    softmax statistics (``lse``) and ``out`` of the whole list given, the gradients are sums over the slots, so the
    parts add up (in fp32 here; an id that a query holds in two different parts is not detected)."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    K = ids.shape[1]
    if K <= BWD_MAX_SLOTS:
        return _mla_bwd_op(q, kv, out, dout, ids, lse, int(q_start), float(sm_scale), int(d_v))
    dq32 = dkv32 = None
    for k0 in range(0, K, BWD_MAX_SLOTS):
        part = ids[:, k0:k0 + BWD_MAX_SLOTS]
        if part.shape[1] % 64:
            part = torch.nn.functional.pad(part, (0, 64 - part.shape[1] % 64), value=-1)
        dq, dkv = _mla_bwd_op(q, kv, out, dout, part.contiguous(), lse, int(q_start), float(sm_scale), int(d_v))
        dq32 = dq.float() if dq32 is None else dq32.add_(dq)
        dkv32 = dkv.float() if dkv32 is None else dkv32.add_(dkv)
    return dq32.to(torch.bfloat16), dkv32.to(torch.bfloat16)


@torch.library.custom_op("dsa::attn_dist", mutates_args=())
def _attn_dist_op(p_out: torch.Tensor, sm_scale: float) -> torch.Tensor:
    _need_gpu(p_out)
    if p_out.ndim != 3 or p_out.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("attn_dist expects p_out [S,H,K] in bf16 or fp32")
    if p_out.stride(2) != 1:
        p_out = p_out.contiguous()
    S, H, K = p_out.shape
    target = torch.empty(S, K, dtype=torch.float32, device=p_out.device)
    lib = _lib.load()
    with torch.cuda.device(p_out.device):
        _lib.check(lib.dsa_attn_dist(p_out.data_ptr(), int(p_out.dtype == torch.float32), S, H, K,
                                     p_out.stride(0) if S > 0 else H * K, p_out.stride(1), float(sm_scale),
                                     target.data_ptr(), _stream(p_out)), "dsa_attn_dist")
    return target


@_attn_dist_op.register_fake
def _(p_out, sm_scale):
    return p_out.new_empty(p_out.shape[0], p_out.shape[2], dtype=torch.float32)


def attn_dist(p_out, sm_scale: float):
    """fp32 ``[S,K]``: mean over heads of softmax over slots of ``p_out * sm_scale``."""
    return _attn_dist_op(p_out, float(sm_scale))


@torch.library.custom_op("dsa::attn_dist_qk", mutates_args=())
def _attn_dist_qk_op(q: torch.Tensor, kv: torch.Tensor, ids: torch.Tensor, lse: torch.Tensor, q_start: int,
                     sm_scale: float, heads_in_mean: int) -> torch.Tensor:
    _need_gpu(q)
    if q.ndim != 3 or q.shape[-1] != 576 or q.dtype != torch.bfloat16:
        raise ValueError("attn_dist_qk expects q [S,H,576] in bf16")
    if kv.ndim != 2 or kv.shape[-1] != 576 or kv.dtype != torch.bfloat16:
        raise ValueError("attn_dist_qk expects kv [Skv,576] in bf16")
    S, H, _ = q.shape
    K = ids.shape[1]
    if ids.shape[0] != S or lse.shape != (S, H):
        raise ValueError("attn_dist_qk: ids [S,K] and lse [S,H] must match q")
    q, kv, ids, lse = _c(q), _c(kv), _c(ids.to(torch.int32)), _c(lse.float())
    target = torch.empty(S, K, dtype=torch.float32, device=q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        _lib.check(lib.dsa_attn_dist_qk(q.data_ptr(), kv.data_ptr(), ids.data_ptr(), lse.data_ptr(), S, H, int(heads_in_mean),
                                        kv.shape[0], K, int(q_start), float(sm_scale), target.data_ptr(), _stream(q)),
                   "dsa_attn_dist_qk")
    return target


@_attn_dist_qk_op.register_fake
def _(q, kv, ids, lse, q_start, sm_scale, heads_in_mean):
    return q.new_empty(q.shape[0], ids.shape[1], dtype=torch.float32)


def attn_dist_qk(q, kv, ids, lse, q_start: int, sm_scale: float, heads_in_mean: Optional[int] = None,
                 attn_sink: Optional[torch.Tensor] = None):
    """fp32 ``[S,K]``: the same distribution as ``attn_dist(p_out, sm_scale)`` - mean over the first
    ``heads_in_mean`` heads of the softmax over slots - recomputed from q, kv and the forward's
    natural-log ``lse`` instead of from materialised logits.  With an attention sink the forward's
    lse includes the sink term; the softmax over the slots alone has the log-sum-exp
    ``lse + log(1 - exp(sink - lse))``, which is what the kernel is given then."""
    if attn_sink is not None:
        lse = lse + torch.log1p(-torch.exp(attn_sink.to(lse.dtype).view(1, -1) - lse).clamp(max=1.0 - 1e-7))
    hm = int(heads_in_mean or q.shape[1])
    K = ids.shape[1]
    if K <= ATTN_DIST_QK_MAX_SLOTS:
        return _attn_dist_qk_op(q, kv, ids, lse, int(q_start), float(sm_scale), hm)
    # the kernel takes up to 4096 slots; with lse given every slot's value stands alone, so longer lists go in parts
    parts = []
    for k0 in range(0, K, ATTN_DIST_QK_MAX_SLOTS):
        part = ids[:, k0:k0 + ATTN_DIST_QK_MAX_SLOTS]
        n = part.shape[1]
        if n % 64:
            part = torch.nn.functional.pad(part, (0, 64 - n % 64), value=-1)
        parts.append(_attn_dist_qk_op(q, kv, part.contiguous(), lse, int(q_start), float(sm_scale), hm)[:, :n])
    return torch.cat(parts, dim=1)


# --------------------------------------------------------------------------------------------
# rotary position embedding fused with the surrounding copies
# --------------------------------------------------------------------------------------------
ROPE_ADJACENT, ROPE_SPLIT = 0, 1   # where pair i sits in a row: (2i, 2i+1) or (i, i + emb_dim/2)


@torch.library.custom_op("dsa::indexer_kl_loss", mutates_args=())
def _kl_loss_op(scores: torch.Tensor, target: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    _need_gpu(scores, target)
    if scores.ndim != 2 or target.shape != scores.shape:
        raise ValueError("indexer_kl_loss expects scores and target of one shape [S, K]")
    S, K = scores.shape
    scores = scores.float()
    target = target.float()
    if scores.stride(1) != 1:
        scores = scores.contiguous()
    if target.stride(1) != 1:
        target = target.contiguous()
    row_loss = torch.empty(S, dtype=torch.float32, device=scores.device)
    grad = torch.empty(S, K, dtype=torch.float32, device=scores.device)
    lib = _lib.load()
    with torch.cuda.device(scores.device):
        _lib.check(lib.dsa_indexer_kl_loss(scores.data_ptr(), scores.stride(0) if S > 1 else K, target.data_ptr(),
                                           target.stride(0) if S > 1 else K, S, K, float(eps), row_loss.data_ptr(),
                                           grad.data_ptr(), _stream(scores)), "dsa_indexer_kl_loss")
    return row_loss, grad


@_kl_loss_op.register_fake
def _(scores, target, eps):
    return scores.new_empty(scores.shape[0], dtype=torch.float32), scores.new_empty(scores.shape, dtype=torch.float32)


class _IndexerKLLoss(torch.autograd.Function):
    """The loss and its gradient come out of the same kernel; backward only scales what forward kept."""

    @staticmethod
    def forward(ctx, scores, target, eps):
        row_loss, grad = _kl_loss_op(scores.detach(), target.detach(), eps)
        ctx.save_for_backward(grad)
        ctx.in_dtype = scores.dtype
        return row_loss.sum()

    @staticmethod
    def backward(ctx, g):
        (grad,) = ctx.saved_tensors
        return (grad * g).to(ctx.in_dtype), None, None


def indexer_kl_loss(scores: torch.Tensor, target: torch.Tensor, eps: float = 1e-10) -> torch.Tensor:
    """``F.kl_div((softmax(scores, -1) + eps).log(), target + eps, reduction="sum")`` as one kernel
    (dsa_fused.py:931-937 of the reference); differentiable in ``scores``, the target is a constant."""
    return _IndexerKLLoss.apply(scores, target, float(eps))


def _rows_view(t: torch.Tensor, what: str):
    """(data_ptr, token stride, head stride) of a [tokens, heads, width] bf16 view with unit inner stride."""
    if t.dtype != torch.bfloat16 or t.ndim != 3 or (t.shape[-1] > 1 and t.stride(-1) != 1):
        raise ValueError("%s must be a bf16 [tokens, heads, width] view with unit inner stride" % what)
    return t.data_ptr(), t.stride(0), t.stride(1)


def _cos_sin(cos: torch.Tensor, sin: torch.Tensor, emb_dim: int):
    cos2, sin2 = cos.reshape(-1, emb_dim), sin.reshape(-1, emb_dim)
    if cos2.dtype not in (torch.float32, torch.bfloat16):
        cos2, sin2 = cos2.float(), sin2.float()
    if sin2.dtype != cos2.dtype:
        sin2 = sin2.to(cos2.dtype)
    return _c(cos2), _c(sin2)


def thd_positions(cu_seqlens: torch.Tensor, tokens: int, offset: int = 0) -> torch.Tensor:
    """Position of every packed token inside its own sequence (int32 [tokens]); token t of the call
    is global token t + offset.  Tokens past the last sequence get position 0."""
    cu = cu_seqlens.to(torch.int64)
    t = torch.arange(tokens, device=cu.device, dtype=torch.int64) + int(offset)
    seq = torch.searchsorted(cu[1:].contiguous(), t, right=True)
    inside = seq < cu.numel() - 1
    start = cu[seq.clamp(max=cu.numel() - 2)]
    return torch.where(inside, t - start, torch.zeros_like(t)).to(torch.int32)


def rope_rows(pe_src: Optional[torch.Tensor], pe_dst: Optional[torch.Tensor], cos: Optional[torch.Tensor],
              sin: Optional[torch.Tensor], in_pairing: int, out_pairing: int, inverse: bool = False,
              positions: Optional[torch.Tensor] = None, batch: int = 1,
              main_src: Optional[torch.Tensor] = None, main_dst: Optional[torch.Tensor] = None) -> None:
    """Rotates the pe part of every (token, head) row and copies the main part (either may be absent).

    All tensors are [tokens, heads, width] bf16 views (any token / head strides, rows starting on
    16-byte boundaries); ``pe_src`` may be ``pe_dst`` when both pairings are equal; a head stride of 0
    in ``pe_src`` broadcasts one row.  cos / sin: [positions, emb_dim] fp32 or bf16.  Writes in place
    into ``pe_dst`` / ``main_dst``.
    """
    ref = pe_dst if pe_dst is not None else main_dst
    _need_gpu(pe_src, pe_dst, cos, sin, positions, main_src, main_dst)
    tokens, heads = ref.shape[0], ref.shape[1]
    emb = 0
    ps = pd = (None, 0, 0)
    cos2 = sin2 = None
    if pe_dst is not None:
        emb = pe_dst.shape[-1]
        if pe_src.shape != pe_dst.shape:
            raise ValueError("pe_src and pe_dst differ in shape: %s vs %s" % (tuple(pe_src.shape), tuple(pe_dst.shape)))
        ps, pd = _rows_view(pe_src, "pe_src"), _rows_view(pe_dst, "pe_dst")
        cos2, sin2 = _cos_sin(cos, sin, emb)
        if positions is not None:
            positions = _c(positions.int())
            if positions.numel() != tokens:
                raise ValueError("positions must hold one entry per token")
    ms = md = (None, 0, 0)
    d_main = 0
    if main_dst is not None:
        if main_src.shape != main_dst.shape or main_dst.shape[:2] != ref.shape[:2]:
            raise ValueError("main_src / main_dst shapes do not match the pe rows")
        d_main = main_dst.shape[-1]
        ms, md = _rows_view(main_src, "main_src"), _rows_view(main_dst, "main_dst")
    lib = _lib.load()
    with torch.cuda.device(ref.device):
        _lib.check(lib.dsa_rope_rows(ms[0], ms[1], ms[2], md[0], md[1], md[2], d_main, ps[0], ps[1], ps[2], pd[0], pd[1], pd[2],
                                     emb, cos2.data_ptr() if emb else None, sin2.data_ptr() if emb else None,
                                     int(emb and cos2.dtype == torch.float32),
                                     positions.data_ptr() if (emb and positions is not None) else None, int(batch),
                                     tokens, heads, int(in_pairing), int(out_pairing), int(bool(inverse)), _stream(ref)),
                   "dsa_rope_rows")


def rope_headsum_inverse(grad_pe: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, in_pairing: int,
                         positions: Optional[torch.Tensor] = None, batch: int = 1) -> torch.Tensor:
    """d_emb [tokens, emb_dim] bf16 = inverse rotation of bf16(sum over heads of grad_pe [tokens, heads, emb_dim])."""
    _need_gpu(grad_pe, cos, sin, positions)
    g = _rows_view(grad_pe, "grad_pe")
    tokens, heads, emb = grad_pe.shape
    cos2, sin2 = _cos_sin(cos, sin, emb)
    if positions is not None:
        positions = _c(positions.int())
    d_emb = torch.empty(tokens, emb, dtype=torch.bfloat16, device=grad_pe.device)
    lib = _lib.load()
    with torch.cuda.device(grad_pe.device):
        _lib.check(lib.dsa_rope_headsum_inverse(g[0], g[1], g[2], d_emb.data_ptr(), emb, emb, cos2.data_ptr(), sin2.data_ptr(),
                                                int(cos2.dtype == torch.float32),
                                                positions.data_ptr() if positions is not None else None, int(batch),
                                                tokens, heads, int(in_pairing), _stream(grad_pe)),
                   "dsa_rope_headsum_inverse")
    return d_emb


# --------------------------------------------------------------------------------------------
# MLA weight absorption (per-head projections written in place)
# --------------------------------------------------------------------------------------------
def mla_absorb_into(a: torch.Tensor, w: torch.Tensor, c: torch.Tensor) -> None:
    """``c[s, h, :] = a[s, h, :] @ w[h].T`` for bf16 views ``a [S, H, k]``, ``c [S, H, n]`` (any token / head
    strides that are multiples of 8 elements, unit stride inside a row) and contiguous ``w [H, n, k]`` with
    ``(k, n)`` = (128, 512) or (512, 128).  Writes into ``c``; no autograd (see :class:`MlaAbsorb`)."""
    _need_gpu(a, w, c)
    if a.dtype != torch.bfloat16 or c.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("mla_absorb expects bf16 tensors")
    if a.ndim != 3 or c.ndim != 3 or w.ndim != 3 or a.shape[:2] != c.shape[:2] or w.shape != (a.shape[1], c.shape[2], a.shape[2]):
        raise ValueError("mla_absorb: shapes a %s, w %s, c %s do not fit c[s,h,:] = a[s,h,:] @ w[h].T"
                         % (tuple(a.shape), tuple(w.shape), tuple(c.shape)))
    if a.stride(2) != 1 or c.stride(2) != 1:
        raise ValueError("mla_absorb: rows must be contiguous")
    w = _c(w)
    S, H, k = a.shape
    lib = _lib.load()
    with torch.cuda.device(a.device):
        _lib.check(lib.dsa_mla_absorb(a.data_ptr(), a.stride(0), a.stride(1), w.data_ptr(), c.data_ptr(), c.stride(0),
                                      c.stride(1), S, H, k, c.shape[2], _stream(a)), "dsa_mla_absorb")


class MlaAbsorb(torch.autograd.Function):
    """``out[s, h, :] = a[s, h, :] @ w[h].T`` through the HIP kernel, written into ``out`` (a view of a larger
    tensor, returned as is and marked dirty), with the two gradient products as plain library GEMMs."""

    @staticmethod
    def forward(ctx, a, w, out):
        mla_absorb_into(a.detach(), w.detach(), out)
        ctx.save_for_backward(a, w)
        ctx.mark_dirty(out)
        return out

    @staticmethod
    def backward(ctx, grad):
        a, w = ctx.saved_tensors
        g = grad.transpose(0, 1)                       # [H, S, n]
        d_a = torch.bmm(g, w).transpose(0, 1) if ctx.needs_input_grad[0] else None          # [S, H, k]
        d_w = torch.bmm(g.transpose(1, 2), a.transpose(0, 1)) if ctx.needs_input_grad[1] else None   # [H, n, k]
        return d_a, d_w, None


def mla_absorb(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Differentiable per-head projection ``a [S, H, k] , w [H, n, k] -> [S, H, n]``; ``out`` may be a view into
    a larger tensor (for instance the latent columns of the attention query)."""
    if out is None:
        out = a.new_empty(a.shape[0], a.shape[1], w.shape[1])
    return MlaAbsorb.apply(a, w, out)
