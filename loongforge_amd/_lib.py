"""ctypes binding of libdsa_hip.so, the C-ABI library of gfx950 kernels.

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdsa_hip.so")

_c = ctypes
_vp, _i, _i64, _f, _sz = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float, _c.c_size_t

# name -> (restype, argtypes); mirrors include/dsa_hip.h
SIGNATURES = {
    "dsa_version": (_i, []),
    "dsa_last_error": (_c.c_char_p, []),
    "dsa_quant_rowwise_e4m3": (_i, [_vp, _i64, _i, _vp, _vp, _f, _i, _vp]),
    "dsa_rotate_quant_e4m3": (_i, [_vp, _i64, _i, _vp, _vp, _vp, _f, _i, _vp]),
    "dsa_quant_rowwise_e4m3_weights": (_i, [_vp, _i64, _i, _vp, _vp, _f, _i, _i, _vp, _f, _vp, _vp]),
    "dsa_indexer_front_e4m3": (_i, [_vp, _i64, _i, _i, _vp, _vp, _f, _vp, _vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp, _f, _i,
                                    _vp, _f, _vp, _vp]),
    "dsa_indexer_logits": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i64, _i, _i, _vp]),
    "dsa_topk": (_i, [_vp, _i, _i64, _vp, _vp, _i, _vp, _i, _i, _vp, _vp, _vp]),
    "dsa_indexer_topk_workspace_bytes": (_sz, [_i, _i, _i]),
    "dsa_indexer_topk_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _sz, _vp]),
    "dsa_indexer_topk_fwd_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dsa_indexer_bwd_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "dsa_indexer_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dsa_sparse_mla_fwd": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _i, _vp]),
    "dsa_sparse_mla_fwd_ex": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _i, _vp, _i, _vp]),
    "dsa_sparse_mla_bwd_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "dsa_sparse_mla_bwd_workspace_bytes_min": (_sz, [_i, _i, _i, _i]),
    "dsa_sparse_mla_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _sz, _vp]),
    "dsa_indexer_kl_loss": (_i, [_vp, _i64, _vp, _i64, _i, _i, _f, _vp, _vp, _vp]),
    "dsa_attn_dist": (_i, [_vp, _i, _i, _i, _i, _i64, _i64, _f, _vp, _vp]),
    "dsa_attn_dist_qk": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp, _vp]),
    "dsa_mla_absorb": (_i, [_vp, _i64, _i64, _vp, _vp, _i64, _i64, _i, _i, _i, _i, _vp]),
    "dsa_rope_rows": (_i, [_vp, _i64, _i64, _vp, _i64, _i64, _i, _vp, _i64, _i64, _vp, _i64, _i64, _i, _vp, _vp, _i, _vp,
                           _i, _i, _i, _i, _i, _i, _vp]),
    "dsa_rope_headsum_inverse": (_i, [_vp, _i64, _i64, _vp, _i64, _i, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp]),
}

# libdsa_bench.so: measurement aids for the benchmark (include/dsa_hip_bench.h), not part of the boundary
BENCH_LIB_PATH = os.path.join(_HERE, "libdsa_bench.so")
BENCH_SIGNATURES = {
    "dsa_last_error": (_c.c_char_p, []),
    "dsa_sparse_mla_bwd_profile": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _sz, _vp,
                                        _vp]),
    "dsa_probe_hbm_rows": (_i, [_vp, _vp, _i, _i, _i, _i, _vp]),
    "dsa_probe_hbm_read": (_i, [_vp, _sz, _vp, _vp]),
    "dsa_probe_mfma_bf16": (_i, [_i, _i, _vp, _vp, _vp]),
}

_lib = None
_lock = threading.Lock()


class DsaError(RuntimeError):
    """A kernel launch failed or the library rejected its arguments."""


def load():
    """Loads the shared library (once) and declares every entry point's signature."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise DsaError(
                "libdsa_hip.so is missing at %s; build it with `python -m loongforge_amd.csrc.build` "
                "(there is no fallback implementation)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)      # AttributeError if a declared symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = lib
        return _lib


def load_bench():
    """The benchmark-only library (its own copy of the backward with per-launch timing, and plain
    data movers / MFMA loops to quote the kernels against)."""
    if not os.path.exists(BENCH_LIB_PATH):
        raise DsaError("libdsa_bench.so is missing at %s; build it with `python -m loongforge_amd.csrc.build`"
                       % BENCH_LIB_PATH)
    lib = ctypes.CDLL(BENCH_LIB_PATH)
    for name, (res, args) in BENCH_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def check(rc, what, lib=None):
    """Turns a negative status into an exception carrying dsa_last_error() (of `lib`, default the kernels')."""
    if rc != 0:
        msg = (lib or load()).dsa_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError("%s: %s" % (what, msg))
        raise DsaError("%s failed (status %d): %s" % (what, rc, msg))
