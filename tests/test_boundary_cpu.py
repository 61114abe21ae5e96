"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the header
declares, the Python binding table matches the header, and the product path refuses to run
without a HIP device instead of falling back to anything."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dsa_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dsa_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for expected in ["dsa_quant_rowwise_e4m3", "dsa_indexer_logits", "dsa_topk", "dsa_indexer_topk_fwd",
                     "dsa_indexer_bwd", "dsa_sparse_mla_fwd", "dsa_sparse_mla_bwd", "dsa_attn_dist",
                     "dsa_last_error", "dsa_version"]:
        assert expected in names


def test_library_exports_every_declared_symbol():
    from loongforge_amd import _lib

    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), name
    assert set(_lib.SIGNATURES) == set(_declared_functions())
    loaded = _lib.load()
    assert loaded.dsa_version() >= 1
    assert loaded.dsa_last_error() == b""


def test_binding_arity_matches_header():
    from loongforge_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        args = m.group(1).strip()
        n = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        assert n == len(argtypes), (name, n, len(argtypes))


def test_no_cpu_fallback():
    from loongforge_amd import ops

    q = torch.zeros(4, 128, 576, dtype=torch.bfloat16)
    kv = torch.zeros(4, 576, dtype=torch.bfloat16)
    ids = torch.zeros(4, 64, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="HIP device"):
        ops.sparse_mla_fwd(q, kv, ids)
    with pytest.raises(RuntimeError, match="HIP device"):
        ops.quant_rowwise_e4m3(torch.zeros(2, 128, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="HIP device"):
        ops.attn_dist(torch.zeros(2, 4, 64), 0.1)


def test_product_code_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "loongforge_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(".py"):
                src = open(os.path.join(base, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle", src, flags=re.M), f
                assert "dsa_oracle" not in src, f


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from loongforge_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libdsa_hip.so"))
    with pytest.raises(_lib.DsaError, match="missing"):
        _lib.load()


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU; asked for more it says so and exits without touching a device."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert res.returncode != 0
    assert "one GPU" in (res.stdout + res.stderr)
