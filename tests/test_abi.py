"""The C-ABI library loads and exports every symbol the header declares (CPU: no
compute calls), and argument validation answers with error codes, not crashes."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "odysseus_hip.h"


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(ody_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    from odysseus_transformer_amd import _lib
    if not _lib.LIB_PATH.exists():
        from odysseus_transformer_amd import build
        build.build(verbose=False)
    names = _declared()
    assert len(names) >= 15
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes table and header disagree"
    assert _lib.load().ody_version() >= 1


def test_validation_returns_codes_without_a_gpu():
    from odysseus_transformer_amd import _lib
    lib = _lib.load()
    # bad shapes / NULL pointers are rejected before anything touches the device
    with pytest.raises(_lib.OdysseusHipError) as e:
        _lib.call("ody_gemm", 0, 0, 0, 0, 0, 8, 8, 8, 8, 8, 8, 0, 0, 0, 0, 0)
    assert e.value.code == -4 and "NULL" in e.value.msg
    with pytest.raises(_lib.OdysseusHipError) as e:
        _lib.call("ody_attn_fwd", 16, 16, 16, 16, 16, 1, 8, 8, 3, 2, 128, *([128] * 12), 1.0, 1, 0, 0, 0, 0)
    assert e.value.code == -1 and "multiple" in e.value.msg
    with pytest.raises(_lib.OdysseusHipError) as e:
        _lib.call("ody_attn_fwd", 16, 16, 16, 16, 16, 1, 8, 8, 2, 2, 96, *([128] * 12), 1.0, 1, 0, 0, 0, 0)
    assert e.value.code == -2
    with pytest.raises(_lib.OdysseusHipError) as e:     # fp32 row stride of 130 elements: rows not 16-byte aligned
        _lib.call("ody_attn_fwd", 16, 16, 16, 16, 16, 1, 8, 8, 2, 2, 128, 128, 130, *([128] * 10), 1.0, 1, 1, 0, 0, 0)
    assert e.value.code == -3
    with pytest.raises(_lib.OdysseusHipError) as e:
        _lib.call("ody_rmsnorm_fwd", 16, 16, 16, 0, 4, 7, 1e-6, 0, 0)
    assert e.value.code == -2
    assert lib.ody_attn_bwd_workspace_bytes(1, 1000, 1000, 4, 4, 64, 0) == 16128
    assert lib.ody_rmsnorm_bwd_partials(100) == 100 and lib.ody_rmsnorm_bwd_partials(100000) == 256


def test_product_package_never_imports_the_oracle():
    pkg = ROOT / "odysseus_transformer_amd"
    for f in pkg.rglob("*.py"):
        assert "oracle" not in f.read_text(), f"{f} mentions the oracle"


def test_missing_library_fails_loudly(tmp_path):
    """No fallback: with the shared library absent every kernel call raises (checked in a fresh
    interpreter so that the handle this process has already loaded plays no part)."""
    import subprocess
    import sys
    code = (
        "import sys, torch\n"
        f"sys.path.insert(0, {str(ROOT)!r})\n"
        "from odysseus_transformer_amd import ops, _lib\n"
        "try:\n"
        "    _lib.load()\n"
        "except ImportError as e:\n"
        "    print('LOAD', type(e).__name__)\n"
        "try:\n"
        "    ops.gemm(ops.GEMM_NT, torch.zeros(8, 8), torch.zeros(8, 8))\n"
        "except Exception as e:\n"
        "    print('OP', type(e).__name__)\n"
    )
    env = dict(**__import__("os").environ, ODYSSEUS_HIP_LIB=str(tmp_path / "absent.so"))
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120).stdout
    assert "LOAD ImportError" in out
    assert "OP " in out and "OP None" not in out
