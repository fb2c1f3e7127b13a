"""ctypes binding of libodysseus_hip.so (the C ABI declared in include/odysseus_hip.h).

The library is the only compute path of this package: if it cannot be loaded the
import of any op raises, there is no fallback.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libodysseus_hip.so"

ODY_BF16, ODY_F32 = 0, 1
GEMM_NT, GEMM_NN, GEMM_TN = 0, 1, 2
BWD_ACCUMULATE_DQ, BWD_DQ_F32, BWD_REUSE_QUERY_SIDE, BWD_KEEP_DS = 1, 2, 4, 8
ATTN_FWD_NOALLOC_SCRATCH_BYTES = (32 << 20) + (64 << 10)

_i, _i64, _u64, _f, _p, _sz = C.c_int, C.c_int64, C.c_uint64, C.c_float, C.c_void_p, C.c_size_t

# name -> (restype, argtypes); mirrors include/odysseus_hip.h one to one
SIGNATURES = {
    "ody_last_error": (C.c_char_p, []),
    "ody_version": (_i, []),
    "ody_device_info": (_i, [_p, _p, _p]),
    "ody_profile_enable": (_i, [_i]),
    "ody_profile_collect": (_i, [C.c_char_p, _sz]),
    "ody_attn_fwd_workspace_bytes": (_sz, [_i] * 7),
    "ody_attn_fwd": (_i, [_p] * 5 + [_i] * 6 + [_i64] * 12 + [_f, _i, _i, _p, _sz, _p]),
    "ody_attn_fwd_noalloc": (_i, [_p] * 5 + [_i] * 6 + [_i64] * 12 + [_f, _i, _i, _p]),
    "ody_attn_bwd_workspace_bytes": (_sz, [_i] * 7),
    "ody_attn_bwd_ds_bytes": (_sz, [_i] * 8),
    "ody_attn_bwd": (_i, [_p] * 9 + [_i] * 6 + [_i64] * 24 + [_f, _i, _i, _i, _p, _sz, _p]),
    "ody_cast_from_f32": (_i, [_p, _p, _i64, _i, _p]),
    "ody_lse_merge": (_i, [_p] * 4 + [_i] * 4 + [_i64] * 3 + [_i, _p]),
    "ody_gemm_workspace_bytes": (_sz, [_i] * 5),
    "ody_gemm": (_i, [_i] + [_p] * 4 + [_i] * 3 + [_i64] * 3 + [_i, _i, _p, _sz, _p]),
    "ody_linear_residual": (_i, [_p] * 4 + [_i] * 3 + [_i64] * 4 + [_i, _p]),
    "ody_linear_swiglu": (_i, [_p] * 4 + [_i] * 3 + [_i64] * 4 + [_i, _p]),
    "ody_linear_dgrad_swiglu_workspace_bytes": (_sz, [_i] * 4),
    "ody_linear_dgrad_swiglu": (_i, [_p] * 4 + [_i] * 3 + [_i64] * 4 + [_i, _p, _sz, _p]),
    "ody_swiglu_fwd": (_i, [_p, _p, _i, _i, _i64, _i64, _i, _p]),
    "ody_swiglu_bwd": (_i, [_p, _p, _p, _i, _i, _i64, _i64, _i64, _i, _p]),
    "ody_rmsnorm_fwd": (_i, [_p] * 4 + [_i, _i, _f, _i, _p]),
    "ody_rmsnorm_bwd_partials": (_i, [_i]),
    "ody_rmsnorm_bwd": (_i, [_p] * 8 + [_i, _i, _i, _p]),
    "ody_cross_entropy_fwd": (_i, [_p] * 5 + [_i, _i, _i64, _i64, _i, _p]),
    "ody_cross_entropy_bwd": (_i, [_p] * 6 + [_i, _i, _i64, _i64, _i, _p]),
    "ody_rope": (_i, [_p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i64, _f, _i, _i, _p]),
    "ody_rope_table": (_i, [_p, _p, _i64, _i, _f, _p, _p]),
    "ody_adamw": (_i, [_p, _p, _p, _p, _i64, _f, _f, _f, _f, _f, _i64, _i, _p]),
    "ody_linear_rope": (_i, [_p] * 4 + [_i] * 5 + [_i64] * 4 + [_i, _p]),
    "ody_attn_bwd_rope": (_i, [_p] * 9 + [_i] * 6 + [_i64] * 24 + [_f, _i, _i, _i, _p, _sz, _p, _p, _p]),
    "ody_attn_fwd_dropout": (_i, [_p] * 5 + [_i] * 6 + [_i64] * 12 + [_f, _i, _i, _p, _sz, _p, _f, _u64]),
    "ody_attn_bwd_dropout": (_i, [_p] * 9 + [_i] * 6 + [_i64] * 24 + [_f, _i, _i, _i, _p, _sz, _p, _f, _u64]),
}

_lib = None


class OdysseusHipError(RuntimeError):
    """A C-ABI entry point returned a negative status."""

    def __init__(self, fn: str, code: int, msg: str):
        super().__init__(f"{fn} failed with status {code}: {msg}")
        self.fn, self.code, self.msg = fn, code, msg


def load() -> C.CDLL:
    """Loads the library once and declares every prototype.  Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    path = Path(os.environ.get("ODYSSEUS_HIP_LIB", LIB_PATH))
    if not path.exists():
        raise ImportError(
            f"{path} not found: build it with `python -m odysseus_transformer_amd.build` "
            "(hipcc, gfx950).  There is no fallback compute path.")
    lib = C.CDLL(str(path))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library out of sync
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    """Calls an int-returning entry point and raises OdysseusHipError on failure."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise OdysseusHipError(name, rc, lib.ody_last_error().decode("utf-8", "replace"))


def device_info() -> dict:
    """Compute units, engine clock (kHz) and LDS bytes per compute unit of the current device."""
    cu, khz, lds = C.c_int(0), C.c_int(0), C.c_int(0)
    call("ody_device_info", C.addressof(cu), C.addressof(khz), C.addressof(lds))
    return {"compute_units": cu.value, "clock_khz": khz.value, "lds_bytes_per_cu": lds.value}


def profile_enable(on: bool) -> None:
    call("ody_profile_enable", int(on))


def profile_collect() -> dict:
    """{kernel name: (launches, total_ms, min_ms)} of the launches since the last collect."""
    buf = C.create_string_buffer(1 << 16)
    call("ody_profile_collect", buf, len(buf))
    out = {}
    for line in buf.value.decode().splitlines():
        name, n, total, mn = line.split()
        out[name] = (int(n), float(total), float(mn))
    return out
