"""Tensor-level wrappers of the C ABI (torch supplies device memory and the
stream, nothing else) and the autograd functions built from them.

Every function requires CUDA(HIP) tensors and raises otherwise: the HIP library
is the only compute path.
"""
from __future__ import annotations

import math
import os
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import GEMM_NN, GEMM_NT, GEMM_TN


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.ODY_BF16
    if t.dtype == torch.float32:
        return _lib.ODY_F32
    raise TypeError(f"odysseus_transformer_amd supports bfloat16 and float32 tensors, got {t.dtype}")


def _need_gpu(*ts: torch.Tensor) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "odysseus_transformer_amd ops run only on a HIP device (tensor is on "
                f"{t.device}); there is no CPU implementation in this package")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def scratch(nbytes: int, name: str, device) -> torch.Tensor:
    """Kernel scratch of `nbytes` bytes.  When the process-wide arena is set up for this device
    (utils.globals._set_global_memory_buffer, as the reference's train.py:62 does), the bytes come
    from its grow-only buffer `name` -- the use the reference makes of it for its gathered
    activations and weights (utils/linear_tpsp.py:159-165, utils/linear_zero3.py:38-40) -- so that
    steady-state steps allocate no scratch at all.  Buffers of one name alias each other: the
    kernels of one stream run in order, which is what makes the reuse safe; work on several
    streams at once needs the arena off.  Without an arena: a fresh torch allocation."""
    from .utils import globals as _globals
    arena = _globals._Arena.instance
    if arena is not None and nbytes > 0:
        adev = torch.device(arena.dev)
        if adev.type == device.type and (adev.index is None or adev.index == device.index):
            return arena.get_tensor((nbytes,), torch.uint8, name)
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def _same(ref: torch.Tensor, ref_name: str, **others: torch.Tensor) -> None:
    """Every tensor has the dtype, device and shape of `ref` (the kernels read raw pointers)."""
    for name, t in others.items():
        if t.dtype != ref.dtype or t.device != ref.device or t.shape != ref.shape:
            raise ValueError(f"{name} must match {ref_name} ({tuple(ref.shape)}, {ref.dtype}, {ref.device}); "
                             f"got {tuple(t.shape)}, {t.dtype}, {t.device}")


def _blhd(t: torch.Tensor, name: str) -> Tuple[int, int, int]:
    if t.dim() != 4:
        raise ValueError(f"{name} must be (B, L, H, D), got {tuple(t.shape)}")
    if t.stride(3) != 1:
        raise ValueError(f"{name}: head_dim must be contiguous (stride {t.stride()})")
    return t.stride(0), t.stride(1), t.stride(2)


# --------------------------------------------------------------------------- attention
def _check_dropout(dropout_p: float, seed) -> None:
    if not 0.0 <= dropout_p < 1.0:
        raise ValueError(f"dropout_p must be in [0, 1), got {dropout_p}")
    if dropout_p > 0.0 and seed is None:
        raise ValueError("attention dropout needs a seed: the backward reproduces the forward's mask from it")


def attn_fwd(q, k, v, causal: bool = True, scale: Optional[float] = None, out=None, dropout_p: float = 0.0, seed=None):
    """q (B, Lq, Hq, D), k/v (B, Lk, Hkv, D) -> out (B, Lq, Hq, D), lse (B, Hq, Lq) fp32.

    dropout_p > 0 drops entries of the softmax matrix before P . V, scaling the kept ones by
    1 / (1 - dropout_p); which entries is a fixed function of `seed` (an int) and the entry's (batch, head,
    query, key), so attn_bwd with the same dropout_p and seed sees the same mask.  lse is that of the full P."""
    _need_gpu(q, k, v)
    _check_dropout(dropout_p, seed)
    B, Lq, Hq, D = q.shape
    Lk, Hkv = k.shape[1], k.shape[2]
    if k.shape != v.shape or k.shape[0] != B or k.shape[3] != D or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError(f"k {tuple(k.shape)} {k.dtype} / v {tuple(v.shape)} {v.dtype} do not match "
                         f"q {tuple(q.shape)} {q.dtype}")
    if out is None:
        out = torch.empty((B, Lq, Hq, D), dtype=q.dtype, device=q.device)
    _same(q, "q", out=out)
    lse = torch.empty((B, Hq, Lq), dtype=torch.float32, device=q.device)
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    ws_bytes = _lib.load().ody_attn_fwd_workspace_bytes(B, Lq, Lk, Hq, Hkv, D, _dt(q))
    ws = scratch(ws_bytes, "attn_fwd_workspace", q.device) if ws_bytes else None
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            B, Lq, Lk, Hq, Hkv, D, *_blhd(q, "q"), *_blhd(k, "k"), *_blhd(v, "v"), *_blhd(out, "out"),
            scale, int(causal), _dt(q), ws.data_ptr() if ws_bytes else 0, ws_bytes, _stream())
    if dropout_p > 0.0:
        _lib.call("ody_attn_fwd_dropout", *args, float(dropout_p), int(seed) & 0xFFFFFFFFFFFFFFFF)
    else:
        _lib.call("ody_attn_fwd", *args)
    return out, lse


def attn_fwd_noalloc(q, k, v, out, lse, causal: bool = True, scale: Optional[float] = None) -> None:
    """attn_fwd into caller-owned `out` (B, Lq, Hq, D) and `lse` (B, Hq, Lq) fp32 without allocating
    anything: the kernel's scratch is a buffer the library holds on the device.  Shapes beyond that
    buffer (_lib.ATTN_FWD_NOALLOC_SCRATCH_BYTES) raise; calls that overlap on one device race."""
    _need_gpu(q, k, v, out, lse)
    B, Lq, Hq, D = q.shape
    Lk, Hkv = k.shape[1], k.shape[2]
    if k.shape != v.shape or k.shape[0] != B or k.shape[3] != D or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError(f"k {tuple(k.shape)} {k.dtype} / v {tuple(v.shape)} {v.dtype} do not match "
                         f"q {tuple(q.shape)} {q.dtype}")
    _same(q, "q", out=out)
    if lse.dtype != torch.float32 or not lse.is_contiguous() or tuple(lse.shape) != (B, Hq, Lq):
        raise ValueError("lse must be a contiguous float32 tensor (B, Hq, Lq)")
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    _lib.call("ody_attn_fwd_noalloc", q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
              B, Lq, Lk, Hq, Hkv, D, *_blhd(q, "q"), *_blhd(k, "k"), *_blhd(v, "v"), *_blhd(out, "out"),
              scale, int(causal), _dt(q), _stream())


def attn_bwd(q, k, v, out, lse, dout, causal: bool = True, scale: Optional[float] = None,
             dq=None, dk=None, dv=None, accumulate_dq: bool = False, workspace=None, reuse_query_side: bool = False,
             rope_tables=None, keep_ds: Optional[bool] = None, dropout_p: float = 0.0, seed=None):
    """Gradients of attn_fwd.  `out`/`lse` may be the merged results of a ring step.  dropout_p / seed: those of the
    forward call (on the plain kernels: not with keep_ds=True or rope_tables).

    dq may be a float32 tensor although q is bfloat16: with accumulate_dq that is the running dq of a
    ring step, summed exactly over the key blocks.  reuse_query_side=True (needs the `workspace` of
    the previous call, with the same q / out / lse / dout) skips the scratch that depends on the
    queries only.  rope_tables=(table_q, table_k) (rope_table() of the query / key positions; bf16,
    head_dim 128) makes dq and dk the gradients of the projection BEFORE its rotary embedding.

    keep_ds spends scratch memory to save arithmetic: the dK/dV kernel keeps dS (2 bytes per visible
    query-key pair: about B * Hq * L * L bytes when causal) and dQ becomes one product over it instead of a second
    pass over S and dP.  bfloat16, head_dim 128, Lq and Lk multiples of 256, causal only with Lq == Lk.  It is
    opt-in: None (the default) turns it on only where the shape qualifies, no `workspace` is passed and the
    scratch stays within the budget of set_keep_ds_max_bytes() / ODYSSEUS_KEEP_DS_MAX_BYTES (0 unless set) or is
    already there in the arena; True insists (ValueError where the shape does not qualify); False never."""
    _need_gpu(q, k, v, out, lse, dout)
    _check_dropout(dropout_p, seed)
    if dropout_p > 0.0:
        if keep_ds or rope_tables is not None:
            raise ValueError("attention dropout runs on the plain kernels: no keep_ds, no rope_tables")
        keep_ds = False
    B, Lq, Hq, D = q.shape
    Lk, Hkv = k.shape[1], k.shape[2]
    if dq is None:
        if accumulate_dq:
            raise ValueError("accumulate_dq needs an existing dq")
        dq = torch.empty_like(q)
    dk = torch.empty_like(k) if dk is None else dk
    dv = torch.empty_like(v) if dv is None else dv
    dq_f32 = dq.dtype == torch.float32 and q.dtype != torch.float32
    _same(q, "q", out=out, dout=dout)
    if dq.shape != q.shape or dq.device != q.device or (dq.dtype != q.dtype and not dq_f32):
        raise ValueError(f"dq must have q's shape and device and q's dtype or float32; got {tuple(dq.shape)} {dq.dtype}")
    _same(k, "k", v=v, dk=dk, dv=dv)
    if k.dtype != q.dtype or k.shape[0] != B or k.shape[3] != D or tuple(lse.shape) != (B, Hq, Lq):
        raise ValueError(f"k {tuple(k.shape)} {k.dtype} / lse {tuple(lse.shape)} do not match q {tuple(q.shape)} {q.dtype}")
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    lib = _lib.load()
    ws_bytes = lib.ody_attn_bwd_workspace_bytes(B, Lq, Lk, Hq, Hkv, D, _dt(q))
    ds_bytes = lib.ody_attn_bwd_ds_bytes(B, Lq, Lk, Hq, Hkv, D, _dt(q), int(causal)) if keep_ds is not False else 0
    if keep_ds and ds_bytes == 0:
        raise ValueError(_KEEP_DS_SHAPES)
    ws = None
    if keep_ds is None:
        keep_ds = workspace is None and _keep_ds_fits(ws_bytes, ds_bytes, q.device)
        if keep_ds:
            try:
                ws = scratch(ws_bytes + ds_bytes, "attn_bwd_workspace", q.device)
            except torch.OutOfMemoryError:   # the memory is not there: the recomputing kernels need none of it,
                keep_ds = False              # and this size is not tried again (the allocator's retry synchronises)
                _KEEP_DS_OOM[str(q.device)] = min(ds_bytes, _KEEP_DS_OOM.get(str(q.device), 1 << 62))
    if keep_ds:
        ws_bytes += ds_bytes
    if workspace is None:
        if reuse_query_side:
            raise ValueError("reuse_query_side needs the workspace of the previous call")
        if ws is None:
            ws = scratch(ws_bytes, "attn_bwd_workspace", q.device)
    else:
        ws = workspace
        if ws.dtype != torch.uint8 or ws.numel() < ws_bytes or ws.device != q.device or not ws.is_contiguous():
            raise ValueError(f"workspace must be a contiguous uint8 tensor of at least {ws_bytes} bytes on {q.device}")
    flags = (_lib.BWD_ACCUMULATE_DQ if accumulate_dq else 0) | (_lib.BWD_DQ_F32 if dq_f32 else 0) | \
            (_lib.BWD_REUSE_QUERY_SIDE if reuse_query_side else 0) | (_lib.BWD_KEEP_DS if keep_ds else 0)
    if lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous float32 tensor (B, Hq, Lq)")
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
            dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
            B, Lq, Lk, Hq, Hkv, D, *_blhd(q, "q"), *_blhd(k, "k"), *_blhd(v, "v"), *_blhd(out, "out"),
            *_blhd(dout, "dout"), *_blhd(dq, "dq"), *_blhd(dk, "dk"), *_blhd(dv, "dv"),
            scale, int(causal), flags, _dt(q), ws.data_ptr(), ws_bytes, _stream())
    if dropout_p > 0.0:
        _lib.call("ody_attn_bwd_dropout", *args, float(dropout_p), int(seed) & 0xFFFFFFFFFFFFFFFF)
    elif rope_tables is None:
        _lib.call("ody_attn_bwd", *args)
    else:
        tq, tk = rope_tables
        for t, n, rows in ((tq, "table_q", B * Lq), (tk, "table_k", B * Lk)):
            _need_gpu(t)
            if t.dtype != torch.bfloat16 or not t.is_contiguous() or tuple(t.shape) != (rows, D) or t.device != q.device:
                raise ValueError(f"{n} must be a contiguous bfloat16 ({rows}, {D}) tensor on {q.device}")
        _lib.call("ody_attn_bwd_rope", *args, tq.data_ptr(), tk.data_ptr())
    return dq, dk, dv


_KEEP_DS_MAX_BYTES: Optional[int] = None
_KEEP_DS_OOM: dict = {}   # device -> smallest dS scratch whose allocation failed there (never tried again at or above it)
_KEEP_DS_SHAPES = "keep_ds needs bfloat16, head_dim 128, Lq and Lk multiples of 256 and, if causal, Lq == Lk"


def keep_ds_max_bytes(device=None) -> int:
    """Largest dS scratch that attn_bwd takes on its own (keep_ds=None).  Kept dS is opt-in -- it holds about
    B * Hq * L * L bytes for the life of the arena (4 GiB at 4 heads x 32768 tokens, 64 GiB at L = 131072) for a
    few percent of speed: set_keep_ds_max_bytes(), else the environment variable ODYSSEUS_KEEP_DS_MAX_BYTES, else 0.
    Scratch that the arena's "attn_bwd_workspace" buffer already holds is used whatever the limit says: it costs
    nothing more."""
    if _KEEP_DS_MAX_BYTES is not None:
        return _KEEP_DS_MAX_BYTES
    env = os.environ.get("ODYSSEUS_KEEP_DS_MAX_BYTES")
    if env is not None:
        return int(env)
    return 0


def set_keep_ds_max_bytes(nbytes: Optional[int]) -> None:
    """The budget of kept dS for calls that leave keep_ds=None; 0 turns it off, None restores the default (off unless
    ODYSSEUS_KEEP_DS_MAX_BYTES says otherwise)."""
    global _KEEP_DS_MAX_BYTES
    _KEEP_DS_MAX_BYTES = nbytes
    _KEEP_DS_OOM.clear()


def _arena_holds(name: str, device) -> int:
    """Bytes that the arena's uint8 buffer `name` already holds on `device` (0 without an arena)."""
    from .utils import globals as _globals
    arena = _globals._Arena.instance
    if arena is None:
        return 0
    adev = torch.device(arena.dev)
    if adev.type != device.type or (adev.index is not None and adev.index != device.index):
        return 0
    backing = arena.buffer.get((name, torch.uint8))
    return 0 if backing is None else backing.numel()


def _keep_ds_fits(ws_bytes: int, ds_bytes: int, device) -> bool:
    """The policy of keep_ds=None: within the budget (and not a size that already failed to allocate on this device),
    or free because the arena's buffer is that large already."""
    if ds_bytes <= 0:
        return False
    if ws_bytes + ds_bytes <= _arena_holds("attn_bwd_workspace", device):
        return True
    return ds_bytes <= keep_ds_max_bytes(device) and ds_bytes < _KEEP_DS_OOM.get(str(device), 1 << 62)


def attn_bwd_workspace(q, k, keep_ds: bool = False, causal: bool = True) -> torch.Tensor:
    """A workspace for attn_bwd on these shapes, for callers that make several calls with the same queries
    (keep_ds: with room for the kept dS of attn_bwd(..., keep_ds=True))."""
    B, Lq, Hq, D = q.shape
    lib = _lib.load()
    n = lib.ody_attn_bwd_workspace_bytes(B, Lq, k.shape[1], Hq, k.shape[2], D, _dt(q))
    if keep_ds:
        ds = lib.ody_attn_bwd_ds_bytes(B, Lq, k.shape[1], Hq, k.shape[2], D, _dt(q), int(causal))
        if ds == 0:
            raise ValueError(_KEEP_DS_SHAPES)
        n += ds
    return torch.empty(n, dtype=torch.uint8, device=q.device)


def attn_bwd_workspace_bytes(q, k, keep_ds: bool = False, causal: bool = True) -> Optional[int]:
    """Bytes of workspace that attn_bwd needs on these shapes; None if keep_ds is asked for a shape that cannot keep dS."""
    B, Lq, Hq, D = q.shape
    lib = _lib.load()
    n = lib.ody_attn_bwd_workspace_bytes(B, Lq, k.shape[1], Hq, k.shape[2], D, _dt(q))
    if keep_ds:
        ds = lib.ody_attn_bwd_ds_bytes(B, Lq, k.shape[1], Hq, k.shape[2], D, _dt(q), int(causal))
        if ds == 0:
            return None
        n += ds
    return n


def _shared_bwd_workspace(q, calls):
    """One workspace for a sequence of attn_bwd calls with the same queries: `calls` is a list of (k, causal).
    Returns it with the keep_ds setting of every call: on where the shape qualifies and the scratch stays within
    keep_ds_max_bytes(), all off if that much memory is not there."""
    B, Lq, Hq, D = q.shape
    lib = _lib.load()
    base = [lib.ody_attn_bwd_workspace_bytes(B, Lq, k.shape[1], Hq, k.shape[2], D, _dt(q)) for k, _ in calls]
    ds = [lib.ody_attn_bwd_ds_bytes(B, Lq, k.shape[1], Hq, k.shape[2], D, _dt(q), int(c)) for k, c in calls]
    limit = keep_ds_max_bytes(q.device)
    failed = _KEEP_DS_OOM.get(str(q.device), 1 << 62)
    keeps = [0 < d <= limit and d < failed for d in ds]
    if any(keeps):
        try:
            n = max(b + (d if kp else 0) for b, d, kp in zip(base, ds, keeps))
            return torch.empty(n, dtype=torch.uint8, device=q.device), keeps
        except torch.OutOfMemoryError:
            _KEEP_DS_OOM[str(q.device)] = min(failed, min(d for d, kp in zip(ds, keeps) if kp))
    return torch.empty(max(base), dtype=torch.uint8, device=q.device), [False] * len(calls)


def cast_from_f32(src, dtype) -> torch.Tensor:
    """Rounds a contiguous float32 tensor to `dtype` (the end of an fp32 accumulation over ring blocks)."""
    _need_gpu(src)
    if src.dtype != torch.float32 or not src.is_contiguous():
        raise ValueError("cast_from_f32 takes a contiguous float32 tensor")
    if dtype == torch.float32:
        return src
    dst = torch.empty(src.shape, dtype=dtype, device=src.device)
    if src.numel() % 8:
        return dst.copy_(src)
    _lib.call("ody_cast_from_f32", src.data_ptr(), dst.data_ptr(), src.numel(), _dt(dst), _stream())
    return dst


def lse_merge_(out_acc, lse_acc, out_blk, lse_blk) -> None:
    """In place: folds (out_blk, lse_blk) into the fp32 running (out_acc, lse_acc)."""
    _need_gpu(out_acc, lse_acc, out_blk, lse_blk)
    B, L, H, D = out_blk.shape
    if out_acc.dtype != torch.float32 or not out_acc.is_contiguous() or tuple(out_acc.shape) != (B, L, H, D):
        raise ValueError("out_acc must be a contiguous float32 (B, L, H, D) tensor")
    for t, n in ((lse_acc, "lse_acc"), (lse_blk, "lse_blk")):
        if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (B, H, L):
            raise ValueError(f"{n} must be a contiguous float32 (B, H, L) tensor")
    _lib.call("ody_lse_merge", out_acc.data_ptr(), lse_acc.data_ptr(), out_blk.data_ptr(), lse_blk.data_ptr(),
              B, L, H, D, *_blhd(out_blk, "out_blk"), _dt(out_blk), _stream())


# --------------------------------------------------------------------------- linears
def _rowmajor2d(t: torch.Tensor, name: str) -> int:
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with unit column stride, got shape {tuple(t.shape)} stride {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def gemm(op: int, a, b, bias=None, out=None, accumulate: bool = False):
    """op NT: a (M,K) b (N,K); NN: a (M,K) b (K,N); TN: a (K,M) b (K,N) -> (M,N)."""
    _need_gpu(a, b, bias, out)
    if op == GEMM_NT:
        (M, K), (N, K2) = a.shape, b.shape
    elif op == GEMM_NN:
        (M, K), (K2, N) = a.shape, b.shape
    elif op == GEMM_TN:
        (K, M), (K2, N) = a.shape, b.shape
    else:
        raise ValueError(f"unknown gemm op {op}")
    if K != K2:
        raise ValueError(f"inner dimensions differ: {tuple(a.shape)} vs {tuple(b.shape)} for op {op}")
    if a.dtype != b.dtype:
        raise TypeError(f"dtype mismatch {a.dtype} vs {b.dtype}")
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an existing out")
        out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    if tuple(out.shape) != (M, N) or out.dtype != a.dtype:
        raise ValueError(f"out must be ({M}, {N}) {a.dtype}, got {tuple(out.shape)} {out.dtype}")
    if bias is not None and (tuple(bias.shape) != (N,) or bias.dtype != a.dtype or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous ({N},) {a.dtype} tensor, got {tuple(bias.shape)} {bias.dtype}")
    ws_bytes = _lib.load().ody_gemm_workspace_bytes(op, M, N, K, _dt(a))
    ws = scratch(ws_bytes, "gemm_workspace", a.device) if ws_bytes else None
    _lib.call("ody_gemm", op, a.data_ptr(), b.data_ptr(), out.data_ptr(), 0 if bias is None else bias.data_ptr(),
              M, N, K, _rowmajor2d(a, "a"), _rowmajor2d(b, "b"), _rowmajor2d(out, "out"),
              int(accumulate), _dt(a), ws.data_ptr() if ws is not None else 0, ws_bytes, _stream())
    return out


def _lin_args(x, w, name):
    if x.dim() != 2 or w.dim() != 2 or x.stride(1) != 1 or w.stride(1) != 1:
        raise ValueError(f"{name}: 2-D row-major operands expected, got {tuple(x.shape)} {x.stride()} and "
                         f"{tuple(w.shape)} {w.stride()}")
    if x.dtype != w.dtype or x.device != w.device:
        raise TypeError(f"{name}: operands differ in dtype or device ({x.dtype} {x.device} vs {w.dtype} {w.device})")


def linear_residual(x, weight, residual):
    """x (M, K) W (N, K)^T + residual (M, N), the add in the product's epilogue."""
    _need_gpu(x, weight, residual)
    _lin_args(x, weight, "linear_residual")
    (M, K), N = x.shape, weight.shape[0]
    if weight.shape[1] != K or tuple(residual.shape) != (M, N) or residual.dtype != x.dtype or residual.stride(1) != 1:
        raise ValueError(f"linear_residual: x {tuple(x.shape)}, weight {tuple(weight.shape)}, residual "
                         f"{tuple(residual.shape)} {residual.dtype} do not fit")
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    _lib.call("ody_linear_residual", x.data_ptr(), weight.data_ptr(), residual.data_ptr(), y.data_ptr(), M, N, K,
              _rowmajor2d(x, "x"), _rowmajor2d(weight, "weight"), _rowmajor2d(residual, "residual"), y.stride(0),
              _dt(x), _stream())
    return y


_ROPE_TABLE_LAST = None   # (position tensor, its version, rows, head_dim, base, device, stream, table) of the last table built


def _tensor_version(t) -> int:
    """The autograd version counter of `t`; inference tensors (torch.inference_mode) have none and cannot be
    modified in place outside that mode: -1."""
    try:
        return t._version
    except RuntimeError:
        return -1


def rope_table(position_ids, rows: int, head_dim: int, base: float = 10000.0, device=None, inv_freq=None) -> torch.Tensor:
    """(rows, head_dim) bfloat16: [r, 2 j] = cos, [r, 2 j + 1] = sin of position r times frequency j, rounded
    as rope_ rounds them.  position_ids: int64 with `rows` elements in the order of the rows -- or with rows / B
    elements, one sequence that every batch entry shares, e.g. (1, L) for (B, L) rows -- or None for arange.

    The layers of a model are handed one and the same position tensor: the last table is kept and returned again
    for the same tensor object (unmodified since), shape, base and stream.  Treat the result as read-only."""
    global _ROPE_TABLE_LAST
    pos_arg = position_ids
    if position_ids is not None:
        _need_gpu(position_ids)
        device = position_ids.device
    if device is None:
        raise ValueError("rope_table needs position_ids or a device")
    device = torch.device(device)
    key = (None if pos_arg is None else _tensor_version(pos_arg), rows, head_dim, float(base), str(device), _stream())
    last = _ROPE_TABLE_LAST
    if inv_freq is None and last is not None and last[0] is pos_arg and last[1] == key:
        return last[2]
    if position_ids is not None:
        position_ids = position_ids.to(torch.int64).reshape(-1)
        n = position_ids.numel()
        if n != rows:
            if n == 0 or rows % n:
                raise ValueError(f"{n} positions for {rows} rows")
            position_ids = position_ids.repeat(rows // n)     # one sequence shared by the batch
        position_ids = position_ids.contiguous()
    custom_freq = inv_freq is not None
    if inv_freq is None:
        inv_freq = rope_inv_freq(head_dim, base, device)
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2 or not inv_freq.is_contiguous():
        raise ValueError("inv_freq must be a contiguous float32 tensor of head_dim / 2 elements")
    table = torch.empty((rows, head_dim), dtype=torch.bfloat16, device=device)
    _lib.call("ody_rope_table", position_ids.data_ptr() if position_ids is not None else 0, inv_freq.data_ptr(), rows,
              head_dim, float(base), table.data_ptr(), _stream())
    if not custom_freq:
        _ROPE_TABLE_LAST = (pos_arg, key, table)   # holding pos_arg keeps its identity from being reused
    return table


def linear_rope(x, weight, table, n_rot: int, head_dim: int):
    """x (M, K) W (N, K)^T with the first n_rot heads of head_dim columns rotated by row m of `table`
    (rope_table) in the product's epilogue: the packed QKV projection and its rotary embedding in one kernel."""
    _need_gpu(x, weight, table)
    _lin_args(x, weight, "linear_rope")
    (M, K), N = x.shape, weight.shape[0]
    if weight.shape[1] != K or N % head_dim or not 0 <= n_rot <= N // head_dim:
        raise ValueError(f"linear_rope: x {tuple(x.shape)}, weight {tuple(weight.shape)}, n_rot {n_rot}, head_dim {head_dim}")
    if x.dtype != torch.bfloat16 or head_dim != 128:
        raise ValueError("linear_rope: bfloat16 and head_dim 128 only")
    if table.dtype != torch.bfloat16 or tuple(table.shape) != (M, head_dim) or not table.is_contiguous():
        raise ValueError(f"linear_rope: table must be a contiguous bfloat16 ({M}, {head_dim}) tensor")
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    _lib.call("ody_linear_rope", x.data_ptr(), weight.data_ptr(), table.data_ptr(), y.data_ptr(), M, N, K, n_rot, head_dim,
              _rowmajor2d(x, "x"), _rowmajor2d(weight, "weight"), table.stride(0), y.stride(0), _dt(x), _stream())
    return y


def linear_swiglu(x, w_gate_up):
    """gate_up = x (T, K) Wgu (2 I, K)^T and h = silu(gate) * up in one kernel -> (gate_up, h)."""
    _need_gpu(x, w_gate_up)
    _lin_args(x, w_gate_up, "linear_swiglu")
    (T, K), I2 = x.shape, w_gate_up.shape[0]
    if w_gate_up.shape[1] != K or I2 % 2:
        raise ValueError(f"linear_swiglu: x {tuple(x.shape)} and the packed weight {tuple(w_gate_up.shape)} do not fit")
    gate_up = torch.empty((T, I2), dtype=x.dtype, device=x.device)
    h = torch.empty((T, I2 // 2), dtype=x.dtype, device=x.device)
    _lib.call("ody_linear_swiglu", x.data_ptr(), w_gate_up.data_ptr(), gate_up.data_ptr(), h.data_ptr(), T, I2 // 2, K,
              _rowmajor2d(x, "x"), _rowmajor2d(w_gate_up, "w_gate_up"), gate_up.stride(0), h.stride(0), _dt(x), _stream())
    return gate_up, h


def linear_dgrad_swiglu(dy, w_down, gate_up):
    """d_gate_up from dy (T, K) and the down weight (K, I): dh = dy Wd never leaves the kernel."""
    _need_gpu(dy, w_down, gate_up)
    _lin_args(dy, w_down, "linear_dgrad_swiglu")
    (T, K), I = dy.shape, w_down.shape[1]
    if w_down.shape[0] != K or tuple(gate_up.shape) != (T, 2 * I) or gate_up.dtype != dy.dtype or gate_up.stride(1) != 1:
        raise ValueError(f"linear_dgrad_swiglu: dy {tuple(dy.shape)}, w_down {tuple(w_down.shape)}, gate_up "
                         f"{tuple(gate_up.shape)} {gate_up.dtype} do not fit")
    dgu = torch.empty((T, 2 * I), dtype=dy.dtype, device=dy.device)
    ws_bytes = _lib.load().ody_linear_dgrad_swiglu_workspace_bytes(T, I, K, _dt(dy))
    if ws_bytes == 0 and any(t.data_ptr() % 16 or t.stride(0) % 8 for t in (dy, w_down, gate_up, dgu)):
        # the size query goes by the shape alone; the one-kernel path also wants 16-byte aligned rows, and a
        # column-sliced view without them takes the two-kernel path, which keeps dh (T, I) in a workspace
        ws_bytes = (T * I * dy.element_size() + 255) & ~255
    ws = scratch(ws_bytes, "dgrad_swiglu_workspace", dy.device) if ws_bytes else None
    _lib.call("ody_linear_dgrad_swiglu", dy.data_ptr(), w_down.data_ptr(), gate_up.data_ptr(), dgu.data_ptr(), T, I, K,
              _rowmajor2d(dy, "dy"), _rowmajor2d(w_down, "w_down"), _rowmajor2d(gate_up, "gate_up"), dgu.stride(0),
              _dt(dy), ws.data_ptr() if ws is not None else 0, ws_bytes, _stream())
    return dgu


# --------------------------------------------------------------------------- elementwise
def swiglu_fwd(gate_up):
    _need_gpu(gate_up)
    gu = gate_up.reshape(-1, gate_up.shape[-1])
    T, I2 = gu.shape
    h = torch.empty((T, I2 // 2), dtype=gu.dtype, device=gu.device)
    _lib.call("ody_swiglu_fwd", gu.data_ptr(), h.data_ptr(), T, I2 // 2, _rowmajor2d(gu, "gate_up"), h.stride(0),
              _dt(gu), _stream())
    return h.view(*gate_up.shape[:-1], I2 // 2)


def swiglu_bwd(gate_up, dh):
    _need_gpu(gate_up, dh)
    gu = gate_up.reshape(-1, gate_up.shape[-1])
    d = dh.reshape(-1, dh.shape[-1])
    if d.stride(1) != 1:
        d = d.contiguous()
    T, I2 = gu.shape
    dgu = torch.empty((T, I2), dtype=gu.dtype, device=gu.device)
    _lib.call("ody_swiglu_bwd", gu.data_ptr(), d.data_ptr(), dgu.data_ptr(), T, I2 // 2,
              _rowmajor2d(gu, "gate_up"), _rowmajor2d(d, "dh"), dgu.stride(0), _dt(gu), _stream())
    return dgu.view(gate_up.shape)


def check_rmsnorm_args(x, weight, rstd=None, dy=None) -> None:
    """The kernels read raw pointers: the weight must be a contiguous (d,) tensor of x's dtype on
    x's device, dy must match x, rstd must hold one float32 per row."""
    d = x.shape[-1]
    if weight.dtype != x.dtype:
        raise TypeError(f"rmsnorm: weight is {weight.dtype} but the activations are {x.dtype}; cast the module "
                        "(`.to(dtype)`) so that both agree")
    if tuple(weight.shape) != (d,) or not weight.is_contiguous() or weight.device != x.device:
        raise ValueError(f"rmsnorm: weight must be a contiguous ({d},) tensor on {x.device}, got "
                         f"{tuple(weight.shape)} on {weight.device}")
    if dy is not None and (dy.dtype != x.dtype or dy.shape != x.shape or dy.device != x.device):
        raise ValueError(f"rmsnorm: dy must match x ({tuple(x.shape)}, {x.dtype}, {x.device}); got "
                         f"{tuple(dy.shape)}, {dy.dtype}, {dy.device}")
    if rstd is not None:
        rows = x.numel() // d if d else 0
        if rstd.dtype != torch.float32 or rstd.numel() != rows or not rstd.is_contiguous() or rstd.device != x.device:
            raise ValueError(f"rmsnorm: rstd must be a contiguous float32 tensor of {rows} rows on {x.device}; got "
                             f"{tuple(rstd.shape)}, {rstd.dtype}, {rstd.device}")


def check_rope_args(x, n_rot, position_ids, inv_freq) -> None:
    B, L, H, D = x.shape
    if not 0 <= n_rot <= H:
        raise ValueError(f"n_rot={n_rot} exceeds the {H} heads of x")
    if D % 2:
        raise ValueError(f"rope: head_dim {D} is odd")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or tuple(inv_freq.shape) != (D // 2,)
                                 or not inv_freq.is_contiguous() or inv_freq.device != x.device):
        raise ValueError(f"rope: inv_freq must be a contiguous float32 ({D // 2},) tensor on {x.device}; got "
                         f"{tuple(inv_freq.shape)}, {inv_freq.dtype}, {inv_freq.device}")
    if position_ids is not None:
        if position_ids.dtype not in (torch.int64, torch.int32) or position_ids.device != x.device:
            raise ValueError(f"rope: position_ids must be an integer tensor on {x.device}; got "
                             f"{position_ids.dtype} on {position_ids.device}")
        if position_ids.shape[-1] != L or position_ids.numel() not in (L, B * L):
            raise ValueError(f"rope: position_ids {tuple(position_ids.shape)} do not cover (B={B}, L={L})")


def rmsnorm_fwd(x, weight, eps: float = 1e-6):
    _need_gpu(x, weight)
    check_rmsnorm_args(x, weight)
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    T, d = x2.shape
    y = torch.empty_like(x2)
    rstd = torch.empty(T, dtype=torch.float32, device=x.device)
    _lib.call("ody_rmsnorm_fwd", x2.data_ptr(), weight.data_ptr(), y.data_ptr(), rstd.data_ptr(), T, d, float(eps),
              _dt(x2), _stream())
    return y.view(x.shape), rstd


def rmsnorm_bwd(x, weight, rstd, dy, dx_add=None):
    """dx, dw of rmsnorm; `dx_add` (same shape as x) is added to dx inside the kernel: the
    gradient that reaches the norm's input over the residual connection."""
    _need_gpu(x, weight, rstd, dy, dx_add)
    check_rmsnorm_args(x, weight, rstd, dy)
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    dy2 = dy.reshape(-1, dy.shape[-1]).contiguous()
    add_ptr = 0
    if dx_add is not None:
        if dx_add.dtype != x.dtype or dx_add.shape != x.shape or dx_add.device != x.device:
            raise ValueError(f"rmsnorm: dx_add must match x ({tuple(x.shape)}, {x.dtype}, {x.device})")
        dx_add = dx_add.reshape(-1, x.shape[-1]).contiguous()
        add_ptr = dx_add.data_ptr()
    T, d = x2.shape
    dx = torch.empty_like(x2)
    dw = torch.empty_like(weight)
    nparts = _lib.load().ody_rmsnorm_bwd_partials(T)
    partial = scratch(nparts * d * 4, "rmsnorm_dw_partials", x.device)
    _lib.call("ody_rmsnorm_bwd", x2.data_ptr(), weight.data_ptr(), rstd.data_ptr(), dy2.data_ptr(), add_ptr,
              dx.data_ptr(), partial.data_ptr(), dw.data_ptr(), T, d, _dt(x2), _stream())
    return dx.view(x.shape), dw


_INV_FREQ_CACHE = {}


def rope_inv_freq(head_dim: int, base: float, device) -> torch.Tensor:
    """base^(-2j/D), evaluated on the host in fp32 the way HF's rotary module does, then moved."""
    key = (head_dim, float(base), str(device))
    t = _INV_FREQ_CACHE.get(key)
    if t is None:
        t = (1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))).to(device)
        _INV_FREQ_CACHE[key] = t
    return t


def rope_(x, n_rot: int, position_ids=None, base: float = 10000.0, inverse: bool = False, inv_freq=None) -> None:
    """Rotates heads [0, n_rot) of x (B, L, H, D) in place."""
    _need_gpu(x, position_ids, inv_freq)
    B, L, H, D = x.shape
    if inv_freq is None:
        inv_freq = rope_inv_freq(D, base, x.device)
    check_rope_args(x, n_rot, position_ids, inv_freq)
    pos_ptr = 0
    if position_ids is not None:
        position_ids = position_ids.to(torch.int64).expand(B, L).contiguous()
        pos_ptr = position_ids.data_ptr()
    _lib.call("ody_rope", x.data_ptr(), pos_ptr, inv_freq.data_ptr(), B, L, n_rot, D, *_blhd(x, "x"),
              float(base), int(inverse), _dt(x), _stream())


# --------------------------------------------------------------------------- autograd
class FlashAttnFunc(torch.autograd.Function):
    """Causal/full attention with GQA over (B, L, H, D) tensors; returns (out, lse)."""

    @staticmethod
    def forward(ctx, q, k, v, softmax_scale, causal, dropout_p=0.0, seed=None):
        out, lse = attn_fwd(q, k, v, causal=causal, scale=softmax_scale, dropout_p=dropout_p, seed=seed)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.softmax_scale, ctx.causal, ctx.dropout = softmax_scale, causal, (dropout_p, seed)
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, k, v, out, lse = ctx.saved_tensors
        if dout.stride(3) != 1:
            dout = dout.contiguous()
        dq, dk, dv = attn_bwd(q, k, v, out, lse, dout, causal=ctx.causal, scale=ctx.softmax_scale,
                              dropout_p=ctx.dropout[0], seed=ctx.dropout[1])
        return dq, dk, dv, None, None, None, None


class RingBlocksAttnFunc(torch.autograd.Function):
    """One rank's inner loop of ring attention (entered at decoder/ring.py:30-37 in the reference):
    the local queries against a sequence of K/V blocks as they would arrive over the ring.  Block
    `causal_block` is the diagonal one (causally masked); every other block is fully visible.
    Forward merges each block's (out, lse) into an fp32 running pair; backward runs the per-block
    flash backward with the FINAL out / lse and accumulates dq over the blocks.

    apply(q, causal_block, softmax_scale, *k_blocks, *v_blocks) -> (out, lse)."""

    @staticmethod
    def forward(ctx, q, causal_block, softmax_scale, *kv):
        nb = len(kv) // 2
        ks, vs = kv[:nb], kv[nb:]
        B, L, H, D = q.shape
        acc = torch.zeros((B, L, H, D), dtype=torch.float32, device=q.device)
        lse = torch.full((B, H, L), float("-inf"), dtype=torch.float32, device=q.device)
        for b in range(nb):
            ob, lb = attn_fwd(q, ks[b], vs[b], causal=(b == causal_block), scale=softmax_scale)
            lse_merge_(acc, lse, ob, lb)
        out = cast_from_f32(acc, q.dtype)
        ctx.save_for_backward(q, out, lse, *kv)
        ctx.causal_block, ctx.softmax_scale = causal_block, softmax_scale
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, out, lse, *kv = ctx.saved_tensors
        nb = len(kv) // 2
        ks, vs = kv[:nb], kv[nb:]
        if dout.stride(3) != 1:
            dout = dout.contiguous()
        # the running dq stays in fp32 over the blocks and is rounded once; delta, the start values and the
        # Q / dO images depend on the queries only and are built by the first block's call
        dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
        same_kv_shape = all(k.shape == ks[0].shape for k in ks)
        ws, keeps = _shared_bwd_workspace(q, [(ks[b], b == ctx.causal_block) for b in range(nb)]) if nb else (None, [])
        dks, dvs = [], []
        for b in range(nb):
            _, dk, dv = attn_bwd(q, ks[b], vs[b], out, lse, dout, causal=(b == ctx.causal_block),
                                 scale=ctx.softmax_scale, dq=dq, accumulate_dq=(b > 0), workspace=ws,
                                 reuse_query_side=(b > 0 and same_kv_shape), keep_ds=keeps[b])
            dks.append(dk)
            dvs.append(dv)
        return (cast_from_f32(dq, q.dtype), None, None, *dks, *dvs)


def ring_blocks_attn(q, k_blocks, v_blocks, causal_block: Optional[int] = 0, softmax_scale: Optional[float] = None):
    """Functional form of RingBlocksAttnFunc; causal_block=None makes every block fully visible."""
    cb = -1 if causal_block is None else int(causal_block)
    return RingBlocksAttnFunc.apply(q, cb, softmax_scale, *k_blocks, *v_blocks)


class ZigzagRingRankAttnFunc(torch.autograd.Function):
    """One rank's compute of zigzag ring attention (the routine decoder/ring.py:30-37 of the reference calls,
    ring_flash_attn's zigzag_ring_flash_attn_func: the sequence is cut into 2N chunks and rank r holds chunks r and
    2N-1-r, see utils/apply_seq_parallel.py:93-99).  The K/V blocks a rank receives over the ring are arguments
    here: block s is the local K/V of rank (r - s) mod N.

        step 0           local queries x local keys, causal (chunk r precedes chunk 2N-1-r)
        source rank < r  all local queries x the FIRST chunk of the block, fully visible
        source rank > r  the queries of the SECOND local chunk x the whole block, fully visible

    Every step's (out, lse) is merged into fp32 running pairs (one per local chunk); backward runs the per-step
    flash backward with the final out / lse, a running fp32 dq, and returns each block's dK / dV (zero in the
    half a step did not read), which the ring would send on with the block.

    apply(q, rank, world_size, softmax_scale, *k_blocks, *v_blocks) -> (out, lse)."""

    @staticmethod
    def _steps(rank, world):
        """[(query chunk range, key chunk range, causal)] in units of chunks of the local sequence (0..2)."""
        steps = [((0, 2), (0, 2), True)]
        for s in range(1, world):
            src = (rank - s) % world
            steps.append(((0, 2), (0, 1), False) if src < rank else ((1, 2), (0, 2), False))
        return steps

    @staticmethod
    def forward(ctx, q, rank, world, softmax_scale, *kv):
        if len(kv) != 2 * world:
            raise ValueError(f"{world} key and {world} value blocks expected, got {len(kv)} tensors")
        ks, vs = kv[:world], kv[world:]
        B, L2, H, D = q.shape
        if L2 % 2:
            raise ValueError(f"the local sequence holds two chunks of equal length, got {L2} tokens")
        c = L2 // 2
        for t in kv:
            if t.shape[1] != L2:
                raise ValueError(f"every block holds two chunks of {c} tokens, got {tuple(t.shape)}")
        acc = [torch.zeros((B, c, H, D), dtype=torch.float32, device=q.device) for _ in range(2)]
        lse = [torch.full((B, H, c), float("-inf"), dtype=torch.float32, device=q.device) for _ in range(2)]
        for s, ((q0, q1), (k0, k1), causal) in enumerate(ZigzagRingRankAttnFunc._steps(rank, world)):
            ob, lb = attn_fwd(q[:, q0 * c:q1 * c], ks[s][:, k0 * c:k1 * c], vs[s][:, k0 * c:k1 * c], causal=causal,
                              scale=softmax_scale)
            for i, ch in enumerate(range(q0, q1)):
                lb_ch = lb if q1 - q0 == 1 else lb[:, :, i * c:(i + 1) * c].contiguous()
                lse_merge_(acc[ch], lse[ch], ob[:, i * c:(i + 1) * c], lb_ch)
        out = torch.cat([cast_from_f32(a, q.dtype) for a in acc], dim=1)
        lse_full = torch.cat(lse, dim=2)
        ctx.save_for_backward(q, out, lse_full, *kv)
        ctx.rank, ctx.world, ctx.softmax_scale = rank, world, softmax_scale
        ctx.mark_non_differentiable(lse_full)
        return out, lse_full

    @staticmethod
    def backward(ctx, dout, _dlse):
        q, out, lse, *kv = ctx.saved_tensors
        world = ctx.world
        ks, vs = kv[:world], kv[world:]
        c = q.shape[1] // 2
        if dout.stride(3) != 1:
            dout = dout.contiguous()
        dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
        lse_b = lse[:, :, c:].contiguous()
        steps = list(ZigzagRingRankAttnFunc._steps(ctx.rank, world))
        # sized for the largest step (both query chunks against both key chunks); a step with fewer queries asks for less
        ws, _ = _shared_bwd_workspace(q, [(ks[0], False)])
        dks = [torch.zeros_like(k) for k in ks]
        dvs = [torch.zeros_like(v) for v in vs]
        prev = None
        for s, ((q0, q1), (k0, k1), causal) in enumerate(steps):
            qs, kr = slice(q0 * c, q1 * c), slice(k0 * c, k1 * c)
            kind = (q0, q1, k0, k1)
            need = attn_bwd_workspace_bytes(q[:, qs], ks[s][:, kr], True, causal)
            attn_bwd(q[:, qs], ks[s][:, kr], vs[s][:, kr], out[:, qs], lse if q1 - q0 == 2 else lse_b, dout[:, qs],
                     causal=causal, scale=ctx.softmax_scale, dq=dq[:, qs], dk=dks[s][:, kr], dv=dvs[s][:, kr],
                     accumulate_dq=(s > 0), workspace=ws, reuse_query_side=(kind == prev),
                     keep_ds=(need is not None and need <= ws.numel()))
            prev = kind
        return (cast_from_f32(dq, q.dtype), None, None, None, *dks, *dvs)


def zigzag_ring_rank_attn(q, k_blocks, v_blocks, rank: int, world_size: int, softmax_scale: Optional[float] = None):
    """Functional form of ZigzagRingRankAttnFunc: (out, lse) of rank `rank`'s two chunks."""
    return ZigzagRingRankAttnFunc.apply(q, int(rank), int(world_size), softmax_scale, *k_blocks, *v_blocks)


def flash_attn_func(q, k, v, dropout_p: float = 0.0, softmax_scale: Optional[float] = None, causal: bool = False,
                    return_lse: bool = False, seed: Optional[int] = None):
    """Signature of the routine the reference reaches at decoder/odysseus.py:256-263.

    dropout_p > 0: the mask's seed is `seed`, or one drawn from torch's default CPU generator, so that
    torch.manual_seed makes runs repeatable; the backward reproduces the mask from it.  (The reference's routine draws
    its masks from a generator of its own: the masks differ, their distribution and the arithmetic do not.)  The seed is
    a host value: a captured graph replays the mask it was captured with -- pass `seed` per step there."""
    if dropout_p != 0.0 and seed is None:
        seed = int(torch.randint(0, 1 << 62, (1,)).item())
    out, lse = FlashAttnFunc.apply(q, k, v, softmax_scale, causal, float(dropout_p), seed)
    return (out, lse) if return_lse else out


class RMSNormFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        y, rstd = rmsnorm_fwd(x, weight, eps)
        ctx.save_for_backward(x, weight, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, rstd = ctx.saved_tensors
        dx, dw = rmsnorm_bwd(x, weight, rstd, dy)
        return dx, dw, None


class SwiGLUFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate_up):
        ctx.save_for_backward(gate_up)
        return swiglu_fwd(gate_up)

    @staticmethod
    def backward(ctx, dh):
        (gate_up,) = ctx.saved_tensors
        return swiglu_bwd(gate_up, dh)


class RoPEFunc(torch.autograd.Function):
    """Rotates the first n_rot heads of a packed (B, L, H, D) projection; out of place for autograd."""

    @staticmethod
    def forward(ctx, x, n_rot, position_ids, base):
        y = x.clone()
        rope_(y, n_rot, position_ids, base)
        ctx.n_rot, ctx.base = n_rot, base
        ctx.position_ids = position_ids
        return y

    @staticmethod
    def backward(ctx, dy):
        dx = dy.clone() if dy.stride(3) == 1 else dy.contiguous()
        rope_(dx, ctx.n_rot, ctx.position_ids, ctx.base, inverse=True)
        return dx, None, None, None


class RMSNormForkFunc(torch.autograd.Function):
    """(norm(x), x): the point where the residual stream forks into a normalised branch and the skip
    connection.  Autograd would add the two gradients that come back with a kernel of its own; here the
    skip gradient goes into the norm's backward kernel as `dx_add`."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        y, rstd = rmsnorm_fwd(x, weight, eps)
        ctx.save_for_backward(x, weight, rstd)
        ctx.set_materialize_grads(False)
        return y, x.view_as(x)

    @staticmethod
    def backward(ctx, dy, dskip):
        x, weight, rstd = ctx.saved_tensors
        if dy is None:
            return dskip, None, None
        dx, dw = rmsnorm_bwd(x, weight, rstd, dy, dx_add=dskip)
        return dx, dw, None


class LinearResidualFunc(torch.autograd.Function):
    """residual + x W^T with the add in the product's epilogue; backward: dX = dY W, dW = dY^T X and
    the residual's gradient is dY itself."""

    @staticmethod
    def forward(ctx, x, weight, residual):
        ctx.save_for_backward(x, weight)
        y = linear_residual(x.reshape(-1, x.shape[-1]), weight, residual.reshape(-1, residual.shape[-1]))
        return y.view(residual.shape)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1])
        dy2 = dy2 if dy2.stride(1) == 1 else dy2.contiguous()
        dx = gemm(GEMM_NN, dy2, weight).view(x.shape)
        x2 = x.reshape(-1, x.shape[-1])
        dw = gemm(GEMM_TN, dy2, x2 if x2.stride(1) == 1 else x2.contiguous())
        return dx, dw, dy


class QKVRoPEAttnFunc(torch.autograd.Function):
    """Packed QKV projection, rotary embedding of q and k and causal GQA attention with no separate rotary
    pass (bf16, head_dim 128): forward rotates in the projection's epilogue, backward un-rotates dq and dk in the
    epilogues of the attention backward (decoder/odysseus.py:180-263 of the reference, utils/linear_tpsp.py:173,
    217,291 for the three products).  Returns (qkv, out, lse); qkv is the rotated projection (for a KV cache)."""

    @staticmethod
    def forward(ctx, x, weight, n_heads, n_kv_heads, head_dim, position_ids, rope_base, softmax_scale):
        B, L, K = x.shape
        x2 = x.reshape(B * L, K)
        x2 = x2 if x2.stride(1) == 1 else x2.contiguous()
        # the tensor as the caller handed it over: every layer passes the same object, which is what the table's
        # cache goes by (a (1, L) tensor serves all B batch entries)
        table = rope_table(position_ids, B * L, head_dim, rope_base, device=x.device)
        H = n_heads + 2 * n_kv_heads
        qkv = linear_rope(x2, weight, table, n_heads + n_kv_heads, head_dim).view(B, L, H, head_dim)
        a, b = n_heads, n_heads + n_kv_heads
        out, lse = attn_fwd(qkv[:, :, :a], qkv[:, :, a:b], qkv[:, :, b:], causal=True, scale=softmax_scale)
        ctx.save_for_backward(x2, weight, qkv, out, lse, table)
        ctx.dims = (n_heads, n_kv_heads, head_dim, softmax_scale, x.shape)
        ctx.mark_non_differentiable(lse, qkv)
        return qkv, out, lse

    @staticmethod
    def backward(ctx, _dqkv, dout, _dlse):
        x2, weight, qkv, out, lse, table = ctx.saved_tensors
        n_heads, n_kv_heads, head_dim, softmax_scale, x_shape = ctx.dims
        if dout.stride(3) != 1:
            dout = dout.contiguous()
        dqkv = torch.empty_like(qkv)
        a, b = n_heads, n_heads + n_kv_heads
        attn_bwd(qkv[:, :, :a], qkv[:, :, a:b], qkv[:, :, b:], out, lse, dout, causal=True, scale=softmax_scale,
                 dq=dqkv[:, :, :a], dk=dqkv[:, :, a:b], dv=dqkv[:, :, b:], rope_tables=(table, table))
        d2 = dqkv.view(x2.shape[0], -1)
        dx = gemm(GEMM_NN, d2, weight).view(x_shape)
        dw = gemm(GEMM_TN, d2, x2)
        return dx, dw, None, None, None, None, None, None


class SwiGLUMLPResidualFunc(torch.autograd.Function):
    """[residual +] down(silu(gate) * up) with gate_up = x Wgu^T, every elementwise step inside a product's
    epilogue: SwiGLU in the gate_up product, the residual add (when a residual is given) in the down
    product, the SwiGLU backward in the down product's input gradient (decoder/odysseus.py:293-295 and
    the add at decoder/ring.py:86)."""

    @staticmethod
    def forward(ctx, x, w_gate_up, w_down, residual):
        x2 = x.reshape(-1, x.shape[-1])
        x2 = x2 if x2.stride(1) == 1 else x2.contiguous()
        gate_up, h = linear_swiglu(x2, w_gate_up)
        if residual is not None:
            y = linear_residual(h, w_down, residual.reshape(-1, residual.shape[-1]))
        else:
            y = gemm(GEMM_NT, h, w_down)
        ctx.save_for_backward(x2, w_gate_up, w_down, gate_up, h)
        ctx.x_shape, ctx.has_residual = x.shape, residual is not None
        return y.view(*x.shape[:-1], w_down.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x2, w_gate_up, w_down, gate_up, h = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1])
        dy2 = dy2 if dy2.stride(1) == 1 else dy2.contiguous()
        dw_down = gemm(GEMM_TN, dy2, h)
        dgu = linear_dgrad_swiglu(dy2, w_down, gate_up)
        dx = gemm(GEMM_NN, dgu, w_gate_up).view(ctx.x_shape)
        dw_gate_up = gemm(GEMM_TN, dgu, x2)
        return dx, dw_gate_up, dw_down, dy if ctx.has_residual else None


def rmsnorm(x, weight, eps: float = 1e-6):
    return RMSNormFunc.apply(x, weight, eps)


def rmsnorm_fork(x, weight, eps: float = 1e-6):
    """-> (rmsnorm(x), x) with the two returning gradients summed inside the norm's backward kernel."""
    return RMSNormForkFunc.apply(x, weight, eps)


def swiglu(gate_up):
    return SwiGLUFunc.apply(gate_up)


def apply_rope_packed(qkv, n_rot: int, position_ids=None, base: float = 10000.0):
    return RoPEFunc.apply(qkv, n_rot, position_ids, base)
