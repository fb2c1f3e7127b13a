"""GPU parity: attention forward/backward through the C ABI vs. the CPU oracle."""
import math

import pytest
import torch

from conftest import TOL_BF16, TOL_F32, TOL_LSE, assert_parity, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu

CASES = [
    # B, Lq, Lk, Hq, Hkv, D, causal
    (1, 128, 128, 2, 2, 128, True),
    (1, 256, 256, 4, 4, 128, True),
    (2, 200, 200, 4, 2, 128, True),      # ragged length, GQA 2:1, batch 2
    (1, 333, 333, 4, 1, 128, True),      # GQA 4:1
    (1, 257, 257, 8, 8, 64, True),       # head_dim 64
    (1, 192, 320, 4, 4, 128, False),     # full block, Lq != Lk (ring step)
    (1, 192, 320, 4, 2, 128, True),      # causal with key offset
    (1, 1, 1, 1, 1, 128, True),          # single token
    (1, 1024, 1024, 4, 1, 128, True),
    (1, 300, 100, 4, 2, 128, True),      # fewer keys than queries: the first 200 queries see no key
    (2, 200, 72, 8, 8, 64, True),        # the same at head_dim 64
]


def _inputs(B, Lq, Lk, Hq, Hkv, D, dtype, seed):
    q = randn((B, Lq, Hq, D), seed, dtype=dtype)
    k = randn((B, Lk, Hkv, D), seed + 1, dtype=dtype)
    v = randn((B, Lk, Hkv, D), seed + 2, dtype=dtype)
    do = randn((B, Lq, Hq, D), seed + 3, dtype=dtype)
    return q, k, v, do


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_D%d_c%d" % c)
def test_attention_fwd_bwd(case, dtype, dev):
    from odysseus_transformer_amd import ops
    B, Lq, Lk, Hq, Hkv, D, causal = case
    print(f"case={case} dtype={dtype}", flush=True)
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    q, k, v, do = _inputs(B, Lq, Lk, Hq, Hkv, D, dtype, seed=17)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(),
                                                  causal=causal)
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=causal)
    torch.cuda.synchronize()
    assert_parity(o, o_ref, tol, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    dq, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal)
    torch.cuda.synchronize()
    # with a single key dS = P (dP - delta) is identically zero: compare on the scale of the inputs
    floor = 1.0 if Lk == 1 else 1e-3
    assert_parity(dq, dq_ref, tol, "dq", floor)
    assert_parity(dk, dk_ref, tol, "dk", floor)
    assert_parity(dv, dv_ref, tol, "dv")


def test_attention_strided_views_of_packed_qkv(dev):
    """q/k/v as head-axis slices of one packed (B, L, Hq+2Hkv, D) buffer, no copies."""
    from odysseus_transformer_amd import ops
    B, L, Hq, Hkv, D = 1, 384, 4, 2, 128
    qkv = randn((B, L, Hq + 2 * Hkv, D), 5, dtype=torch.bfloat16)
    q, k, v = oracle.split_qkv(qkv.view(B, L, -1), Hq, Hkv, D)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float())
    g = qkv.to(dev)
    qg, kg, vg = g[:, :, :Hq], g[:, :, Hq:Hq + Hkv], g[:, :, Hq + Hkv:]
    assert not qg.is_contiguous()
    o, lse = ops.attn_fwd(qg, kg, vg, causal=True)
    assert_parity(o, o_ref, TOL_BF16, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    # gradients written straight into a packed dqkv buffer
    do = randn((B, L, Hq, D), 6, dtype=torch.bfloat16)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float())
    dqkv = torch.zeros_like(g)
    ops.attn_bwd(qg, kg, vg, o, lse, do.to(dev), dq=dqkv[:, :, :Hq], dk=dqkv[:, :, Hq:Hq + Hkv],
                 dv=dqkv[:, :, Hq + Hkv:])
    assert_parity(dqkv[:, :, :Hq], dq_ref, TOL_BF16, "dq")
    assert_parity(dqkv[:, :, Hq:Hq + Hkv], dk_ref, TOL_BF16, "dk")
    assert_parity(dqkv[:, :, Hq + Hkv:], dv_ref, TOL_BF16, "dv")


def test_attention_row_properties(dev):
    """Size-independent facts: row 0 sees only key 0; softmax rows sum to one (via lse)."""
    from odysseus_transformer_amd import ops
    B, L, H, D = 1, 4096, 4, 128
    q, k, v, _ = _inputs(B, L, L, H, H, D, torch.bfloat16, seed=3)
    qg, kg, vg = q.to(dev), k.to(dev), v.to(dev)
    o, lse = ops.attn_fwd(qg, kg, vg, causal=True)
    assert torch.equal(o[:, 0].cpu(), v[:, 0])
    s00 = (q[:, 0].float() * k[:, 0].float()).sum(-1) / math.sqrt(D)
    assert torch.allclose(lse[:, :, 0].cpu(), s00, atol=1e-4, rtol=1e-4)
    # row-sampled fp64 brute force at full length
    rows = torch.tensor([1, 63, 64, 127, 128, 1000, 2047, 2048, 4095])
    for h in range(H):
        s = (q[0, rows, h].double() @ k[0, :, h].double().T) / math.sqrt(D)
        s = s.masked_fill(torch.arange(L)[None, :] > rows[:, None], float("-inf"))
        ref_lse = torch.logsumexp(s, -1)
        ref_o = torch.softmax(s, -1) @ v[0, :, h].double()
        assert torch.allclose(lse[0, h, rows].cpu().double(), ref_lse, atol=TOL_LSE, rtol=TOL_LSE)
        assert_parity(o[0, rows, h], ref_o, TOL_BF16, f"out head {h}")


def test_attention_scores_beyond_the_reference_window(dev):
    """The head_dim-128 forward fixes its softmax reference from the first keys and hands a
    query block whose later scores exceed it by more than 2^64 to the online-rescaling
    kernel: the results must be right on both sides of that switch."""
    from odysseus_transformer_amd import ops
    B, L, H, D = 1, 700, 2, 128
    q, k, v, do = _inputs(B, L, L, H, H, D, torch.bfloat16, seed=29)
    # head 0: early keys score about -90, a run of late keys about +90 (in units of log 2: +-130)
    q[:, :, 0] = 2.0
    k[:, :, 0] = -4.0
    k[:, 500:520, 0] = 4.0
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=True)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float())
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=True)
    assert torch.isfinite(o).all() and torch.isfinite(lse).all()
    assert_parity(o, o_ref, TOL_BF16, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    dq, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=True)
    # head 0 is built to be degenerate: every query's softmax sits on a handful of keys, so its dS
    # is small by cancellation in whole blocks of rows; the gradients are held to the scale of the
    # tensor here, and to the scale of their own block in every other test
    assert rel_err(dq, dq_ref) <= TOL_BF16 and rel_err(dk, dk_ref) <= TOL_BF16 and rel_err(dv, dv_ref) <= TOL_BF16
    assert_parity(dq[:, :, 1:], dq_ref[:, :, 1:], TOL_BF16, "dq of the ordinary head")
    assert_parity(dk[:, :, 1:], dk_ref[:, :, 1:], TOL_BF16, "dk of the ordinary head")
    assert_parity(dv[:, :, 1:], dv_ref[:, :, 1:], TOL_BF16, "dv of the ordinary head")


def test_attention_errors(dev):
    from odysseus_transformer_amd import ops
    from odysseus_transformer_amd._lib import OdysseusHipError
    q = torch.zeros(1, 8, 3, 128, dtype=torch.bfloat16, device=dev)
    k = torch.zeros(1, 8, 2, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(OdysseusHipError):          # Hq not a multiple of Hkv
        ops.attn_fwd(q, k, k)
    q = torch.zeros(1, 8, 2, 96, dtype=torch.bfloat16, device=dev)
    with pytest.raises(OdysseusHipError):          # head_dim not built
        ops.attn_fwd(q, q, q)
    with pytest.raises(RuntimeError):              # CPU tensors are refused, no fallback
        ops.attn_fwd(q.cpu(), q.cpu(), q.cpu())


def _random_cases(n, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    cases = []
    for _ in range(n):
        hkv = [1, 2, 4][r(0, 2)]
        grp = [1, 2, 4][r(0, 2)]
        lq = [r(1, 96), r(97, 400), r(401, 1100)][r(0, 2)]
        kind = r(0, 3)                       # 0/1: square causal, 2: causal with more keys, 3: full block
        lk = lq if kind < 2 else lq + r(1, 500) if kind == 2 else r(1, 900)
        cases.append((r(1, 2), lq, lk, hkv * grp, hkv, kind != 3))
    return cases


@pytest.mark.parametrize("case", _random_cases(36, 2024), ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_c%d" % c)
def test_attention_random_shapes(case, dev):
    """Ragged lengths on both sides of every tile size (32, 64, 256), key offsets, group sizes 1/2/4."""
    from odysseus_transformer_amd import ops
    B, Lq, Lk, Hq, Hkv, causal = case
    print(f"case={case}", flush=True)
    q, k, v, do = _inputs(B, Lq, Lk, Hq, Hkv, 128, torch.bfloat16, seed=Lq * 7 + Lk)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(),
                                                  causal=causal)
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=causal)
    dq, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal)
    floor = 1.0 if Lk == 1 else 1e-3
    assert_parity(o, o_ref, TOL_BF16, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    assert_parity(dq, dq_ref, TOL_BF16, "dq", floor)
    assert_parity(dk, dk_ref, TOL_BF16, "dk", floor)
    assert_parity(dv, dv_ref, TOL_BF16, "dv")


def _random_long_cases(n, seed):
    """One long and one arbitrary side: the shapes on which the kernels cut a block's range into parts."""
    g = torch.Generator().manual_seed(seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    cases = []
    for _ in range(n):
        hkv = [1, 2][r(0, 1)]
        grp = [1, 2][r(0, 1)]
        long, short = r(2049, 5200), r(1, 1400)
        kind = r(0, 3)                       # 0: long queries, 1: long keys, 2: both long and causal, 3: causal with more keys
        lq, lk = [(long, short), (short, long), (long, long), (short, short + long)][kind]
        cases.append((1, lq, lk, hkv * grp, hkv, kind >= 2))
    return cases


@pytest.mark.parametrize("case", _random_long_cases(10, 31), ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_c%d" % c)
def test_attention_random_long_shapes(case, dev):
    """Ragged lengths where one side is long enough for the key split of the forward and the range parts of the
    backward to apply (recomputing kernels: the lengths are not multiples of 256)."""
    test_attention_random_shapes(case, dev)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("case", _random_cases(10, 77), ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_c%d" % c)
def test_attention_random_shapes_fp32(case, D, dev):
    """The fp32 kernels on ragged lengths around their 32- and 128-row tiles, key offsets and groups."""
    from odysseus_transformer_amd import ops
    B, Lq, Lk, Hq, Hkv, causal = case
    print(f"case={case} D={D}", flush=True)
    q, k, v, do = _inputs(B, Lq, Lk, Hq, Hkv, D, torch.float32, seed=Lq * 5 + Lk + D)
    o_ref, lse_ref = oracle.attention_fwd(q, k, v, causal=causal)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q, k, v, o_ref, lse_ref, do, causal=causal)
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=causal)
    dq0 = randn((B, Lq, Hq, D), 99).to(dev)
    dq = dq0.clone()
    _, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, dq=dq, accumulate_dq=True)
    floor = 1.0 if Lk == 1 else 1e-3
    assert_parity(o, o_ref, TOL_F32, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    assert_parity(dq - dq0, dq_ref, 4 * TOL_F32, "dq", floor)  # the difference of two rounded sums
    assert_parity(dk, dk_ref, TOL_F32, "dk", floor)
    assert_parity(dv, dv_ref, TOL_F32, "dv")


KEEP_DS_CASES = [
    # B, L, Hq, Hkv
    (1, 256, 1, 1),
    (2, 512, 2, 2),      # batch 2: the tiles of every (batch, head) are their own region
    (1, 768, 4, 1),      # GQA 4:1: the dK/dV kernel writes per-query-head partials
    (1, 1280, 4, 2),     # 5 blocks: an odd number of 256-row blocks
]


@pytest.mark.parametrize("keep_ds", [False, True], ids=["recompute", "keep_ds"])
@pytest.mark.parametrize("case", KEEP_DS_CASES, ids=lambda c: "B%d_L%d_H%d_%d" % c)
def test_attention_bwd_kept_ds(case, keep_ds, dev):
    """dQ as one product over the dS tiles that the dK/dV kernel keeps, against the oracle -- and the recomputing
    kernels on the same shapes, which the default setting no longer takes there."""
    from odysseus_transformer_amd import ops
    B, L, Hq, Hkv = case
    print(f"case={case} keep_ds={keep_ds}", flush=True)
    q, k, v, do = _inputs(B, L, L, Hq, Hkv, 128, torch.bfloat16, seed=L + Hq)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=True)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(), causal=True)
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=True)
    dq, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=True, keep_ds=keep_ds)
    assert_parity(dq, dq_ref, TOL_BF16, "dq", 1e-3)
    assert_parity(dk, dk_ref, TOL_BF16, "dk", 1e-3)
    assert_parity(dv, dv_ref, TOL_BF16, "dv")
    # the same dq through the other destinations of the epilogue: an fp32 running sum, a bf16 one, the rotary tables
    acc0 = randn((B, L, Hq, 128), 5).to(dev)
    acc = acc0.clone()
    ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=True, dq=acc, accumulate_dq=True, keep_ds=keep_ds)
    assert_parity((acc - acc0).cpu(), dq_ref, TOL_BF16, "dq added to an fp32 buffer", 1e-3)
    accb = acc0.to(torch.bfloat16)
    ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=True, dq=accb, accumulate_dq=True, keep_ds=keep_ds)
    assert_parity(accb, acc0.to(torch.bfloat16).float().cpu() + dq_ref, TOL_BF16, "dq added to a bf16 buffer")
    pos = torch.arange(L, device=dev).repeat(B, 1)
    table = ops.rope_table(pos, B * L, 128, 10000.0)
    dq_r, dk_r, _ = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=True, rope_tables=(table, table), keep_ds=keep_ds)
    cos, sin = oracle.rope_cos_sin(pos.cpu(), 128, 10000.0)
    assert_parity(dq_r, oracle.apply_rope_bwd(dq_ref, cos, sin), TOL_BF16, "dq rotated back", 1e-3)
    assert_parity(dk_r, oracle.apply_rope_bwd(dk_ref, cos, sin), TOL_BF16, "dk rotated back", 1e-3)


def test_attention_bwd_kept_ds_policy(dev):
    """keep_ds=None takes the kept-dS kernels only within a budget the caller set (or in scratch the arena already
    holds); True on a shape that does not qualify is an error; the C ABI refuses a workspace without room for dS."""
    from odysseus_transformer_amd import ops, _lib
    lib = _lib.load()
    assert lib.ody_attn_bwd_ds_bytes(1, 512, 512, 2, 2, 128, _lib.ODY_BF16, 1) == 2 * 3 * 128 * 1024   # 3 blocks per head
    assert lib.ody_attn_bwd_ds_bytes(1, 512, 768, 2, 2, 128, _lib.ODY_BF16, 0) == 2 * 6 * 128 * 1024   # 2 x 3 blocks
    for args in ((1, 500, 500, 2, 2, 128, _lib.ODY_BF16, 1), (1, 512, 700, 2, 2, 128, _lib.ODY_BF16, 0),
                 (1, 512, 768, 2, 2, 128, _lib.ODY_BF16, 1), (1, 512, 512, 2, 2, 64, _lib.ODY_BF16, 1),
                 (1, 512, 512, 2, 2, 128, _lib.ODY_F32, 1)):
        assert lib.ody_attn_bwd_ds_bytes(*args) == 0, args
    q, k, v, do = (t.to(dev) for t in _inputs(1, 512, 512, 2, 2, 128, torch.bfloat16, seed=3))
    o, lse = ops.attn_fwd(q, k, v, causal=True)

    def kernels(**kw):
        _lib.profile_enable(True)
        try:
            ops.attn_bwd(q, k, v, o, lse, do, causal=True, **kw)
            torch.cuda.synchronize()
            return set(_lib.profile_collect())
        finally:
            _lib.profile_enable(False)

    # opt-in: without a budget the backward recomputes (no dS scratch is taken behind the caller's back)
    assert ops.keep_ds_max_bytes(dev) == 0
    assert "attn_bwd_dq_pipe" in kernels()
    assert "attn_bwd_dq_kept" in kernels(keep_ds=True)
    ops.set_keep_ds_max_bytes(1 << 30)
    try:
        assert "attn_bwd_dq_kept" in kernels()
        ops.set_keep_ds_max_bytes(1 << 10)            # a budget below what this shape needs
        assert "attn_bwd_dq_pipe" in kernels()
    finally:
        ops.set_keep_ds_max_bytes(None)
    # scratch that the arena already holds costs nothing more: used whatever the budget says
    from odysseus_transformer_amd.utils import globals as g
    g._set_global_memory_buffer(dev)
    try:
        assert "attn_bwd_dq_pipe" in kernels()
        g.get_global_memory_buffer().get_tensor((4 << 20,), torch.uint8, "attn_bwd_workspace")
        assert "attn_bwd_dq_kept" in kernels()
    finally:
        g._destroy_global_memory_buffer()
    with pytest.raises(ValueError):
        ops.attn_bwd(q[:, :500], k[:, :500], v[:, :500], o[:, :500], lse[:, :, :500].contiguous(), do[:, :500],
                     causal=True, keep_ds=True)
    small = ops.attn_bwd_workspace(q, k)
    with pytest.raises(ValueError):
        ops.attn_bwd(q, k, v, o, lse, do, causal=True, workspace=small, keep_ds=True)


@pytest.mark.parametrize("case", [(1, 512, 768, 2, 2), (2, 768, 256, 4, 2), (1, 256, 1024, 4, 1)],
                         ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d" % c)
def test_attention_bwd_kept_ds_full_blocks(case, dev):
    """Kept dS for a fully visible block of keys (a ring step): any whole number of 256-row blocks on either side,
    and the running fp32 dq that such a step adds into."""
    from odysseus_transformer_amd import ops
    B, Lq, Lk, Hq, Hkv = case
    print(f"case={case}", flush=True)
    q, k, v, do = _inputs(B, Lq, Lk, Hq, Hkv, 128, torch.bfloat16, seed=Lq + Lk)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=False)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(), causal=False)
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=False)
    acc0 = randn((B, Lq, Hq, 128), 6).to(dev)
    acc = acc0.clone()
    _, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=False, dq=acc, accumulate_dq=True, keep_ds=True)
    assert_parity((acc - acc0).cpu(), dq_ref, TOL_BF16, "dq added to an fp32 buffer", 1e-3)
    assert_parity(dk, dk_ref, TOL_BF16, "dk", 1e-3)
    assert_parity(dv, dv_ref, TOL_BF16, "dv")
    dq2, dk2, dv2 = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=False, keep_ds=False)
    assert torch.equal(dk2, dk) and torch.equal(dv2, dv)
    assert_parity(dq2, dq_ref, TOL_BF16, "dq of the recomputing kernel", 1e-3)


@pytest.mark.parametrize("case", [(1, 4096, 512, 2, 2, False, True, False), (1, 512, 4096, 2, 2, False, False, True),
                                  (1, 4096, 4096, 2, 1, True, True, True), (1, 4096, 4096, 2, 2, True, True, True),
                                  (1, 4100, 600, 2, 2, False, True, False), (2, 2304, 2304, 1, 1, True, True, True),
                                  (1, 500, 4200, 2, 1, False, True, True), (1, 4100, 4100, 2, 2, True, True, True)],
                         ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_c%d_kv%d_q%d" % c)
def test_attention_bwd_range_parts(case, dev):
    """Few key blocks against many queries, or few query blocks against many keys (the steps of a ring over short
    blocks): the dK/dV kernel cuts each block's query range, the dQ kernel over kept dS each block's key range, into
    parts that leave fp32 partial sums, and a second kernel adds them up.  Every destination of dq, against the oracle."""
    from odysseus_transformer_amd import ops, _lib
    B, Lq, Lk, Hq, Hkv, causal, kv_parts, q_parts = case
    print(f"range parts case={case}", flush=True)
    keep = Lq % 256 == 0 and Lk % 256 == 0
    q, k, v, do = _inputs(B, Lq, Lk, Hq, Hkv, 128, torch.bfloat16, seed=Lq + 3 * Lk)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(), causal=causal)
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=causal)
    _lib.profile_enable(True)
    try:
        dq, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, keep_ds=keep)
        torch.cuda.synchronize()
        ran = set(_lib.profile_collect())
    finally:
        _lib.profile_enable(False)
    assert ("attn_bwd_group_sum" in ran) == kv_parts and ("attn_bwd_dq_sum" in ran) == q_parts, ran
    assert_parity(dq, dq_ref, TOL_BF16, "dq", 1e-3)
    assert_parity(dk, dk_ref, TOL_BF16, "dk", 1e-3)
    assert_parity(dv, dv_ref, TOL_BF16, "dv")
    # the partial sums do not depend on the order in which the blocks ran
    dq_b, dk_b, dv_b = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, keep_ds=keep)
    assert torch.equal(dq_b, dq) and torch.equal(dk_b, dk) and torch.equal(dv_b, dv)
    if keep:   # the recomputing dQ kernel cuts its key range the same way; dK / dV do not depend on which dQ kernel runs
        _lib.profile_enable(True)
        try:
            dq_r, dk_r, dv_r = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, keep_ds=False)
            torch.cuda.synchronize()
            ran = set(_lib.profile_collect())
        finally:
            _lib.profile_enable(False)
        assert "attn_bwd_dq_pipe" in ran and ("attn_bwd_dq_sum" in ran) == q_parts, ran
        assert torch.equal(dk_r, dk) and torch.equal(dv_r, dv)
        assert_parity(dq_r, dq_ref, TOL_BF16, "dq of the recomputing kernel", 1e-3)
    acc0 = randn((B, Lq, Hq, 128), 5).to(dev)
    acc = acc0.clone()
    ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, dq=acc, accumulate_dq=True, keep_ds=keep)
    assert_parity((acc - acc0).cpu(), dq_ref, TOL_BF16, "dq added to an fp32 buffer", 1e-3)
    accb = acc0.to(torch.bfloat16)
    ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, dq=accb, accumulate_dq=True, keep_ds=keep)
    assert_parity(accb, acc0.to(torch.bfloat16).float().cpu() + dq_ref, TOL_BF16, "dq added to a bf16 buffer")
    pos_q = (torch.arange(Lq, device=dev) + (Lk - Lq if causal else 0)).repeat(B, 1)
    pos_k = torch.arange(Lk, device=dev).repeat(B, 1)
    tq, tk = ops.rope_table(pos_q, B * Lq, 128, 10000.0), ops.rope_table(pos_k, B * Lk, 128, 10000.0)
    dq_r, dk_r, _ = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, rope_tables=(tq, tk), keep_ds=keep)
    cq, sq = oracle.rope_cos_sin(pos_q.cpu(), 128, 10000.0)
    ck, sk = oracle.rope_cos_sin(pos_k.cpu(), 128, 10000.0)
    assert_parity(dq_r, oracle.apply_rope_bwd(dq_ref, cq, sq), TOL_BF16, "dq rotated back", 1e-3)
    assert_parity(dk_r, oracle.apply_rope_bwd(dk_ref, ck, sk), TOL_BF16, "dk rotated back", 1e-3)


@pytest.mark.parametrize("case", [(1, 512, 4096, 2, 2, 4, False), (1, 300, 2100, 4, 1, 4, False), (2, 256, 1100, 2, 2, 2, False),
                                  (1, 2048, 1024, 4, 4, 2, False), (1, 2048, 2048, 4, 4, 4, True), (1, 1100, 1500, 2, 1, 2, True)],
                         ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_parts%d_c%d" % c)
def test_attention_fwd_key_split(case, dev):
    """Few query blocks (the steps of a ring over 16384-token chunks): the forward cuts every block's key range into
    parts, one block per (query block, part), and merges them.  Same (out, lse) as the oracle, the overflow fallback
    still reaches the blocks it must, and a workspace without room for the parts gives the unsplit result."""
    from odysseus_transformer_amd import ops, _lib
    B, Lq, Lk, Hq, Hkv, parts, causal = case
    D = 128
    print(f"key split case={case}", flush=True)
    lib = _lib.load()
    with_parts = lib.ody_attn_fwd_workspace_bytes(B, Lq, Lk, Hq, Hkv, D, _lib.ODY_BF16)
    per_part = ((B * Lq * Hq * D * 4 + 255) & ~255) + ((B * Hq * Lq * 4 + 255) & ~255)
    unsplit = ((B * Hq * ((Lq + 255) // 256) * 4 + 255) & ~255) + B * Hkv * ((Lk + 63) // 64) * 16384
    assert with_parts >= unsplit + parts * (per_part - 512), "the workspace query leaves no room for the parts"
    q, k, v, _ = _inputs(B, Lq, Lk, Hq, Hkv, D, torch.bfloat16, seed=23)

    def unsplit_fwd(qg, kg, vg):
        """through the C ABI with a workspace that has room for the flags and the V images only"""
        out = torch.empty_like(qg)
        lse = torch.empty((B, Hq, Lq), dtype=torch.float32, device=dev)
        ws = torch.empty(unsplit, dtype=torch.uint8, device=dev)
        _lib.call("ody_attn_fwd", qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), out.data_ptr(), lse.data_ptr(), B, Lq, Lk, Hq,
                  Hkv, D, *ops._blhd(qg, "q"), *ops._blhd(kg, "k"), *ops._blhd(vg, "v"), *ops._blhd(out, "out"),
                  1.0 / math.sqrt(D), int(causal), _lib.ODY_BF16, ws.data_ptr(), unsplit, torch.cuda.current_stream().cuda_stream)
        return out, lse

    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal)
    qg, kg, vg = (t.to(dev) for t in (q, k, v))
    _lib.profile_enable(True)
    try:
        o, lse = ops.attn_fwd(qg, kg, vg, causal=causal)
        torch.cuda.synchronize()
        assert "attn_fwd_split_merge" in _lib.profile_collect()
        o2, lse2 = unsplit_fwd(qg, kg, vg)
        torch.cuda.synchronize()
        assert "attn_fwd_split_merge" not in _lib.profile_collect()
    finally:
        _lib.profile_enable(False)
    assert_parity(o, o_ref, TOL_BF16, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    assert_parity(o2, o_ref, TOL_BF16, "o unsplit")
    assert rel_err(o, o2.float()) <= 1e-2 and torch.allclose(lse, lse2, atol=1e-4, rtol=1e-4)
    # late keys far above the early ones: the parts' references differ, and the blocks that overflow are redone
    q[:, :, 0], k[:, :, 0] = 2.0, -4.0
    k[:, Lk // 2 + 40:Lk // 2 + 60, 0] = 4.0
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal)
    o, lse = ops.attn_fwd(q.to(dev), k.to(dev), vg, causal=causal)
    assert_parity(o, o_ref, TOL_BF16, "o with late large scores")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("case", [(1, 300, 300, 4, 2, 128, True), (2, 257, 700, 2, 2, 128, False), (1, 1100, 1100, 4, 1, 128, True),
                                  (1, 200, 330, 4, 4, 64, True), (1, 96, 96, 2, 1, 64, False)],
                         ids=lambda c: "B%d_Lq%d_Lk%d_H%d_%d_D%d_c%d" % c)
def test_attention_dropout_fwd_bwd(case, dtype, dev):
    """Attention dropout (the dropout_p the reference hands to its attention routine, decoder/odysseus.py:228): the
    kernels evaluate the same counter hash as the oracle, so with the same seed they must agree entry for entry;
    lse is that of the undropped softmax; dropout_p = 0 is the ordinary call."""
    from odysseus_transformer_amd import ops
    B, Lq, Lk, Hq, Hkv, D, causal = case
    print(f"dropout case={case} {dtype}", flush=True)
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    pdrop, seed = 0.2, 0x9E3779B97F4A7C15 + Lq
    q, k, v, do = _inputs(B, Lq, Lk, Hq, Hkv, D, dtype, seed=11 + Lq)
    o_ref, lse_ref = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal, dropout_p=pdrop, seed=seed)
    dq_ref, dk_ref, dv_ref = oracle.attention_bwd(q.float(), k.float(), v.float(), o_ref, lse_ref, do.float(), causal=causal,
                                                  dropout_p=pdrop, seed=seed)
    o_plain, _ = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal)
    assert rel_err(o_ref, o_plain) > 0.1                     # the mask does something
    qg, kg, vg, dog = (t.to(dev) for t in (q, k, v, do))
    o, lse = ops.attn_fwd(qg, kg, vg, causal=causal, dropout_p=pdrop, seed=seed)
    dq, dk, dv = ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, dropout_p=pdrop, seed=seed)
    assert_parity(o, o_ref, tol, "o")
    assert torch.allclose(lse.cpu(), lse_ref, atol=TOL_LSE, rtol=TOL_LSE)
    assert_parity(dq, dq_ref, tol, "dq", 1e-3)
    assert_parity(dk, dk_ref, tol, "dk", 1e-3)
    assert_parity(dv, dv_ref, tol, "dv", 1e-3)
    # another seed is another mask; the running fp32 dq of a ring step takes the dropout path too
    o2, _ = ops.attn_fwd(qg, kg, vg, causal=causal, dropout_p=pdrop, seed=seed + 1)
    assert rel_err(o2, o.float().cpu()) > 0.1
    acc0 = randn((B, Lq, Hq, D), 5).to(dev)
    acc = acc0.clone()
    ops.attn_bwd(qg, kg, vg, o, lse, dog, causal=causal, dq=acc, accumulate_dq=True, dropout_p=pdrop, seed=seed)
    assert_parity((acc - acc0).cpu(), dq_ref, 4 * tol if dtype == torch.float32 else tol, "dq added to an fp32 buffer", 1e-3)
    # through autograd, with the seed drawn from torch's generator
    qa, ka, va = (t.clone().requires_grad_(True) for t in (qg, kg, vg))
    torch.manual_seed(77)
    drawn = int(torch.randint(0, 1 << 62, (1,)).item())
    torch.manual_seed(77)
    oa = ops.flash_attn_func(qa, ka, va, pdrop, causal=causal)
    oa.backward(dog)
    o3, lse3 = oracle.attention_fwd(q.float(), k.float(), v.float(), causal=causal, dropout_p=pdrop, seed=drawn)
    dq3, dk3, dv3 = oracle.attention_bwd(q.float(), k.float(), v.float(), o3, lse3, do.float(), causal=causal, dropout_p=pdrop, seed=drawn)
    assert_parity(oa, o3, tol, "o through autograd")
    assert_parity(qa.grad, dq3, tol, "dq through autograd", 1e-3)
    assert_parity(ka.grad, dk3, tol, "dk through autograd", 1e-3)
    assert_parity(va.grad, dv3, tol, "dv through autograd", 1e-3)


def test_attention_dropout_errors(dev):
    from odysseus_transformer_amd import ops, _lib
    q, k, v, do = (t.to(dev) for t in _inputs(1, 256, 256, 2, 2, 128, torch.bfloat16, seed=3))
    with pytest.raises(ValueError):
        ops.attn_fwd(q, k, v, dropout_p=0.1)                   # no seed
    with pytest.raises(ValueError):
        ops.attn_fwd(q, k, v, dropout_p=1.0, seed=1)
    o, lse = ops.attn_fwd(q, k, v, dropout_p=0.1, seed=1)
    with pytest.raises(ValueError):
        ops.attn_bwd(q, k, v, o, lse, do, dropout_p=0.1, seed=1, keep_ds=True)
    with pytest.raises(_lib.OdysseusHipError) as e:               # the C ABI checks the probability itself
        _lib.call("ody_attn_fwd_dropout", q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), 1, 256, 256, 2, 2, 128,
                  *ops._blhd(q, "q"), *ops._blhd(k, "k"), *ops._blhd(v, "v"), *ops._blhd(o, "o"), 0.088, 1, _lib.ODY_BF16, 0, 0, 0,
                  1.5, 1)
    assert e.value.code == -1
    o0, lse0 = ops.attn_fwd(q, k, v, dropout_p=0.0)
    o1, lse1 = ops.attn_fwd(q, k, v)
    assert torch.equal(o0, o1) and torch.equal(lse0, lse1)
