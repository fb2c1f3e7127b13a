"""GPU parity: the three products of a linear layer through ody_gemm vs. the CPU oracle."""
import pytest
import torch

from conftest import TOL_BF16, TOL_F32, randn, rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu

SHAPES = [
    # M, N, K
    (64, 64, 64),
    (256, 256, 256),
    (128, 128, 64),        # interior tiles, a single K slab
    (256, 384, 192),       # interior tiles, odd number of K slabs
    (300, 136, 72),        # ragged in every direction (multiples of 8)
    (2048, 1536, 512),     # the fp32 configuration's QKV projection
    (520, 2752, 512),      # gate_up of the fp32 configuration, ragged M
    (1024, 768, 4096),
    (4096, 4096, 512),     # enough tiles for the 256 x 256 kernel
    (1000, 1096, 256),     # whole tiles plus a ragged strip on the right and at the bottom
    (4104, 3848, 128),     # the same with 256 x 256 tiles
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "M%d_N%d_K%d" % s)
def test_linear_fwd_dgrad_wgrad(shape, dtype, dev):
    from odysseus_transformer_amd import ops
    M, N, K = shape
    print(f"shape={shape} dtype={dtype}", flush=True)
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    x = randn((M, K), 1, dtype=dtype)
    w = randn((N, K), 2, std=0.02, dtype=dtype)
    dy = randn((M, N), 3, dtype=dtype)
    y_ref = oracle.linear_fwd(x.float(), w.float())
    dx_ref, dw_ref, _ = oracle.linear_bwd(x.float(), w.float(), dy.float())
    xg, wg, dyg = x.to(dev), w.to(dev), dy.to(dev)
    y = ops.gemm(ops.GEMM_NT, xg, wg)              # X W^T
    dx = ops.gemm(ops.GEMM_NN, dyg, wg)            # dY W
    dw = ops.gemm(ops.GEMM_TN, dyg, xg)            # dY^T X
    torch.cuda.synchronize()
    assert rel_err(y, y_ref) <= tol, "fwd"
    assert rel_err(dx, dx_ref) <= tol, "dgrad"
    assert rel_err(dw, dw_ref) <= tol, "wgrad"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_bias_accumulate_and_strides(dtype, dev):
    from odysseus_transformer_amd import ops
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    M, N, K = 200, 264, 136
    x = randn((M, K + 24), 4, dtype=dtype)[:, 8:8 + K]          # row stride > K, offset start
    w = randn((N, K), 5, std=0.05, dtype=dtype)
    b = randn((N,), 6, dtype=dtype)
    c0 = randn((M, N), 7, dtype=dtype)
    ref = oracle.linear_fwd(x.float(), w.float(), b.float()) + c0.float()
    xg = randn((M, K + 24), 4, dtype=dtype).to(dev)[:, 8:8 + K]
    out = c0.to(dev).clone()
    ops.gemm(ops.GEMM_NT, xg, w.to(dev), bias=b.to(dev), out=out, accumulate=True)
    assert rel_err(out, ref) <= tol


@pytest.mark.parametrize("op", ["nt", "nn", "tn"])
def test_bias_accumulate_and_strides_on_interior_tiles(op, dev):
    """The kernel for full tiles: padded leading dimensions, bias and accumulation into C."""
    from odysseus_transformer_amd import ops
    dt = torch.bfloat16
    M, N, K = 512, 256, 320
    shape_a = {"nt": (M, K), "nn": (M, K), "tn": (K, M)}[op]
    shape_b = {"nt": (N, K), "nn": (K, N), "tn": (K, N)}[op]
    a = randn((shape_a[0], shape_a[1] + 40), 11, dtype=dt)[:, 16:16 + shape_a[1]]
    b = randn((shape_b[0], shape_b[1] + 8), 12, std=0.05, dtype=dt)[:, :shape_b[1]]
    bias = randn((N,), 13, dtype=dt)
    c0 = randn((M, N + 16), 14, dtype=dt)[:, 8:8 + N]
    af = a.float().t() if op == "tn" else a.float()
    bf = b.float().t() if op == "nt" else b.float()
    ref = af @ bf + bias.float() + c0.float()
    ag = randn((shape_a[0], shape_a[1] + 40), 11, dtype=dt).to(dev)[:, 16:16 + shape_a[1]]
    bg = randn((shape_b[0], shape_b[1] + 8), 12, std=0.05, dtype=dt).to(dev)[:, :shape_b[1]]
    out = randn((M, N + 16), 14, dtype=dt).to(dev)[:, 8:8 + N]
    code = {"nt": ops.GEMM_NT, "nn": ops.GEMM_NN, "tn": ops.GEMM_TN}[op]
    ops.gemm(code, ag, bg, bias=bias.to(dev), out=out, accumulate=True)
    assert rel_err(out, ref) <= TOL_BF16


@pytest.mark.parametrize("shape", [(77, 53, 41), (130, 66, 33), (5, 3, 1), (259, 131, 100), (2901, 2903, 37)],
                         ids=lambda s: "M%d_N%d_K%d" % s)
def test_fp32_any_shape_and_alignment(shape, dev):
    """fp32 takes extents that are not multiples of 4 and views that start on odd elements."""
    from odysseus_transformer_amd import ops
    M, N, K = shape
    print(f"shape={shape}", flush=True)
    x = randn((M, K + 3), 21)[:, 1:1 + K]
    w = randn((N, K), 22, std=0.05)
    dy = randn((M, N + 1), 23)[:, 1:]
    b = randn((N,), 24)
    c0 = randn((M, N), 25)
    xg, wg, dyg = randn((M, K + 3), 21).to(dev)[:, 1:1 + K], w.to(dev), randn((M, N + 1), 23).to(dev)[:, 1:]
    out = c0.to(dev).clone()
    ops.gemm(ops.GEMM_NT, xg, wg, bias=b.to(dev), out=out, accumulate=True)
    assert rel_err(out, x @ w.T + b + c0) <= TOL_F32, "fwd"
    assert rel_err(ops.gemm(ops.GEMM_NN, dyg, wg), dy @ w) <= TOL_F32, "dgrad"
    assert rel_err(ops.gemm(ops.GEMM_TN, dyg, xg), dy.T @ x) <= TOL_F32, "wgrad"


def test_linearity_at_full_size(dev):
    """Size-independent property at a rank-shard shape: X (W1 + W2)^T == X W1^T + X W2^T
    up to bf16 rounding, and the wgrad of a row-permuted batch is unchanged."""
    from odysseus_transformer_amd import ops
    M, N, K = 8192, 1536, 4096
    x = randn((M, K), 11, dtype=torch.bfloat16).to(dev)
    w1 = randn((N, K), 12, std=0.02, dtype=torch.bfloat16).to(dev)
    w2 = randn((N, K), 13, std=0.02, dtype=torch.bfloat16).to(dev)
    y12 = ops.gemm(ops.GEMM_NT, x, (w1.float() + w2.float()).bfloat16())
    y1, y2 = ops.gemm(ops.GEMM_NT, x, w1), ops.gemm(ops.GEMM_NT, x, w2)
    assert rel_err(y12, y1.float() + y2.float()) <= TOL_BF16
    dy = randn((M, N), 14, dtype=torch.bfloat16).to(dev)
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(0)).to(dev)
    dw = ops.gemm(ops.GEMM_TN, dy, x)
    dwp = ops.gemm(ops.GEMM_TN, dy[perm].contiguous(), x[perm].contiguous())
    assert rel_err(dwp, dw.float()) <= 5e-3
    # spot check rows against fp64
    rows = torch.tensor([0, 1, 777, M - 1], device=dev)
    ref = x[rows].double() @ w1.double().T
    assert rel_err(y1[rows], ref) <= TOL_BF16


def test_gemm_errors(dev):
    from odysseus_transformer_amd import ops
    from odysseus_transformer_amd._lib import OdysseusHipError
    a = torch.zeros(16, 20, dtype=torch.bfloat16, device=dev)   # K = 20 is not a multiple of 8
    with pytest.raises(OdysseusHipError):
        ops.gemm(ops.GEMM_NT, a, a)
    with pytest.raises(ValueError):
        ops.gemm(ops.GEMM_NT, a, torch.zeros(16, 24, dtype=torch.bfloat16, device=dev))
