"""The allocation-free forward entry point (ody_attn_fwd_noalloc): same results, bit for bit, as
ody_attn_fwd, from the library's own device-resident scratch; two calls in a row, the second on a
smaller input, so that what the first call left in the shared scratch cannot leak into the second."""
import pytest
import torch

from conftest import randn

pytestmark = pytest.mark.gpu


def _pair(B, Lq, Lk, Hq, Hkv, D, causal, seed, dev, dtype=torch.bfloat16, spike=False):
    from odysseus_transformer_amd import ops
    q = randn((B, Lq, Hq, D), seed, dtype=dtype)
    k = randn((B, Lk, Hkv, D), seed + 1, dtype=dtype)
    v = randn((B, Lk, Hkv, D), seed + 2, dtype=dtype)
    if spike:
        # late keys far above the early ones: the forward flags the query blocks concerned in its
        # scratch and a second kernel redoes them, so the flags of this call are left set
        q[:, :, 0], k[:, :, 0] = 2.0, -4.0
        k[:, Lk // 2:Lk // 2 + 20, 0] = 4.0
    qg, kg, vg = q.to(dev), k.to(dev), v.to(dev)
    ref_o, ref_lse = ops.attn_fwd(qg, kg, vg, causal=causal)
    out = torch.full_like(ref_o, float("nan"))
    lse = torch.full_like(ref_lse, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    ops.attn_fwd_noalloc(qg, kg, vg, out, lse, causal=causal)
    after = torch.cuda.memory_stats()["allocation.all.allocated"]
    torch.cuda.synchronize()
    assert after == before, "the allocation-free entry point went through the caching allocator"
    assert torch.equal(out, ref_o), f"out differs (B={B} Lq={Lq} Lk={Lk} Hq={Hq} Hkv={Hkv} D={D})"
    assert torch.equal(lse, ref_lse), f"lse differs (B={B} Lq={Lq} Lk={Lk} Hq={Hq} Hkv={Hkv} D={D})"


def test_noalloc_forward_matches_the_workspace_entry_point_twice(dev):
    print("noalloc: first call, 1400 keys with flagged blocks", flush=True)
    _pair(1, 1400, 1400, 4, 2, 128, True, 40, dev, spike=True)
    print("noalloc: second call, smaller input", flush=True)
    _pair(1, 333, 333, 4, 2, 128, True, 50, dev)
    print("noalloc: third call, key offset and batch 2", flush=True)
    _pair(2, 200, 520, 4, 1, 128, True, 60, dev)
    print("noalloc: kernels that need no scratch (head_dim 64, fp32)", flush=True)
    _pair(1, 257, 257, 4, 4, 64, True, 70, dev)
    _pair(1, 130, 130, 2, 1, 128, False, 80, dev, dtype=torch.float32)


def test_noalloc_rejects_what_does_not_fit(dev):
    from odysseus_transformer_amd import _lib, ops
    from odysseus_transformer_amd._lib import OdysseusHipError
    L, Hkv = 40000, 4                          # 160000 key rows x 256 bytes > 32 MiB
    need = _lib.load().ody_attn_fwd_workspace_bytes(1, 64, L, 4, Hkv, 128, _lib.ODY_BF16)
    assert need > _lib.ATTN_FWD_NOALLOC_SCRATCH_BYTES
    q = torch.zeros((1, 64, 4, 128), dtype=torch.bfloat16, device=dev)
    k = torch.zeros((1, L, Hkv, 128), dtype=torch.bfloat16, device=dev)
    out, lse = torch.empty_like(q), torch.empty((1, 4, 64), dtype=torch.float32, device=dev)
    with pytest.raises(OdysseusHipError) as e:
        ops.attn_fwd_noalloc(q, k, k, out, lse)
    assert e.value.code == -5 and "scratch" in e.value.msg
    # the largest benchmark shard fits: 4 kv heads x 32768 keys
    assert _lib.load().ody_attn_fwd_workspace_bytes(1, 32768, 32768, 4, 4, 128, _lib.ODY_BF16) \
        <= _lib.ATTN_FWD_NOALLOC_SCRATCH_BYTES
