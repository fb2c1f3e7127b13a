"""The parity metric itself has to be able to fail: a kernel that drops the late part of a long
causal sequence must not pass.  Under a causal mask the rows of out / dq / dk / dv shrink like
1 / sqrt(position), so a relative error normalised by the whole tensor's largest entry is blind
to the bulk of a long sequence; the per-row metric and the sampled checks are not."""
import pytest
import torch

from conftest import TOL_BF16, assert_parity, block_rel_err, randn, rel_err
import odysseus_oracle as oracle
from sampled import edge_samples, sampled_checks


def test_whole_tensor_metric_is_blind_to_a_dropped_half_and_the_block_metric_is_not():
    L, H, D = 32768, 1, 128
    ref = randn((1, L, H, D), 1) / torch.arange(1, L + 1).sqrt()[None, :, None, None]
    broken = ref.clone()
    broken[:, L // 2:] = 0                           # "the kernel never wrote the last half"
    assert rel_err(broken, ref) <= TOL_BF16          # the old bar lets it through
    assert block_rel_err(broken, ref) > 0.5            # the block-wise bar does not
    with pytest.raises(AssertionError):
        assert_parity(broken, ref, TOL_BF16, "dv")
    noisy = (ref.bfloat16()).float()                 # an honest bf16 rounding passes both
    assert_parity(noisy, ref, TOL_BF16, "rounded")


def test_block_metric_keeps_zero_blocks_from_blowing_up_and_forgives_one_ill_conditioned_row():
    ref = torch.zeros(256, 8)
    ref[:64] = 1.0
    a = ref + 1e-6
    assert block_rel_err(a, ref) < 1e-2 and rel_err(a, ref) < 1e-5
    ref = torch.ones(256, 8)
    ref[100] = 1e-3                       # a row that is small by cancellation ...
    a = ref.clone()
    a[100] += 1e-3                        # ... and off by 100 % of itself, 0.1 % of its neighbours
    assert block_rel_err(a, ref) <= 2e-3
    a[64:128] = 0                         # a whole missing block is not forgiven
    assert block_rel_err(a, ref) > 0.5


@pytest.mark.parametrize("which", ["dv", "dk", "dq", "out", "lse"])
def test_sampled_checks_catch_a_dropped_half(which):
    """The oracle's own results pass the sampled checks; the same results with the last half of
    one tensor zeroed (or the lse shifted there) do not."""
    L, Hq, Hkv, D = 2048, 2, 1, 128
    q, do = randn((1, L, Hq, D), 11), randn((1, L, Hq, D), 12)
    k, v = randn((1, L, Hkv, D), 13), randn((1, L, Hkv, D), 14)
    o, lse = oracle.attention_fwd(q, k, v, causal=True)
    dq, dk, dv = oracle.attention_bwd(q, k, v, o, lse, do, causal=True)
    rows, cols = edge_samples(L, 4, 1), edge_samples(L, 4, 2)
    args = lambda t: (q[0], k[0], v[0], do[0], t["out"][0], t["lse"][0], t["dq"][0], t["dk"][0], t["dv"][0],
                      True, rows, cols)
    good = {"out": o, "lse": lse, "dq": dq, "dk": dk, "dv": dv}
    if which == "dv":                                # run the passing case once
        sampled_checks(*args(good), tol=1e-3)
    bad = {n: t.clone() for n, t in good.items()}
    if which == "lse":
        bad["lse"][:, :, L // 2:] += 0.01
    else:
        bad[which][:, L // 2:] = 0
    with pytest.raises(AssertionError):
        sampled_checks(*args(bad), tol=TOL_BF16)
