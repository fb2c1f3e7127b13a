"""Size-independent parity checks for attention results too long for a whole-result backward on the
CPU: the oracle's forward over the whole sequence (every lse and out row), brute-force fp64
recomputation of sampled query rows (lse, out, dq) and key columns (dk, dv) over the full length,
plus checksums that hold for any input.  Samples are runs of RUN consecutive positions, and every
run is held to the tolerance on its own scale (the block-wise metric of conftest.py with the run
as the block); nothing the references are built from comes from the device."""
import math

import torch

from conftest import TOL_BF16, TOL_LSE, assert_parity, block_rel_err
import odysseus_oracle as oracle

F64 = torch.float64
RUN = 4          # consecutive positions per sample


def oracle_forward(q, k, v, causal, progress=None):
    """The oracle's fp32 forward, one query head at a time: out (L, Hq, D), lse (Hq, L)."""
    Lq, Hq, D = q.shape
    grp = Hq // k.shape[1]
    o_ref = torch.empty((Lq, Hq, D), dtype=torch.float32)
    lse_ref = torch.empty((Hq, Lq), dtype=torch.float32)
    for h in range(Hq):
        g = h // grp
        o, l = oracle.attention_fwd(q[None, :, h:h + 1].float(), k[None, :, g:g + 1].float(),
                                    v[None, :, g:g + 1].float(), causal=causal)
        o_ref[:, h], lse_ref[h] = o[0, :, 0], l[0, 0]
        if progress:
            print(f"  {progress}: oracle forward, head {h + 1}/{Hq}", flush=True)
    return o_ref, lse_ref


def sampled_checks(q, k, v, do, o, lse, dq, dk, dv, causal, rows, cols, tol=TOL_BF16, progress=None):
    """q, do, o, dq: (L, Hq, D); k, v, dk, dv: (Lk, Hkv, D); lse: (Hq, L) -- CPU tensors.
    Causal masking is bottom-right aligned: query i sees keys j <= i + (Lk - Lq)."""
    Lq, Hq, D = q.shape
    Lk, Hkv, _ = k.shape
    grp, off, scale = Hq // Hkv, Lk - Lq, 1.0 / math.sqrt(D)
    rows, cols = torch.as_tensor(rows), torch.as_tensor(cols)
    jj, ii = torch.arange(Lk), torch.arange(Lq)
    # ---- every row of the forward against the oracle's forward
    o_ref_all, lse_ref_all = oracle_forward(q, k, v, causal, progress)
    assert torch.allclose(lse.float(), lse_ref_all, atol=TOL_LSE, rtol=TOL_LSE), "lse (all rows)"
    assert_parity(o, o_ref_all, tol, "out (all rows)")
    for h in range(Hq):
        g = h // grp
        kd, vd = k[:, g].to(F64), v[:, g].to(F64)
        # ---- sampled query rows in fp64: lse, out, dq
        s = (q[rows, h].to(F64) @ kd.T) * scale
        if causal:
            s = s.masked_fill(jj[None, :] > rows[:, None] + off, float("-inf"))
        l_ref = torch.logsumexp(s, -1)
        p = torch.exp(s - l_ref[:, None])
        o_ref = p @ vd
        dod = do[rows, h].to(F64)
        ds = p * (dod @ vd.T - (dod * o_ref).sum(-1, keepdim=True))
        dq_ref = (ds @ kd) * scale
        assert torch.allclose(lse[h, rows].to(F64), l_ref, atol=TOL_LSE, rtol=TOL_LSE), f"lse head {h}"
        assert torch.allclose(lse_ref_all[h, rows].to(F64), l_ref, atol=1e-4, rtol=1e-4), f"oracle lse head {h}"
        assert block_rel_err(o[rows, h], o_ref, block=RUN) <= tol, f"out head {h}"
        assert block_rel_err(dq[rows, h], dq_ref, block=RUN) <= tol, f"dq head {h}"
    for g in range(Hkv):
        dk_ref = torch.zeros((len(cols), D), dtype=F64)
        dv_ref = torch.zeros((len(cols), D), dtype=F64)
        for h in range(g * grp, (g + 1) * grp):
            # ---- sampled key columns: dk, dv, with the row statistics (lse, delta) of the
            # oracle's forward, not the device's
            qd, dod = q[:, h].to(F64), do[:, h].to(F64)
            s = (qd @ k[cols, g].to(F64).T) * scale
            p = torch.exp(s - lse_ref_all[h].to(F64)[:, None])
            if causal:
                p = p.masked_fill(cols[None, :] > ii[:, None] + off, 0.0)
            delta = (dod * o_ref_all[:, h].to(F64)).sum(-1, keepdim=True)
            ds = p * (dod @ v[cols, g].to(F64).T - delta)
            dv_ref += p.T @ dod
            dk_ref += (ds.T @ qd) * scale
        assert block_rel_err(dv[cols, g], dv_ref, block=RUN) <= tol, f"dv kv-head {g}"
        assert block_rel_err(dk[cols, g], dk_ref, block=RUN) <= tol, f"dk kv-head {g}"
        # ---- checksums over every key: rows of P sum to one, rows of dS sum to zero
        hs = slice(g * grp, (g + 1) * grp)
        sum_do = do[:, hs].to(F64).sum((0, 1))
        sum_dv = dv[:, g].to(F64).sum(0)
        assert (sum_dv - sum_do).abs().max() <= tol * sum_do.abs().max(), f"sum dv kv-head {g}"
        bound = tol * dk[:, g].to(F64).abs().sum(0).max()
        assert dk[:, g].to(F64).sum(0).abs().max() <= bound, f"sum dk kv-head {g}"
    return o_ref_all, lse_ref_all


def edge_samples(L, n_mid, seed):
    """Runs of RUN consecutive positions starting at tile edges at both ends of the sequence, its
    middle, one per sixteenth and `n_mid` random places; returned flat, run after run."""
    g = torch.Generator().manual_seed(seed)
    mid = torch.randint(0, L, (n_mid,), generator=g).tolist()
    edges = [0, 29, 61, 125, 253, L // 2 - 2, L - 259, L - RUN]
    seg = [(s * L) // 16 + int(torch.randint(0, max(L // 16, 1), (1,), generator=g)) for s in range(16)]
    starts = sorted(set(min(max(x, 0), max(L - RUN, 0)) for x in edges + mid + seg))
    return [x + r for x in starts for r in range(min(RUN, L))]
