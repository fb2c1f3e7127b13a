"""Size-independent parity checks for attention results too long for a whole-result oracle run:
brute-force fp64 recomputation of sampled query rows (lse, out, dq) and key columns (dk, dv)
over the full length, plus checksums that hold for any input."""
import math

import torch

from conftest import TOL_BF16, TOL_LSE, rel_err

F64 = torch.float64


def sampled_checks(q, k, v, do, o, lse, dq, dk, dv, causal, rows, cols, tol=TOL_BF16):
    """q, do, o, dq: (L, Hq, D); k, v, dk, dv: (Lk, Hkv, D); lse: (Hq, L) -- CPU tensors.
    Causal masking is bottom-right aligned: query i sees keys j <= i + (Lk - Lq)."""
    Lq, Hq, D = q.shape
    Lk, Hkv, _ = k.shape
    grp, off, scale = Hq // Hkv, Lk - Lq, 1.0 / math.sqrt(D)
    rows, cols = torch.as_tensor(rows), torch.as_tensor(cols)
    jj, ii = torch.arange(Lk), torch.arange(Lq)
    for h in range(Hq):
        g = h // grp
        kd, vd = k[:, g].to(F64), v[:, g].to(F64)
        # ---- sampled query rows: lse, out, dq
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
        assert rel_err(o[rows, h], o_ref) <= tol, f"out head {h}"
        assert rel_err(dq[rows, h], dq_ref) <= tol, f"dq head {h}"
    for g in range(Hkv):
        dk_ref = torch.zeros((len(cols), D), dtype=F64)
        dv_ref = torch.zeros((len(cols), D), dtype=F64)
        for h in range(g * grp, (g + 1) * grp):
            # ---- sampled key columns: dk, dv (row statistics lse and delta taken from the
            # device results, which the row samples above vouch for)
            qd, dod = q[:, h].to(F64), do[:, h].to(F64)
            s = (qd @ k[cols, g].to(F64).T) * scale
            p = torch.exp(s - lse[h].to(F64)[:, None])
            if causal:
                p = p.masked_fill(cols[None, :] > ii[:, None] + off, 0.0)
            delta = (dod * o[:, h].to(F64)).sum(-1, keepdim=True)
            ds = p * (dod @ v[cols, g].to(F64).T - delta)
            dv_ref += p.T @ dod
            dk_ref += (ds.T @ qd) * scale
        assert rel_err(dv[cols, g], dv_ref) <= tol, f"dv kv-head {g}"
        assert rel_err(dk[cols, g], dk_ref) <= tol, f"dk kv-head {g}"
        # ---- checksums over every key: rows of P sum to one, rows of dS sum to zero
        hs = slice(g * grp, (g + 1) * grp)
        sum_do = do[:, hs].to(F64).sum((0, 1))
        sum_dv = dv[:, g].to(F64).sum(0)
        assert (sum_dv - sum_do).abs().max() <= tol * sum_do.abs().max(), f"sum dv kv-head {g}"
        bound = tol * dk[:, g].to(F64).abs().sum(0).max()
        assert dk[:, g].to(F64).sum(0).abs().max() <= bound, f"sum dk kv-head {g}"


def edge_samples(L, n_mid, seed):
    g = torch.Generator().manual_seed(seed)
    mid = torch.randint(0, L, (n_mid,), generator=g).tolist()
    edges = [0, 1, 31, 32, 63, 64, 127, 128, 255, 256, 257, L // 2 - 1, L // 2, L - 257, L - 256, L - 2, L - 1]
    return sorted(set(x for x in edges + mid if 0 <= x < L))
