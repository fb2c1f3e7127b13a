"""The one-pass AdamW (ody_adamw behind odysseus_transformer_amd.optim.AdamW) against the oracle's step and against
torch.optim.AdamW: trajectories over several steps, odd lengths, both dtypes, interchangeable state dicts."""
import copy

import pytest
import torch

from conftest import rel_err
import odysseus_oracle as oracle

pytestmark = pytest.mark.gpu
HP = dict(lr=2e-3, betas=(0.9, 0.98), eps=1e-8, weight_decay=0.05)


@pytest.mark.parametrize("n", [13, 4096, 1000003])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_adamw_trajectory_against_the_oracle(n, dtype, dev):
    from odysseus_transformer_amd.optim import AdamW
    g = torch.Generator().manual_seed(n)
    p0 = torch.randn(n, generator=g).to(dtype)
    grads = [(torch.randn(n, generator=g) * (0.1 + s)).to(dtype) for s in range(4)]
    param = torch.nn.Parameter(p0.to(dev))
    opt = AdamW([param], **HP)
    p, m, v = p0.clone(), torch.zeros(n, dtype=dtype), torch.zeros(n, dtype=dtype)
    for step, gr in enumerate(grads, 1):
        param.grad = gr.to(dev)
        opt.step()
        # the oracle on the values the kernel saw (its stored state), rounded once to the storage type like the kernel's
        pf, mf, vf = oracle.adamw_step(p.float(), gr.float(), m.float(), v.float(), step, **HP)
        p, m, v = pf.to(dtype), mf.to(dtype), vf.to(dtype)
        st = opt.state[param]
        tol = 1e-6 if dtype == torch.float32 else 8e-3       # one bf16 ulp where a sum lands on a rounding boundary
        assert rel_err(param.detach(), pf) <= tol, (step, rel_err(param.detach(), pf))
        assert rel_err(st["exp_avg"], mf) <= tol and rel_err(st["exp_avg_sq"], vf) <= tol
        # carry the kernel's own stored values forward so that errors do not compound in the comparison
        p, m, v = param.detach().cpu().clone(), st["exp_avg"].cpu().clone(), st["exp_avg_sq"].cpu().clone()
    assert int(st["step"].item()) == len(grads)


def test_adamw_state_interchanges_with_torch(dev):
    """Two steps here, state handed to torch.optim.AdamW (and back): the third step agrees."""
    from odysseus_transformer_amd.optim import AdamW
    g = torch.Generator().manual_seed(77)
    w0 = torch.randn(300, 40, generator=g)
    grads = [torch.randn(300, 40, generator=g) for _ in range(3)]
    a = torch.nn.Parameter(w0.clone().to(dev))
    oa = AdamW([a], **HP)
    for gr in grads[:2]:
        a.grad = gr.to(dev)
        oa.step()
    b = torch.nn.Parameter(a.detach().clone())
    ob = torch.optim.AdamW([b], **HP)
    ob.load_state_dict(copy.deepcopy(oa.state_dict()))     # load_state_dict does not copy tensors that already fit
    a.grad, b.grad = grads[2].to(dev), grads[2].to(dev)
    oa.step()
    ob.step()
    assert rel_err(a.detach(), b.detach().float()) <= 1e-6
    oc = AdamW([torch.nn.Parameter(b.detach().clone())], **HP)
    oc.load_state_dict(copy.deepcopy(ob.state_dict()))
    assert int(oc.state[oc.param_groups[0]["params"][0]]["step"].item()) == 3


def test_adamw_refuses_what_it_cannot_do(dev):
    from odysseus_transformer_amd.optim import AdamW
    with pytest.raises(ValueError):
        AdamW([torch.nn.Parameter(torch.zeros(4))], lr=-1.0)
    p = torch.nn.Parameter(torch.zeros(4))
    p.grad = torch.ones(4)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        AdamW([p]).step()                                  # a CPU parameter: there is no CPU path
    q = torch.nn.Parameter(torch.zeros(8, device=dev))
    AdamW([q]).step()                                      # no gradient yet: nothing to do, no state
