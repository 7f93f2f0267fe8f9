"""Writes tests/golden/*.npz from the CPU oracle (oracle/palimpsa_oracle.py).

The reference repository stores no vectors for the operator, so these fixtures are produced by the
oracle after it has been pinned by tests/test_oracle_pins.py.  They freeze (a) the seeded inputs of
the benchmark configurations as this torch build generates them and (b) the oracle's outputs, so that
drift in either shows up as a failing CPU test, and they give the GPU tests a second, stored target.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import layer_glue_oracle as lo  # noqa: E402
from oracle import palimpsa_oracle as po  # noqa: E402


def c0_case():
    """Benchmark configuration 0: B=2, T=256, H=4, dk=dv=32, fp32, seed 0; outputs every 16th token."""
    inp = po.make_inputs(2, 256, 4, 32, 32, seed=0)
    o, _, mu, I = po.palimpsa_recurrence(*[inp[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")])
    return dict(o_every16=o[:, ::16].numpy(), final_mu=mu.numpy(), final_I=I.numpy(),
                q_head=inp["q"][0, :4, 0].numpy(), gt_head=inp["gt"][0, :8].numpy())


def grad_case():
    """Small forward+backward with initial state and uncertainty output, float64 autograd."""
    B, T, H, dk, dv = 1, 70, 2, 16, 16
    inp = po.make_inputs(B, T, H, dk, dv, seed=5, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(6)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(B, H, dv, dk, generator=gen)
    do = torch.randn(B, T, H, dv, generator=gen)
    dov = torch.randn(B, T, H, dv, generator=gen) * 0.3
    names = ["q", "k", "v", "b", "gt", "g", "Ip"]
    leaves = [inp[n].double().requires_grad_(True) for n in names] + [mu0.double().requires_grad_(True),
                                                                      I0.double().requires_grad_(True)]
    o, ov, fmu, fI = po.palimpsa_recurrence(*leaves, scale=0.5, output_uncertainty=True, compute_dtype=torch.float64)
    gr = torch.autograd.grad((o * do.double()).sum() + (ov * dov.double()).sum(), leaves)
    out = {"d" + n: g.numpy() for n, g in zip(names + ["mu0", "I0"], gr)}
    out.update(o=o.detach().numpy(), o_var=ov.detach().numpy(), final_mu=fmu.detach().numpy(),
               final_I=fI.detach().numpy())
    return out


def varlen_case():
    """Packed documents [0,3,70,71,200], H=2, d=32, bf16-rounded rows, float32 oracle."""
    cu = [0, 3, 70, 71, 200]
    inp = po.make_inputs(1, 200, 2, 32, 32, seed=9, dtype=torch.bfloat16)
    o, _, mu, I = po.palimpsa_recurrence(*[inp[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")], cu_seqlens=cu)
    return dict(cu=np.array(cu), o=o.numpy(), final_mu=mu.numpy(), final_I=I.numpy())


def gla_inputs():
    """Seeded inputs of the case without the precision state: B=1, T=90, H=2, dk=32, dv=48, bf16-rounded rows."""
    B, T, H, dk, dv = 1, 90, 2, 32, 48
    gen = torch.Generator().manual_seed(21)
    q = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1).bfloat16()
    v = torch.randn(B, T, H, dv, generator=gen).bfloat16()
    g = -torch.nn.functional.softplus(torch.randn(B, T, H, generator=gen)) * torch.tensor([0.1, 1.5])
    S0 = torch.randn(B, H, dk, dv, generator=gen) * 0.2
    do = torch.randn(B, T, H, dv, generator=gen)
    return q, k, v, g, S0, do


def gla_case():
    """Scalar-gated linear attention = the Palimpsa recurrence with b = 0, Ip = 1, gt = -g, unit rate (I stays 1, so
    mu = M): outputs, final state and all gradients from the float64 oracle by autograd."""
    q, k, v, g, S0, do = gla_inputs()
    H = q.shape[2]
    leaves = [x.double().requires_grad_(True) for x in (q, k, v, g, S0)]
    ones = torch.ones(H, dtype=torch.float64)
    mu0 = leaves[4].transpose(-1, -2)                       # the oracle keeps the state as [N,H,dv,dk]
    o, _, fmu, _ = po.palimpsa_recurrence(leaves[0], leaves[1], leaves[2], torch.zeros_like(leaves[2]), -leaves[3], ones, ones,
                                          mu0, torch.ones_like(mu0), scale=0.25, compute_dtype=torch.float64)
    gr = torch.autograd.grad((o * do.double()).sum(), leaves)
    out = {"d" + n: x.numpy() for n, x in zip(("q", "k", "v", "g", "S0"), gr)}
    out.update(o=o.detach().numpy(), final_state=fmu.detach().transpose(-1, -2).contiguous().numpy())
    return out


def glue_inputs():
    lead, Hqk, H, dk, dv = (1, 13), 2, 4, 16, 24
    gen = torch.Generator().manual_seed(31)
    r = lambda *s: torch.randn(*s, generator=gen)
    a = dict(q_raw=r(*lead, Hqk, dk), k_raw=r(*lead, Hqk, dk), x=r(*lead, H, dv), dt_raw=r(*lead, H) - 1.0,
             dt_bias=r(H), bs_raw=r(*lead, H), b_raw=r(*lead, H, dv), b_scale=r(H) + 1.0)
    for n in ("q_raw", "k_raw", "x", "dt_raw", "bs_raw", "b_raw"):
        a[n] = a[n].bfloat16()
    extra = dict(o=r(*lead, H, dv).bfloat16(), gate=r(*lead, H, dv).bfloat16(), D=r(H), weight=1.0 + 0.2 * r(dv),
                 dy=r(*lead, H, dv).bfloat16())
    wts = [r(*lead, H, dk), r(*lead, H, dk), r(*lead, H, dv), r(*lead, H, dv), r(*lead, H)]
    return a, extra, wts


def glue_case():
    """Layer glue either side of the operator (oracle/layer_glue_oracle.py), bf16-rounded inputs, float64:
    prologue outputs and the gradients of sum(output * weight); epilogue output and gradients."""
    a, extra, wts = glue_inputs()
    names = list(a)
    leaves = {n: a[n].double().requires_grad_(True) for n in names}
    outs = lo.prologue(**leaves, model_dtype=torch.bfloat16)
    loss = sum((y * w.double()).sum() for y, w in zip(outs, wts))
    gr = torch.autograd.grad(loss, [leaves[n] for n in names])
    out = {"pro_" + n: y.detach().numpy() for n, y in zip(("q", "k", "v", "b", "gt"), outs)}
    out.update({"pro_d" + n: x.numpy() for n, x in zip(names, gr)})
    ev = [extra["o"], a["x"], extra["D"], extra["gate"], extra["weight"]]
    el = [t.double().requires_grad_(True) for t in ev]
    y = lo.epilogue(*el, 1e-6)
    eg = torch.autograd.grad((y * extra["dy"].double()).sum(), el)
    out["epi_y"] = y.detach().numpy()
    out.update({"epi_d" + n: x.numpy() for n, x in zip(("o", "x", "D", "gate", "weight"), eg)})
    return out


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "simple_gla_grad.npz"), **gla_case())
    np.savez_compressed(os.path.join(HERE, "layer_glue_grad.npz"), **glue_case())
    np.savez_compressed(os.path.join(HERE, "c0_recurrent_fp32.npz"), **c0_case())
    np.savez_compressed(os.path.join(HERE, "small_grad_state_var.npz"), **grad_case())
    np.savez_compressed(os.path.join(HERE, "varlen_forward.npz"), **varlen_case())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))
