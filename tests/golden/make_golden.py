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


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "c0_recurrent_fp32.npz"), **c0_case())
    np.savez_compressed(os.path.join(HERE, "small_grad_state_var.npz"), **grad_case())
    np.savez_compressed(os.path.join(HERE, "varlen_forward.npz"), **varlen_case())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))
