"""Shared helpers of the parity tests: seeded inputs, error metrics, oracle runs."""
from __future__ import annotations

import torch

from oracle import palimpsa_oracle as po

# fp32 kernels: max |x - ref| / max |ref| <= 1e-4
FP32_REL_TOL = 1e-4
# bf16-input kernels: max |x - ref| <= 2e-2 on outputs
BF16_OUT_ABS_TOL = 2e-2
# bf16-input kernels: max |dx - dref| / max |dref| <= 5e-2 on gradients
# ("normalised" = by the largest reference entry; the reference script's own
#  normalisation max|d|/mean|ref| (check_palimpsa.py:28-32) is printed next to it)
BF16_GRAD_NORM_TOL = 5e-2
# fp32 rows through the chunked kernels (operands split into two bf16 halves): the fp32 bar, outputs and states
# max|x - ref| / max(1, max|ref|), gradients max|dx - dref| / max|dref|
CHUNK_FP32_OUT_TOL = 1e-4
CHUNK_FP32_GRAD_TOL = 1e-4


def max_rel(x: torch.Tensor, ref: torch.Tensor) -> float:
    x = x.detach().double().cpu()
    ref = ref.detach().double().cpu()
    den = ref.abs().max().item()
    return (x - ref).abs().max().item() / (den if den > 0 else 1.0)


def max_abs(x: torch.Tensor, ref: torch.Tensor) -> float:
    return (x.detach().double().cpu() - ref.detach().double().cpu()).abs().max().item()


def mean_norm(x: torch.Tensor, ref: torch.Tensor) -> float:
    ref = ref.detach().double().cpu()
    den = ref.abs().mean().item()
    return (x.detach().double().cpu() - ref).abs().max().item() / (den if den > 0 else 1.0)


def rounded(inp: dict, dtype) -> dict:
    """Inputs as the kernels see them: q,k,v,b rounded to ``dtype`` (gates stay fp32)."""
    out = dict(inp)
    for n in ("q", "k", "v", "b"):
        out[n] = inp[n].to(dtype)
    return out


def to_device(inp: dict, dev) -> dict:
    return {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in inp.items()}


def oracle_forward(inp: dict, scale=None, mu0=None, I0=None, cu=None, want_var=False, dtype=torch.float32):
    """Oracle on the (already rounded) inputs, upcast to ``dtype`` on the CPU."""
    return po.palimpsa_recurrence(
        inp["q"].float(), inp["k"].float(), inp["v"].float(), inp["b"].float(), inp["gt"].float(),
        inp["g"], inp["Ip"], mu0, I0, scale=scale, cu_seqlens=cu, output_uncertainty=want_var,
        var_scale_power=1, compute_dtype=dtype)


def oracle_grads(inp: dict, do, dovar=None, scale=None, mu0=None, I0=None, cu=None, dtype=torch.float64):
    """Gradients of sum(o*do) (+ sum(o_var*dovar)) through the oracle, by autograd."""
    names = ["q", "k", "v", "b", "gt", "g", "Ip"]
    leaves = [inp[n].detach().to(dtype).clone().requires_grad_(True) for n in names]
    st = []
    if mu0 is not None:
        st = [mu0.detach().to(dtype).clone().requires_grad_(True), I0.detach().to(dtype).clone().requires_grad_(True)]
    o, ov, fmu, fI = po.palimpsa_recurrence(*leaves, *(st if st else [None, None]), scale=scale, cu_seqlens=cu,
                                            output_uncertainty=dovar is not None, var_scale_power=1,
                                            compute_dtype=dtype)
    loss = (o * do.to(dtype)).sum()
    if dovar is not None:
        loss = loss + (ov * dovar.to(dtype)).sum()
    gr = torch.autograd.grad(loss, leaves + st)
    out = dict(zip(names + (["mu0", "I0"] if st else []), gr))
    out["o"] = o.detach()
    out["o_var"] = None if ov is None else ov.detach()
    return out
