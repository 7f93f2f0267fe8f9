"""``palimpsa_ref``: the plain-PyTorch token loop of the operator's public API.

Mirror of palimpsa_ref in the reference
(palimpsa/ops/palimpsa/chunk_palimpsa_forgetting_scalar.py:669-725): same
signature, same fp32 arithmetic, same return packing, and the same quirk that
``y_var`` uses the pre-scaled q (so it carries scale**2, :709/:718) whereas the
kernels carry scale once.  Runs on whatever device the inputs live on (the
reference relies on a global default device, :700-703).  It is part of the
API surface, not the test oracle, and no kernel path calls it.
"""
from __future__ import annotations

import torch


def palimpsa_ref(q, k, v, b, gt, g, Ip, initial_mu_state=None, initial_I_state=None, scale=None,
                 output_final_state=False, output_uncertainty=False):
    dtype_in = v.dtype
    q, k, v, b, gt, g, Ip = [x.float() for x in (q, k, v, b, gt, g, Ip)]
    if scale is None:
        scale = q.shape[-1] ** -0.5
    B, T, H, DV = b.shape
    DK = k.shape[-1]
    dev = v.device
    y = torch.zeros(B, T, H, DV, device=dev)
    y_var = torch.zeros(B, T, H, DV, device=dev)
    if initial_mu_state is None:
        mu_prev = torch.zeros(B, H, DV, DK, device=dev)
        I_prev = Ip[None, :, None, None]
    else:
        mu_prev, I_prev = initial_mu_state, initial_I_state
    qs = q * scale
    prior = Ip[None, :, None, None]
    mu, I = mu_prev, I_prev
    for t in range(T):
        decay = torch.exp(-gt[:, t, :, None, None] * g[None, :, None, None])
        k_t = k[:, t, :, None, :]
        M = v[:, t, :, :, None] * k_t + decay * mu_prev * I_prev
        I = b[:, t, :, :, None] * k_t.square() + (1 - decay) * prior + decay * I_prev
        mu = M / I
        y[:, t] = (mu * qs[:, t, :, None, :]).sum(-1)
        y_var[:, t] = (qs[:, t, :, None, :].square() / I).sum(-1)
        mu_prev, I_prev = mu, I
    out = (y.to(dtype_in), y_var.to(dtype_in)) if output_uncertainty else y.to(dtype_in)
    if output_final_state:
        return out, mu, I
    return out
