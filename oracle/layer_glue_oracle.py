"""CPU restatement of the element-wise work of the reference layer either side of the operator
(TEST INFRASTRUCTURE ONLY: the checker for pal_prologue_* / pal_epilogue_*; never imported by the package).

What it restates (citations are into the reference repository):

* ``prologue``: palimpsa/layers/palimpsa.py:263-279 —
  head split (:263-264), repeat of the q/k heads (:266-267),
  ``dt = softplus(dt_proj(h).float() + dt_bias)`` (:269), ``q, k = F.normalize(q), F.normalize(k)`` (:271),
  ``bs = sigmoid(bs_proj(h).float()).to(h.dtype)`` (:272), ``v = x * bs`` (:273),
  ``b = (sigmoid(b_raw.float()) * softplus(b_scale.float()) * bs).to(h.dtype)`` (:276-279).
  It is written with the same torch library routines as the reference lines.
* ``epilogue``: palimpsa/layers/palimpsa.py:337-343 — ``o + x * D`` (:338) and
  ``FusedRMSNormGated(head_v_dim, eps)(o, gate)`` (:341; built at :141-145).  FusedRMSNormGated is a
  module of flash-linear-attention, a dependency that is not in the reference tree and not installed
  here (unpinned version): its published behaviour — RMS norm over the last dim with a learnable
  weight, times ``gate * sigmoid(gate)`` — is restated, and is **parity unpinned** against the
  third-party code itself.  What the mathematics fixes is pinned in tests/test_layer_glue_oracle_cpu.py:
  the ungated case against ``torch.nn.functional.rms_norm``, the gate against ``F.silu``, unit norms and
  head repetition of q/k, and ``torch.autograd.gradcheck`` of both functions in float64.
* ``mamba_prologue``: palimpsa/layers/meta_mamba2.py:283-299 —
  ``dt = clamp(softplus(dt.float() + dt_bias), *time_step_limit)`` (:283-284), ``dx = (x * dt).to(x.dtype)`` (:294),
  ``b = (sigmoid(b_raw) * softplus(b_scale) * dt).to(h.dtype)`` (:296-299); same torch routines as those lines.
* ``mamba_epilogue``: palimpsa/layers/meta_mamba2.py:355-363 — ``o + x * D`` (:356), heads flattened (:359) and
  ``RMSNormGated(intermediate_size, eps, norm_before_gate=False)(o, gate)`` (:363; built at :130-132), again a module of
  flash-linear-attention (fla.modules.layernorm_gated, the Mamba2 norm): with ``norm_before_gate=False`` it is
  ``rms_norm(x * silu(z)) * weight`` over the whole last dim.  Restated from that published behaviour, **parity unpinned**
  against the third-party code; pinned in the same test file against ``F.rms_norm`` on the gated input, by
  the clamp's limits and by ``gradcheck``.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def prologue(q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw=None, b_scale=None, model_dtype=None, compute=torch.float64,
             eps=1e-12):
    """Returns (q, k, v, b | None, gt) in ``compute`` precision; ``model_dtype`` is the dtype the reference
    rounds ``bs`` to (hidden_states.dtype); None keeps it unrounded."""
    H = x.shape[-2]
    rep = H // q_raw.shape[-2]
    q = F.normalize(q_raw.to(compute), p=2, dim=-1, eps=eps).repeat_interleave(rep, dim=-2)
    k = F.normalize(k_raw.to(compute), p=2, dim=-1, eps=eps).repeat_interleave(rep, dim=-2)
    gt = F.softplus(dt_raw.to(compute) + dt_bias.to(compute))
    bs = torch.sigmoid(bs_raw.to(compute))
    if model_dtype is not None:
        bs = bs.to(model_dtype).to(compute)
    v = x.to(compute) * bs.unsqueeze(-1)
    b = None
    if b_raw is not None:
        b = torch.sigmoid(b_raw.to(compute)) * F.softplus(b_scale.to(compute)).view(-1, 1)
        b = b * bs.unsqueeze(-1)
    return q, k, v, b, gt


def epilogue(o, x, D, gate, weight, eps, compute=torch.float64):
    """rmsnorm(o + x * D) * weight [* gate * sigmoid(gate)] over the last dim, in ``compute`` precision."""
    r = o.to(compute)
    if x is not None:
        r = r + x.to(compute) * D.to(compute).view(-1, 1)
    rstd = torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps)
    y = r * rstd * weight.to(compute)
    if gate is not None:
        g = gate.to(compute)
        y = y * g * torch.sigmoid(g)
    return y


def mamba_prologue(x, dt_raw, dt_bias, b_raw=None, b_scale=None, dt_limit=(0.0, float("inf")), compute=torch.float64):
    """Returns (v, b | None, dt) in ``compute`` precision."""
    dt = F.softplus(dt_raw.to(compute) + dt_bias.to(compute))
    dt = torch.clamp(dt, dt_limit[0], dt_limit[1])
    v = x.to(compute) * dt.unsqueeze(-1)
    b = None
    if b_raw is not None:
        b = torch.sigmoid(b_raw.to(compute)) * F.softplus(b_scale.to(compute)).view(-1, 1)
        b = b * dt.unsqueeze(-1)
    return v, b, dt


def mamba_epilogue(o, x, D, gate, weight, eps, compute=torch.float64):
    """rmsnorm over all heads of ((o + x * D) * gate * sigmoid(gate)) * weight; o [..., H, dv] -> [..., H, dv]."""
    r = o.to(compute)
    if x is not None:
        r = r + x.to(compute).reshape(r.shape) * D.to(compute).view(-1, 1)
    flat = r.flatten(-2)
    if gate is not None:
        g = gate.to(compute).reshape(flat.shape)
        flat = flat * g * torch.sigmoid(g)
    rstd = torch.rsqrt(flat.pow(2).mean(-1, keepdim=True) + eps)
    return (flat * rstd * weight.to(compute).reshape(-1)).reshape(r.shape)
