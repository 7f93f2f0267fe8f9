"""Scalar-gated linear attention served by the Palimpsa kernels.

The reference layer falls back to ``fla.ops.simple_gla`` when its precision state is switched off
(``metaplasticity=False``: palimpsa/layers/palimpsa.py:18, :293-300).  With ``b = 0`` and ``Ip = 1``
the Palimpsa recurrence has ``I = 1`` everywhere, so ``mu = M`` and

    S_t = exp(g_t) S_{t-1} + k_t^T v_t ,   o_t = scale * q_t S_t

is exactly what the kernels compute with ``gt = -g`` and a unit per-head rate.  ``chunk_simple_gla`` and
``fused_recurrent_simple_gla`` keep the keyword names of the layer's call sites (``q, k, v, g,
scale, initial_state, output_final_state, cu_seqlens``), the default ``scale = dk ** -0.5`` and the
``(o, final_state)`` return; the state is ``[N, H, dk, dv]`` fp32 (the transpose of the kernels'
``[N, H, dv, dk]``).  flash-linear-attention itself is not part of the reference tree, so its own
conventions beyond these call sites are not pinned; the arithmetic is pinned by the closed form
``o = scale * ((Q K^T) * L) V`` in the tests.

The precision branch still runs (on zeros), so this path costs what the Palimpsa operator costs;
a kernel specialised for ``b = 0`` is not built.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..palimpsa import chunk_palimpsa, fused_recurrent_palimpsa

__all__ = ["chunk_simple_gla", "fused_recurrent_simple_gla"]


def _run(op, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, **kw):
    if g is None:
        raise ValueError("g (log decay per token and head, [B, T, H]) is required")
    if g.shape != q.shape[:3]:
        raise ValueError(f"g must have shape {tuple(q.shape[:3])}, got {tuple(g.shape)}")
    H = q.shape[2]
    dev = q.device
    b = torch.zeros_like(v)
    rate = torch.ones(H, dtype=torch.float32, device=dev)
    Ip = torch.ones(H, dtype=torch.float32, device=dev)
    mu0 = I0 = None
    if initial_state is not None:
        mu0 = initial_state.float().transpose(-1, -2).contiguous()     # [N,H,dk,dv] -> [N,H,dv,dk]
        I0 = torch.ones_like(mu0)
    out = op(q, k, v, b, -g.float(), rate, Ip, scale=scale, initial_mu_state=mu0, initial_I_state=I0,
             output_final_state=output_final_state, cu_seqlens=cu_seqlens, **kw)
    if output_final_state:
        o, mu, _ = out
        return o, mu.transpose(-1, -2).contiguous()
    return out, None


def chunk_simple_gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: Optional[torch.Tensor] = None,
                     scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                     output_final_state: bool = False, cu_seqlens: Optional[torch.Tensor] = None):
    """Chunked (training / prefill) form; returns ``(o, final_state | None)``."""
    return _run(chunk_palimpsa, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, chunk_size=64)


def fused_recurrent_simple_gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: Optional[torch.Tensor] = None,
                               scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                               output_final_state: bool = False, cu_seqlens: Optional[torch.Tensor] = None):
    """Token-serial (decode) form; returns ``(o, final_state | None)``."""
    return _run(fused_recurrent_palimpsa, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens)
