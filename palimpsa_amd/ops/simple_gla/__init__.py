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

``chunk_simple_gla`` without autograd (prefill, evaluation) runs a forward of its own
(``pal_gla_chunk_fwd``): without the division by ``I`` a tile's output is two plain matrix products, so
the per-token state never has to exist.  With autograd, and on the token-serial path, the precision branch
still runs (on zeros) and the call costs what the Palimpsa operator costs.
"""
from __future__ import annotations

from typing import Optional

import torch

from ... import _lib as L
from ..palimpsa import _common as cm
from ..palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
from ..palimpsa.chunk import _chunk_meta, _count_chunks

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


def _chunk_forward_only(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens):
    """Forward without the precision state through ``pal_gla_chunk_fwd``; nothing is kept for a backward."""
    if g is None:
        raise ValueError("g (log decay per token and head, [B, T, H]) is required")
    if g.shape != q.shape[:3]:
        raise ValueError(f"g must have shape {tuple(q.shape[:3])}, got {tuple(g.shape)}")
    if cu_seqlens is not None and q.shape[0] != 1:
        raise ValueError(f"Batch size must be 1 for Varlen, got {q.shape[0]}")
    if scale is None:
        scale = q.shape[-1] ** -0.5
    H = q.shape[2]
    dev = q.device
    # f_t = exp(-gt_t * rate): the kernels take g itself as gt with a rate of -1
    rate = torch.full((H,), -1.0, dtype=torch.float32, device=dev)
    S0 = None
    if initial_state is not None:
        S0 = initial_state.float().transpose(-1, -2).contiguous()       # [N,H,dk,dv] -> [N,H,dv,dk]
    p = cm.prepare_inputs(q, k, v, v, g, rate, rate, S0, S0, cu_seqlens, recurrent=False)
    B, T = p.q.shape[:2]
    table = offsets = None
    flags = 0
    if p.cu_seqlens is not None:
        meta, total_chunks = _chunk_meta(cu_seqlens)
        meta = meta.to(dev)
        offsets, table = meta[: p.n_seqs + 1], meta[p.n_seqs + 1:]
        flags |= L.PAL_FLAG_VARLEN
    else:
        total_chunks = _count_chunks(T, B)
    o = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev)
    tile_S = torch.empty(total_chunks, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
    final = None
    if output_final_state:
        final = torch.empty(p.n_seqs, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        flags |= L.PAL_FLAG_STORE_FINAL
    if p.init_mu is not None:
        flags |= L.PAL_FLAG_HAS_INIT
    dims = cm.make_dims(p, scale, flags, total_chunks)
    pt = cm._ptr
    tens = L.PalFwdTensors(q=pt(p.q), k=pt(p.k), v=pt(p.v), gt=pt(p.gt), g=pt(p.g), o=pt(o), init_mu=pt(p.init_mu),
                           final_mu=pt(final), cu_seqlens=pt(p.cu_seqlens), chunk_table=pt(table),
                           chunk_offsets=pt(offsets), chunk_mu=pt(tile_S))
    with torch.cuda.device(dev):
        rc = L.load().pal_gla_chunk_fwd(dims, tens, cm.current_stream_ptr(dev))
    L.check(rc, "pal_gla_chunk_fwd")
    o = cm.unpad_last(o, p.dv).to(q.dtype)
    if final is not None:
        final = cm.unpad_state(final, p).transpose(-1, -2).contiguous()
    return o, final


def chunk_simple_gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: Optional[torch.Tensor] = None,
                     scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                     output_final_state: bool = False, cu_seqlens: Optional[torch.Tensor] = None):
    """Chunked (training / prefill) form; returns ``(o, final_state | None)``."""
    needs_grad = torch.is_grad_enabled() and any(
        isinstance(x, torch.Tensor) and x.requires_grad for x in (q, k, v, g, initial_state))
    if not needs_grad:
        return _chunk_forward_only(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens)
    return _run(chunk_palimpsa, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, chunk_size=64)


def fused_recurrent_simple_gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: Optional[torch.Tensor] = None,
                               scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                               output_final_state: bool = False, cu_seqlens: Optional[torch.Tensor] = None):
    """Token-serial (decode) form; returns ``(o, final_state | None)``."""
    return _run(fused_recurrent_palimpsa, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens)
