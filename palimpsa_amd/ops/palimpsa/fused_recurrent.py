"""Token-serial Palimpsa operator (inference / decode path) on HIP kernels.

Mirrors palimpsa/ops/palimpsa/fused_recurrent_palimpsa.py of the reference:
``fused_recurrent_palimpsa`` (:258-297) and ``FusedRecurrentPalimpsaFunction``
(:215-253) keep their names, argument order, defaults, return packing and
ValueErrors.  Differences, all on purpose:

* rows are consumed in their own dtype (bf16 or fp32) by the kernel; the
  reference casts seven tensors to fp32 on the host first (:226-236);
* a backward exists (the reference raises NotImplementedError, :250-253).
"""
from __future__ import annotations

from typing import Optional

import torch

from ... import _lib as L
from . import _common as cm


def _recurrent_forward(q, k, v, b, gt, g, Ip, scale, initial_mu_state, initial_I_state,
                       output_final_state, output_uncertainty, cu_seqlens):
    p = cm.prepare_inputs(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, cu_seqlens, recurrent=True)
    dev = p.q.device
    B, T, H, _ = p.q.shape
    o = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev)
    # the reference leaves o_var in fp32 (fused...py:184-186 after the casts of :226-232)
    o_var = torch.empty(B, T, H, p.dv_p, dtype=torch.float32, device=dev) if output_uncertainty else None
    final_mu = final_I = None
    if output_final_state:
        final_mu = torch.empty(p.n_seqs, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        final_I = torch.empty_like(final_mu)
    flags = 0
    if p.cu_seqlens is not None:
        flags |= L.PAL_FLAG_VARLEN
    if p.init_mu is not None:
        flags |= L.PAL_FLAG_HAS_INIT
    if output_final_state:
        flags |= L.PAL_FLAG_STORE_FINAL
    if output_uncertainty:
        flags |= L.PAL_FLAG_HAS_VAR
    dims = cm.make_dims(p, scale, flags)
    tens = cm.make_fwd_tensors(p, o, o_var, final_mu, final_I)
    with torch.cuda.device(dev):
        rc = L.load().pal_recurrent_fwd(dims, tens, cm.current_stream_ptr(dev))
    L.check(rc, "pal_recurrent_fwd")
    return p, dims, o, o_var, final_mu, final_I


class FusedRecurrentPalimpsaFunction(torch.autograd.Function):
    """Same 13 positional arguments and 4 outputs as the reference Function (fused...py:218)."""

    @staticmethod
    def forward(ctx, q, k, v, b, gt, g, Ip, scale, initial_mu_state, initial_I_state,
                output_final_state, output_uncertainty, cu_seqlens):
        p, dims, o, o_var, final_mu, final_I = _recurrent_forward(
            q, k, v, b, gt, g, Ip, scale, initial_mu_state, initial_I_state,
            output_final_state, output_uncertainty, cu_seqlens)
        ctx.prepared = p
        ctx.scale = float(scale)
        ctx.output_uncertainty = bool(output_uncertainty)
        ctx.in_dtypes = (q.dtype, k.dtype, v.dtype, b.dtype, gt.dtype, g.dtype, Ip.dtype)
        ctx.in_shapes = (g.shape, Ip.shape)
        ctx.has_init = initial_mu_state is not None
        o = cm.unpad_last(o, p.dv).to(v.dtype)
        o_var = cm.unpad_last(o_var, p.dv)
        return o, o_var, cm.unpad_state(final_mu, p), cm.unpad_state(final_I, p)

    @staticmethod
    def backward(ctx, do, do_var, d_final_mu, d_final_I):
        from .recurrent_backward import recurrent_backward

        return recurrent_backward(ctx, do, do_var)


def fused_recurrent_palimpsa(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    b: torch.Tensor,
    gt: torch.Tensor,
    g: torch.Tensor,
    Ip: torch.Tensor,
    scale: float = None,
    initial_mu_state: Optional[torch.Tensor] = None,
    initial_I_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    output_uncertainty: bool = False,
    cu_seqlens: Optional[torch.LongTensor] = None,
):
    """o_t = scale * (M_t / I_t) q_t over a token-serial scan; see the reference docstring-free
    entry point fused_recurrent_palimpsa (fused...py:258-297) for the calling convention.

    Returns ``o`` (or ``(o, o_var)`` with ``output_uncertainty``), followed by
    ``final_mu_state, final_I_state`` when ``output_final_state`` is set.
    """
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f"The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.")
        if initial_mu_state is not None and initial_mu_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError("Initial states mismatch sequence length.")
    if scale is None:
        scale = k.shape[-1] ** -0.5
    o, o_var, final_mu_state, final_I_state = FusedRecurrentPalimpsaFunction.apply(
        q, k, v, b, gt, g, Ip, scale, initial_mu_state, initial_I_state,
        output_final_state, output_uncertainty, cu_seqlens)
    out = (o, o_var) if output_uncertainty else o
    if output_final_state:
        return out, final_mu_state, final_I_state
    return out
