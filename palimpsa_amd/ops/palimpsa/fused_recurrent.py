"""Token-serial Palimpsa operator (inference / decode path) on HIP kernels.

Mirrors palimpsa/ops/palimpsa/fused_recurrent_palimpsa.py of the reference:
``fused_recurrent_palimpsa`` (:258-297) and ``FusedRecurrentPalimpsaFunction``
(:215-253) keep their names, argument order, defaults, return packing and
ValueErrors.  Differences, all on purpose:

* rows are consumed in their own dtype (bf16 or fp32) by the kernel; the
  reference casts seven tensors to fp32 on the host first (:226-236);
* a backward exists (the reference raises NotImplementedError, :250-253): the token-serial backward kernel for
  short sequences, the chunked backward kernels (same gradients, tiles of 64 tokens in parallel) for long ones.
"""
from __future__ import annotations

from typing import Optional

import torch

from ... import _lib as L
from . import _common as cm
from . import _custom_ops as _ops


def _recurrent_forward(q, k, v, b, gt, g, Ip, scale, initial_mu_state, initial_I_state,
                       output_final_state, output_uncertainty, cu_seqlens):
    p = cm.prepare_inputs(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, cu_seqlens, recurrent=True)
    dev = p.q.device
    B, T, H, _ = p.v.shape
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
        ctx.set_materialize_grads(False)   # unused outputs (o_var, final states) send None, not zero tensors
        ctx.save_for_backward(p.q, p.k, p.v, p.b, p.gt, p.g, p.Ip, p.init_mu, p.init_I, p.cu_seqlens)
        ctx.meta = dict(dk=p.dk, dv=p.dv, n_seqs=p.n_seqs, compute_dtype=p.compute_dtype, scale=float(scale),
                        in_dtypes=(q.dtype, k.dtype, v.dtype, b.dtype, gt.dtype, g.dtype, Ip.dtype),
                        g_shape=tuple(g.shape), Ip_shape=tuple(Ip.shape), has_init=p.init_mu is not None,
                        output_uncertainty=bool(output_uncertainty))
        o = cm.unpad_last(o, p.dv).to(v.dtype)
        o_var = cm.unpad_last(o_var, p.dv)
        return o, o_var, cm.unpad_state(final_mu, p), cm.unpad_state(final_I, p)

    @staticmethod
    def backward(ctx, do, do_var, d_final_mu, d_final_I):
        # gradients arriving at the final states are ignored, as in the chunked path (chunk...py:522)
        q, k, v, b, gt, g, Ip, init_mu, init_I, cu = ctx.saved_tensors
        m = ctx.meta
        p = cm.Prepared(q, k, v, b, gt, g, Ip, init_mu, init_I, cu, m["dk"], m["dv"], q.shape[-1], v.shape[-1],
                        m["n_seqs"], m["compute_dtype"])
        if not m["output_uncertainty"]:
            do_var = None
        gr = recurrent_backward(p, m["scale"], do, do_var, m["in_dtypes"], m["g_shape"], m["Ip_shape"])
        return gr[:7] + (None, gr[7], gr[8], None, None, None)


def recurrent_backward(p: "cm.Prepared", scale: float, do, do_var, in_dtypes, g_shape, Ip_shape):
    """pal_recurrent_bwd on prepared (kernel-ready) inputs; returns (dq, dk, dv, db, dgt, dg, dIp, d_init_mu | None,
    d_init_I | None) in the dtypes and shapes of the caller's tensors."""
    import ctypes as C
    q, k, v, b, gt, g, Ip, init_mu, init_I, cu = p.q, p.k, p.v, p.b, p.gt, p.g, p.Ip, p.init_mu, p.init_I, p.cu_seqlens
    dev = q.device
    B, T, H, dv_p = v.shape
    dk_p = q.shape[-1]
    cd = p.compute_dtype
    has_init = init_mu is not None
    has_var = do_var is not None
    if do is None:
        do = torch.zeros(B, T, H, p.dv, dtype=cd, device=dev)

    def prep(x, dt):
        x = x.to(dt)
        if dv_p != p.dv:
            x = torch.nn.functional.pad(x, (0, dv_p - p.dv))
        return x.contiguous()

    do_p = prep(do, cd)
    dovar_p = prep(do_var, torch.float32) if has_var else None
    dq, dk_, dv_, db = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(b)
    dgt = torch.empty(B, T, H, dtype=torch.float32, device=dev)
    dg = torch.empty(H, dtype=torch.float32, device=dev)
    dIp = torch.empty(H, dtype=torch.float32, device=dev)
    d_init_mu = torch.empty_like(init_mu) if has_init else None
    d_init_I = torch.empty_like(init_I) if has_init else None
    flags = 0
    if cu is not None:
        flags |= L.PAL_FLAG_VARLEN
    if has_init:
        flags |= L.PAL_FLAG_HAS_INIT
    if has_var:
        flags |= L.PAL_FLAG_HAS_VAR
    pt = cm._ptr
    grads = L.PalBwdTensors(d_o=pt(do_p), d_o_var=pt(dovar_p), dq=pt(dq), dk=pt(dk_), dv=pt(dv_), db=pt(db),
                            dgt=pt(dgt), dg=pt(dg), dIp=pt(dIp), d_init_mu=pt(d_init_mu), d_init_I=pt(d_init_I))
    lib = L.load()
    mode_flags = L.state_pass_flags()
    route_min = L.recurrent_bwd_chunk_min()
    if (route_min is not None and B * T >= route_min * p.n_seqs
            and lib.pal_chunk_bwd_supported(dk_p, dv_p, cm._pal_dtype(cd), mode_flags) == 0):
        # Long sequences: the token-serial backward walks every sequence token by token (a few microseconds per
        # token and sequence whatever the batch), the chunked backward works on all tiles of 64 tokens at once.  The
        # tile-start states it needs come from a states-only pass of the chunked forward; fp32 rows keep the fp32 bar
        # (split operands).  Same gradients, tested against each other and against the oracle.
        table = offsets = None
        if cu is not None:
            meta, total_chunks = cm.chunk_meta(cu, T, dev)
            offsets, table = meta[: p.n_seqs + 1], meta[p.n_seqs + 1:]
        else:
            total_chunks = (T + L.PAL_CHUNK - 1) // L.PAL_CHUNK * B
        tile_mu = torch.empty(total_chunks, H, dv_p, dk_p, dtype=torch.float32, device=dev)
        tile_I = torch.empty_like(tile_mu)
        dims = L.PalDims(batch=B, seq_len=T, n_seqs=p.n_seqs, n_heads=H, dk=dk_p, dv=dv_p, total_chunks=total_chunks,
                         dtype=cm._pal_dtype(cd), gate_dtype=cm._pal_dtype(gt.dtype), var_dtype=L.PAL_DTYPE_F32,
                         flags=(flags & ~L.PAL_FLAG_HAS_VAR) | mode_flags | L.PAL_FLAG_STATES_ONLY, scale=float(scale),
                         n_qk_heads=q.shape[2])
        tens = L.PalFwdTensors(q=pt(q), k=pt(k), v=pt(v), b=pt(b), gt=pt(gt), g=pt(g), Ip=pt(Ip), o=None,
                               init_mu=pt(init_mu), init_I=pt(init_I), cu_seqlens=pt(cu), chunk_table=pt(table),
                               chunk_offsets=pt(offsets), chunk_mu=pt(tile_mu), chunk_I=pt(tile_I))
        with torch.cuda.device(dev):
            stream = cm.current_stream_ptr(dev)
            L.check(lib.pal_chunk_fwd(dims, tens, stream), "pal_chunk_fwd (tile-start states)")
            dims.flags = flags | mode_flags
            tens.o = pt(do_p)
            ws_bytes = int(lib.pal_chunk_bwd_workspace_bytes(dims))
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
            rc = lib.pal_chunk_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, stream)
        L.check(rc, "pal_chunk_bwd")
    else:
        dims = L.PalDims(batch=B, seq_len=T, n_seqs=p.n_seqs, n_heads=H, dk=dk_p, dv=dv_p, total_chunks=0,
                         dtype=cm._pal_dtype(cd), gate_dtype=cm._pal_dtype(gt.dtype), var_dtype=L.PAL_DTYPE_F32,
                         flags=flags, scale=float(scale), n_qk_heads=q.shape[2])
        tens = L.PalFwdTensors(q=pt(q), k=pt(k), v=pt(v), b=pt(b), gt=pt(gt), g=pt(g), Ip=pt(Ip), o=pt(do_p),
                               init_mu=pt(init_mu), init_I=pt(init_I), cu_seqlens=pt(cu))
        ws_bytes = int(lib.pal_recurrent_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_recurrent_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_recurrent_bwd")
    dts = in_dtypes
    dq = cm.unpad_last(dq, p.dk).to(dts[0])
    dk_ = cm.unpad_last(dk_, p.dk).to(dts[1])
    dv_ = cm.unpad_last(dv_, p.dv).to(dts[2])
    db = cm.unpad_last(db, p.dv).to(dts[3])
    if d_init_mu is not None and (dk_p != p.dk or dv_p != p.dv):
        d_init_mu = d_init_mu[:, :, :p.dv, :p.dk].contiguous()
        d_init_I = d_init_I[:, :, :p.dv, :p.dk].contiguous()
    return (dq, dk_, dv_, db, dgt.to(dts[4]), dg.reshape(g_shape).to(dts[5]), dIp.reshape(Ip_shape).to(dts[6]),
            d_init_mu, d_init_I)


@cm.no_compile
def _eager_recurrent(*args):
    return FusedRecurrentPalimpsaFunction.apply(*args)


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
    if _ops.available() and torch.compiler.is_compiling():
        # under a tracer the work is handed over as opaque library ops (see _custom_ops.py)
        o, o_var, final_mu_state, final_I_state = _ops.recurrent_fwd(
            q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, float(scale), bool(output_final_state),
            bool(output_uncertainty), cu_seqlens)
    else:
        o, o_var, final_mu_state, final_I_state = _eager_recurrent(
            q, k, v, b, gt, g, Ip, scale, initial_mu_state, initial_I_state, output_final_state, output_uncertainty,
            cu_seqlens)
    out = (o, o_var) if output_uncertainty else o
    if output_final_state:
        return out, final_mu_state, final_I_state
    return out
