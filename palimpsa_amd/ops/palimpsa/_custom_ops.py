"""The two operators as ``torch.library`` custom ops, for callers under ``torch.compile``.

The reference wrote its wrapper so that a compiler could trace through it (buffers allocated outside the
autograd Function, no ``.item()``; chunk_palimpsa_forgetting_scalar.py:627-651).  Here the work happens in
ctypes calls that a tracer cannot follow, so the entry points hand a tracer four opaque ops instead:
``palimpsa_amd::chunk_fwd`` / ``chunk_bwd`` and ``palimpsa_amd::recurrent_fwd`` / ``recurrent_bwd``, each with a
shape-only (fake) implementation and the forward ops with ``register_autograd``.  ``chunk_palimpsa`` and
``fused_recurrent_palimpsa`` take this route while ``torch.compiler.is_compiling()`` and the plain eager route
(the autograd Functions of chunk.py / fused_recurrent.py, same kernels) otherwise, so ``fullgraph=True`` callers
compile without a graph break.

Every shape an op returns follows from the shapes of its arguments: with ``cu_seqlens`` the tile-start states are
sized for the largest tile count the packed row can have (``T // 64 + N``), the chunk table itself is built inside
the op.  Absent optional outputs (``o_var``, gradients of a missing initial state) are returned as empty tensors.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from ... import _lib as L
from . import _common as cm

_HAS_CUSTOM_OP = hasattr(torch, "library") and hasattr(torch.library, "custom_op")


def available() -> bool:
    return _HAS_CUSTOM_OP


def _max_tiles(B: int, T: int, n_seqs: int, varlen: bool) -> int:
    return (T // L.PAL_CHUNK + n_seqs) if varlen else (T + L.PAL_CHUNK - 1) // L.PAL_CHUNK * B


def _empty(like: torch.Tensor) -> torch.Tensor:
    return like.new_empty(0)


if _HAS_CUSTOM_OP:
    # ------------------------------------------------------------------------------------------------ chunked
    @torch.library.custom_op("palimpsa_amd::chunk_fwd", mutates_args=())
    def chunk_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b: torch.Tensor, gt: torch.Tensor, g: torch.Tensor,
                  Ip: torch.Tensor, init_mu: Optional[torch.Tensor], init_I: Optional[torch.Tensor], scale: float,
                  output_uncertainty: bool, cu_seqlens: Optional[torch.Tensor], mode_flags: int
                  ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """-> (o, o_var | empty, final_mu, final_I, tile_mu, tile_I).  ``mode_flags``: the knob bits of PalDims.flags
        (L.state_pass_flags() when the call was traced); the backward op gets the same value, so a knob changed
        between the two cannot mix operand modes.  The tile-start states of every tile are always kept (this op does
        not know whether a backward follows): a long prefill without gradients under a tracer needs
        total_chunks * H * dv * dk * 8 bytes where the eager entry point runs in windows of 512 MB."""
        p = cm.prepare_inputs(q, k, v, b, gt, g, Ip, init_mu, init_I, cu_seqlens, recurrent=False)
        dev = p.q.device
        B, T, H, _ = p.v.shape
        varlen = p.cu_seqlens is not None
        table = offsets = None
        flags = L.PAL_FLAG_STORE_FINAL
        if varlen:
            meta, total_chunks = cm.chunk_meta(cu_seqlens, T, dev)
            offsets, table = meta[: p.n_seqs + 1], meta[p.n_seqs + 1:]
            flags |= L.PAL_FLAG_VARLEN
        else:
            total_chunks = _max_tiles(B, T, p.n_seqs, False)
        if p.init_mu is not None:
            flags |= L.PAL_FLAG_HAS_INIT
        if output_uncertainty:
            flags |= L.PAL_FLAG_HAS_VAR
        o = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev)
        o_var = torch.empty_like(o) if output_uncertainty else None
        final_mu = torch.empty(p.n_seqs, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        final_I = torch.empty_like(final_mu)
        tile_mu = torch.empty(_max_tiles(B, T, p.n_seqs, varlen), H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        tile_I = torch.empty_like(tile_mu)
        dims = cm.make_dims(p, scale, flags, total_chunks, var_dtype=p.compute_dtype, mode_flags=mode_flags)
        tens = cm.make_fwd_tensors(p, o, o_var, final_mu, final_I, table, offsets, tile_mu, tile_I)
        with torch.cuda.device(dev):
            rc = L.load().pal_chunk_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_chunk_fwd")
        o = cm.unpad_last(o, p.dv).to(q.dtype)
        o_var = cm.unpad_last(o_var, p.dv).to(q.dtype) if output_uncertainty else _empty(o)
        return o, o_var, cm.unpad_state(final_mu, p), cm.unpad_state(final_I, p), tile_mu, tile_I

    @chunk_fwd.register_fake
    def _(q, k, v, b, gt, g, Ip, init_mu, init_I, scale, output_uncertainty, cu_seqlens, mode_flags):
        B, T, H, dv = v.shape
        dk = q.shape[-1]
        n_seqs = B if cu_seqlens is None else cu_seqlens.shape[0] - 1
        o = q.new_empty(B, T, H, dv)
        o_var = q.new_empty(B, T, H, dv) if output_uncertainty else q.new_empty(0)
        fin = q.new_empty(n_seqs, H, dv, dk, dtype=torch.float32)
        tiles = q.new_empty(_max_tiles(B, T, n_seqs, cu_seqlens is not None), H, cm.padded_dv(dv), cm.padded_dk(dk, False),
                            dtype=torch.float32)
        return o, o_var, fin, torch.empty_like(fin), tiles, torch.empty_like(tiles)

    @torch.library.custom_op("palimpsa_amd::chunk_bwd", mutates_args=())
    def chunk_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b: torch.Tensor, gt: torch.Tensor, g: torch.Tensor,
                  Ip: torch.Tensor, init_mu: Optional[torch.Tensor], init_I: Optional[torch.Tensor], scale: float,
                  cu_seqlens: Optional[torch.Tensor], tile_mu: torch.Tensor, tile_I: torch.Tensor, d_o: torch.Tensor,
                  d_o_var: Optional[torch.Tensor], mode_flags: int
                  ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                             torch.Tensor, torch.Tensor, torch.Tensor]:
        """-> (dq, dk, dv, db, dgt, dg, dIp, d_init_mu | empty, d_init_I | empty)"""
        p = cm.prepare_inputs(q, k, v, b, gt, g, Ip, init_mu, init_I, cu_seqlens, recurrent=False)
        dev = p.q.device
        B, T, H, _ = p.v.shape
        cd = p.compute_dtype
        table = offsets = None
        flags = 0
        if p.cu_seqlens is not None:
            meta, total_chunks = cm.chunk_meta(cu_seqlens, T, dev)
            offsets, table = meta[: p.n_seqs + 1], meta[p.n_seqs + 1:]
            flags |= L.PAL_FLAG_VARLEN
        else:
            total_chunks = _max_tiles(B, T, p.n_seqs, False)
        if p.init_mu is not None:
            flags |= L.PAL_FLAG_HAS_INIT
        if d_o_var is not None:
            flags |= L.PAL_FLAG_HAS_VAR

        def prep_grad(x):
            x = x.to(cd)
            if p.dv_p != p.dv:
                x = torch.nn.functional.pad(x, (0, p.dv_p - p.dv))
            return x.contiguous()

        do_p = prep_grad(d_o)
        dovar_p = prep_grad(d_o_var) if d_o_var is not None else None
        dq, dk_, dv_, db = torch.empty_like(p.q), torch.empty_like(p.k), torch.empty_like(p.v), torch.empty_like(p.b)
        dgt = torch.empty(B, T, H, dtype=torch.float32, device=dev)
        dg = torch.empty(H, dtype=torch.float32, device=dev)
        dIp = torch.empty(H, dtype=torch.float32, device=dev)
        d_mu = torch.empty_like(p.init_mu) if p.init_mu is not None else None
        d_I = torch.empty_like(p.init_I) if p.init_I is not None else None
        dims = cm.make_dims(p, scale, flags, total_chunks, var_dtype=cd, mode_flags=mode_flags)
        tens = cm.make_fwd_tensors(p, do_p, None, None, None, table, offsets, tile_mu, tile_I)
        pt = cm._ptr
        grads = L.PalBwdTensors(d_o=pt(do_p), d_o_var=pt(dovar_p), dq=pt(dq), dk=pt(dk_), dv=pt(dv_), db=pt(db),
                                dgt=pt(dgt), dg=pt(dg), dIp=pt(dIp), d_init_mu=pt(d_mu), d_init_I=pt(d_I))
        lib = L.load()
        ws_bytes = int(lib.pal_chunk_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_chunk_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_chunk_bwd")
        return (cm.unpad_last(dq, p.dk).to(q.dtype), cm.unpad_last(dk_, p.dk).to(k.dtype),
                cm.unpad_last(dv_, p.dv).to(v.dtype), cm.unpad_last(db, p.dv).to(b.dtype), dgt.to(gt.dtype),
                dg.reshape(g.shape).to(g.dtype), dIp.reshape(Ip.shape).to(Ip.dtype),
                cm.unpad_state(d_mu, p).to(init_mu.dtype) if d_mu is not None else _empty(dg),
                cm.unpad_state(d_I, p).to(init_I.dtype) if d_I is not None else _empty(dg))

    @chunk_bwd.register_fake
    def _(q, k, v, b, gt, g, Ip, init_mu, init_I, scale, cu_seqlens, tile_mu, tile_I, d_o, d_o_var, mode_flags):
        return (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(b), torch.empty_like(gt),
                torch.empty_like(g), torch.empty_like(Ip),
                torch.empty_like(init_mu) if init_mu is not None else g.new_empty(0),
                torch.empty_like(init_I) if init_I is not None else g.new_empty(0))

    def _chunk_setup(ctx, inputs, output):
        q, k, v, b, gt, g, Ip, init_mu, init_I, scale, output_uncertainty, cu_seqlens, mode_flags = inputs
        ctx.save_for_backward(q, k, v, b, gt, g, Ip, init_mu, init_I, cu_seqlens, output[4], output[5])
        ctx.scale = scale
        ctx.mode_flags = mode_flags
        ctx.output_uncertainty = output_uncertainty
        ctx.set_materialize_grads(False)

    def _chunk_backward(ctx, d_o, d_o_var, d_fmu, d_fI, d_tmu, d_tI):
        q, k, v, b, gt, g, Ip, init_mu, init_I, cu, tile_mu, tile_I = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros(v.shape, dtype=q.dtype, device=q.device)
        if not ctx.output_uncertainty:
            d_o_var = None
        # gradients arriving at the final states are ignored, as in the reference (chunk...py:522)
        gr = chunk_bwd(q, k, v, b, gt, g, Ip, init_mu, init_I, ctx.scale, cu, tile_mu, tile_I, d_o, d_o_var,
                       ctx.mode_flags)
        d_mu = gr[7] if init_mu is not None else None
        d_I = gr[8] if init_I is not None else None
        return gr[0], gr[1], gr[2], gr[3], gr[4], gr[5], gr[6], d_mu, d_I, None, None, None, None

    chunk_fwd.register_autograd(_chunk_backward, setup_context=_chunk_setup)

    # ------------------------------------------------------------------------------------------- token-serial
    @torch.library.custom_op("palimpsa_amd::recurrent_fwd", mutates_args=())
    def recurrent_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b: torch.Tensor, gt: torch.Tensor,
                      g: torch.Tensor, Ip: torch.Tensor, init_mu: Optional[torch.Tensor], init_I: Optional[torch.Tensor],
                      scale: float, output_final_state: bool, output_uncertainty: bool,
                      cu_seqlens: Optional[torch.Tensor]
                      ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """-> (o, o_var | empty, final_mu | empty, final_I | empty)"""
        from .fused_recurrent import _recurrent_forward
        p, _, o, o_var, fmu, fI = _recurrent_forward(q, k, v, b, gt, g, Ip, scale, init_mu, init_I, output_final_state,
                                                     output_uncertainty, cu_seqlens)
        o = cm.unpad_last(o, p.dv).to(v.dtype)
        e = lambda: o.new_empty(0, dtype=torch.float32)     # outputs may not alias one another
        return (o, cm.unpad_last(o_var, p.dv) if output_uncertainty else e(),
                cm.unpad_state(fmu, p) if output_final_state else e(), cm.unpad_state(fI, p) if output_final_state else e())

    @recurrent_fwd.register_fake
    def _(q, k, v, b, gt, g, Ip, init_mu, init_I, scale, output_final_state, output_uncertainty, cu_seqlens):
        B, T, H, dv = v.shape
        n_seqs = B if cu_seqlens is None else cu_seqlens.shape[0] - 1
        e = lambda: v.new_empty(0, dtype=torch.float32)
        fin = v.new_empty(n_seqs, H, dv, q.shape[-1], dtype=torch.float32) if output_final_state else e()
        return (torch.empty_like(v), v.new_empty(B, T, H, dv, dtype=torch.float32) if output_uncertainty else e(),
                fin, torch.empty_like(fin))

    @torch.library.custom_op("palimpsa_amd::recurrent_bwd", mutates_args=())
    def recurrent_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b: torch.Tensor, gt: torch.Tensor,
                      g: torch.Tensor, Ip: torch.Tensor, init_mu: Optional[torch.Tensor], init_I: Optional[torch.Tensor],
                      scale: float, cu_seqlens: Optional[torch.Tensor], d_o: torch.Tensor,
                      d_o_var: Optional[torch.Tensor]
                      ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                 torch.Tensor, torch.Tensor, torch.Tensor]:
        from .fused_recurrent import recurrent_backward
        p = cm.prepare_inputs(q, k, v, b, gt, g, Ip, init_mu, init_I, cu_seqlens, recurrent=True)
        gr = recurrent_backward(p, float(scale), d_o, d_o_var,
                                in_dtypes=(q.dtype, k.dtype, v.dtype, b.dtype, gt.dtype, g.dtype, Ip.dtype),
                                g_shape=tuple(g.shape), Ip_shape=tuple(Ip.shape))
        return gr[:7] + (gr[7].to(init_mu.dtype) if gr[7] is not None else gr[5].new_empty(0),
                         gr[8].to(init_I.dtype) if gr[8] is not None else gr[5].new_empty(0))

    @recurrent_bwd.register_fake
    def _(q, k, v, b, gt, g, Ip, init_mu, init_I, scale, cu_seqlens, d_o, d_o_var):
        return (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(b), torch.empty_like(gt),
                torch.empty_like(g), torch.empty_like(Ip),
                torch.empty_like(init_mu) if init_mu is not None else g.new_empty(0),
                torch.empty_like(init_I) if init_I is not None else g.new_empty(0))

    def _rec_setup(ctx, inputs, output):
        q, k, v, b, gt, g, Ip, init_mu, init_I, scale, _, output_uncertainty, cu_seqlens = inputs
        ctx.save_for_backward(q, k, v, b, gt, g, Ip, init_mu, init_I, cu_seqlens)
        ctx.scale = scale
        ctx.output_uncertainty = output_uncertainty
        ctx.set_materialize_grads(False)

    def _rec_backward(ctx, d_o, d_o_var, d_fmu, d_fI):
        q, k, v, b, gt, g, Ip, init_mu, init_I, cu = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros_like(v)
        if not ctx.output_uncertainty:
            d_o_var = None
        gr = recurrent_bwd(q, k, v, b, gt, g, Ip, init_mu, init_I, ctx.scale, cu, d_o, d_o_var)
        d_mu = gr[7] if init_mu is not None else None
        d_I = gr[8] if init_I is not None else None
        return gr[0], gr[1], gr[2], gr[3], gr[4], gr[5], gr[6], d_mu, d_I, None, None, None, None

    recurrent_fwd.register_autograd(_rec_backward, setup_context=_rec_setup)
