"""Chunk-parallel Palimpsa operator (training / prefill path) on HIP kernels.

Mirrors palimpsa/ops/palimpsa/chunk_palimpsa_forgetting_scalar.py of the
reference: ``chunk_palimpsa`` (:623-667) and the 17-argument
``ChunkPalimpsa`` autograd Function (:437-620) keep their names, argument
order, defaults, return packing and ValueError.  Deliberate differences:

* the kernels always work on tiles of 64 tokens; ``chunk_size`` is accepted for
  signature compatibility and validated, but results do not depend on it (the
  chunked form is exact for any tile size) and the chunk-state buffers are
  sized for 64-token tiles;
* ``chunk_offsets`` (argument 15 of the Function) carries this build's packed
  chunk metadata for varlen batches: ``[N+1]`` cumulative chunk counts followed
  by ``[total_chunks,4]`` rows (sequence, first token, length, index in
  sequence);
* gradients of fp32 inputs (gt, g, Ip) come back in fp32 instead of being
  rounded to q.dtype (:617-620), and gradients for the initial states are
  returned instead of None;
* no ``torch.autocast`` wrapper (:440, :521).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ... import _lib as L
from . import _common as cm
from . import _custom_ops as _ops


def _count_chunks(T: int, B: int) -> int:
    return (T + L.PAL_CHUNK - 1) // L.PAL_CHUNK * B


# the windowed forward keeps at most this many bytes of tile-start states alive (measured on one sequence of 65536
# tokens, H = 16, 128 x 128: 64 MB 6.3 ms, 128 MB 5.8, 512 MB 5.65, 1 GB 5.73, all 2.1 GB at once 5.8: the output
# kernel is bound by vector issue whether the states come from the last-level cache or from HBM, and every window
# pays the fill of the state pass's pipeline)
_WINDOW_STATE_BYTES = 512 << 20


def _window_tiles(H: int, dv: int, dk: int) -> int:
    return max(16, _WINDOW_STATE_BYTES // (2 * 4 * H * dv * dk))


def _windowed_forward(p, scale, output_uncertainty, o, o_var, final_mu, final_I, window: int) -> None:
    """Forward of one sequence (B == 1) in segments of ``window`` tiles, each started from the final
    state of the one before.  Same kernels and same tiles as the single call; the state crosses a
    segment boundary as (mu, I), which costs one fp32 rounding per boundary."""
    dev = p.q.device
    _, T, H, _ = p.v.shape
    seg = window * L.PAL_CHUNK
    int_mu = torch.empty(window, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
    int_I = torch.empty_like(int_mu)
    # state out alternates between a scratch pair and (final_mu, final_I) such that the last segment
    # writes the final buffers; a segment never reads the buffers it writes
    scratch = (torch.empty_like(final_mu), torch.empty_like(final_I))
    n_seg = (T + seg - 1) // seg
    lib = L.load()
    pt = cm._ptr
    cur_mu, cur_I = p.init_mu, p.init_I
    with torch.cuda.device(dev):
        stream = cm.current_stream_ptr(dev)
        for j in range(n_seg):
            s, e = j * seg, min(T, (j + 1) * seg)
            out_mu, out_I = (final_mu, final_I) if (n_seg - 1 - j) % 2 == 0 else scratch
            flags = L.PAL_FLAG_STORE_FINAL | L.state_pass_flags()
            if cur_mu is not None:
                flags |= L.PAL_FLAG_HAS_INIT
            if output_uncertainty:
                flags |= L.PAL_FLAG_HAS_VAR
            n_tiles = (e - s + L.PAL_CHUNK - 1) // L.PAL_CHUNK
            dims = L.PalDims(batch=1, seq_len=e - s, n_seqs=1, n_heads=H, dk=p.dk_p, dv=p.dv_p, total_chunks=n_tiles,
                             dtype=cm._pal_dtype(p.compute_dtype), gate_dtype=cm._pal_dtype(p.gt.dtype),
                             var_dtype=cm._pal_dtype(p.compute_dtype), flags=flags, scale=float(scale),
                             n_qk_heads=p.q.shape[2])
            tens = L.PalFwdTensors(
                q=pt(p.q[:, s:e]), k=pt(p.k[:, s:e]), v=pt(p.v[:, s:e]), b=pt(p.b[:, s:e]), gt=pt(p.gt[:, s:e]),
                g=pt(p.g), Ip=pt(p.Ip), o=pt(o[:, s:e]), o_var=pt(o_var[:, s:e] if o_var is not None else None),
                init_mu=pt(cur_mu), init_I=pt(cur_I), final_mu=pt(out_mu), final_I=pt(out_I), cu_seqlens=None,
                chunk_table=None, chunk_offsets=None, chunk_mu=pt(int_mu), chunk_I=pt(int_I))
            L.check(lib.pal_chunk_fwd(dims, tens, stream), "pal_chunk_fwd")
            cur_mu, cur_I = out_mu, out_I


class ChunkPalimpsa(torch.autograd.Function):
    """forward(ctx, q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, scale, chunk_size,
    output_final_state, output_uncertainty, cu_seqlens, chunk_offsets, int_mu, int_I)
    -> (o, o_var | None, final_mu, final_I); argument order of chunk...py:441."""

    @staticmethod
    def forward(ctx, q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, scale, chunk_size,
                output_final_state, output_uncertainty, cu_seqlens, chunk_offsets, int_mu, int_I):
        p = cm.prepare_inputs(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, cu_seqlens,
                              recurrent=False)
        dev = p.q.device
        B, T, H, _ = p.v.shape
        table = offsets = None
        if p.cu_seqlens is not None:
            if chunk_offsets is None:
                chunk_offsets, _ = cm.chunk_meta(cu_seqlens, T, dev)
            meta = chunk_offsets.to(device=dev, dtype=torch.int32).contiguous()
            offsets = meta[: p.n_seqs + 1]
            table = meta[p.n_seqs + 1:]
            total_chunks = int(table.numel()) // 4
        else:
            total_chunks = _count_chunks(T, B)
        o = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev)
        # the reference hands o_var back in q.dtype (chunk...py:515)
        o_var = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev) if output_uncertainty else None
        # final states are always produced, as in the reference (chunk...py:475-476)
        final_mu = torch.empty(p.n_seqs, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        final_I = torch.empty_like(final_mu)

        window = _window_tiles(H, p.dv_p, p.dk_p)
        if (not any(ctx.needs_input_grad[:9]) and int_mu is None and int_I is None and p.cu_seqlens is None
                and B == 1 and total_chunks > window):
            # nothing will ask for the tile-start states again: run the sequence in windows of tiles through the
            # state, so that the per-tile states (2*H*dv*dk*4 bytes per tile) never exist for more than one window
            _windowed_forward(p, scale, output_uncertainty, o, o_var, final_mu, final_I, window)
            o = cm.unpad_last(o, p.dv).to(q.dtype)
            o_var = cm.unpad_last(o_var, p.dv).to(q.dtype) if output_uncertainty else None
            return o, o_var, cm.unpad_state(final_mu, p), cm.unpad_state(final_I, p)

        need = (total_chunks, H, p.dv_p, p.dk_p)
        if (int_mu is None or int_I is None or tuple(int_mu.shape) != need or tuple(int_I.shape) != need
                or int_mu.dtype != torch.float32 or int_I.dtype != torch.float32
                or int_mu.device != dev or not int_mu.is_contiguous() or not int_I.is_contiguous()):
            int_mu = torch.empty(need, dtype=torch.float32, device=dev)
            int_I = torch.empty(need, dtype=torch.float32, device=dev)
        flags = L.PAL_FLAG_STORE_FINAL
        if p.cu_seqlens is not None:
            flags |= L.PAL_FLAG_VARLEN
        if p.init_mu is not None:
            flags |= L.PAL_FLAG_HAS_INIT
        if output_uncertainty:
            flags |= L.PAL_FLAG_HAS_VAR
        dims = cm.make_dims(p, scale, flags, total_chunks, var_dtype=p.compute_dtype)
        tens = cm.make_fwd_tensors(p, o, o_var, final_mu, final_I, table, offsets, int_mu, int_I)
        with torch.cuda.device(dev):
            rc = L.load().pal_chunk_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_chunk_fwd")

        # gradients of unused outputs arrive as None instead of zero-filled tensors (the final states'
        # gradients are ignored anyway)
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(p.q, p.k, p.v, p.b, p.gt, p.g, p.Ip, p.init_mu, p.init_I, p.cu_seqlens,
                              table, offsets, int_mu, int_I)
        ctx.meta = dict(dk=p.dk, dv=p.dv, dk_p=p.dk_p, dv_p=p.dv_p, n_seqs=p.n_seqs, compute_dtype=p.compute_dtype,
                        scale=float(scale), flags=(flags | L.state_pass_flags()) & ~L.PAL_FLAG_STORE_FINAL, total_chunks=total_chunks,
                        in_dtypes=(q.dtype, k.dtype, v.dtype, b.dtype, gt.dtype, g.dtype, Ip.dtype),
                        g_shape=tuple(g.shape), Ip_shape=tuple(Ip.shape), has_init=p.init_mu is not None,
                        output_uncertainty=bool(output_uncertainty))
        o = cm.unpad_last(o, p.dv).to(q.dtype)
        o_var = cm.unpad_last(o_var, p.dv).to(q.dtype) if output_uncertainty else None
        return o, o_var, cm.unpad_state(final_mu, p), cm.unpad_state(final_I, p)

    @staticmethod
    def backward(ctx, do, do_var=None, d_mu=None, d_I=None):
        # incoming gradients of the final states are ignored, as in the reference (chunk...py:522)
        (q, k, v, b, gt, g, Ip, init_mu, init_I, cu, table, offsets, int_mu, int_I) = ctx.saved_tensors
        m = ctx.meta
        dev = q.device
        B, T, H, dv_p = v.shape
        dk_p = q.shape[-1]
        cd = m["compute_dtype"]
        has_var = m["output_uncertainty"] and do_var is not None
        if do is None:   # only o_var (or nothing) was used downstream
            do = torch.zeros(B, T, H, m["dv"], dtype=cd, device=dev)

        def prep_grad(x):
            x = x.to(cd)
            if dv_p != m["dv"]:
                x = torch.nn.functional.pad(x, (0, dv_p - m["dv"]))
            return x.contiguous()

        do_p = prep_grad(do)
        dovar_p = prep_grad(do_var) if has_var else None
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        db = torch.empty_like(b)
        dgt = torch.empty(B, T, H, dtype=torch.float32, device=dev)
        dg = torch.empty(H, dtype=torch.float32, device=dev)
        dIp = torch.empty(H, dtype=torch.float32, device=dev)
        d_init_mu = d_init_I = None
        if m["has_init"]:
            d_init_mu = torch.empty_like(init_mu)
            d_init_I = torch.empty_like(init_I)
        flags = m["flags"]
        if has_var:
            flags |= L.PAL_FLAG_HAS_VAR
        else:
            flags &= ~L.PAL_FLAG_HAS_VAR
        dims = L.PalDims(batch=B, seq_len=T, n_seqs=m["n_seqs"], n_heads=H, dk=dk_p, dv=dv_p,
                         total_chunks=m["total_chunks"], dtype=cm._pal_dtype(cd), gate_dtype=cm._pal_dtype(gt.dtype),
                         var_dtype=cm._pal_dtype(cd), flags=flags, scale=m["scale"], n_qk_heads=q.shape[2])
        pt = cm._ptr
        tens = L.PalFwdTensors(q=pt(q), k=pt(k), v=pt(v), b=pt(b), gt=pt(gt), g=pt(g), Ip=pt(Ip), o=pt(do_p),
                               o_var=None, init_mu=pt(init_mu), init_I=pt(init_I), final_mu=None, final_I=None,
                               cu_seqlens=pt(cu), chunk_table=pt(table), chunk_offsets=pt(offsets),
                               chunk_mu=pt(int_mu), chunk_I=pt(int_I))
        grads = L.PalBwdTensors(d_o=pt(do_p), d_o_var=pt(dovar_p), dq=pt(dq), dk=pt(dk), dv=pt(dv), db=pt(db),
                                dgt=pt(dgt), dg=pt(dg), dIp=pt(dIp), d_init_mu=pt(d_init_mu), d_init_I=pt(d_init_I))
        lib = L.load()
        ws_bytes = int(lib.pal_chunk_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_chunk_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_chunk_bwd")
        dts = m["in_dtypes"]
        dq = cm.unpad_last(dq, m["dk"]).to(dts[0])
        dk = cm.unpad_last(dk, m["dk"]).to(dts[1])
        dv = cm.unpad_last(dv, m["dv"]).to(dts[2])
        db = cm.unpad_last(db, m["dv"]).to(dts[3])
        dgt = dgt.to(dts[4])
        dg = dg.reshape(m["g_shape"]).to(dts[5])
        dIp = dIp.reshape(m["Ip_shape"]).to(dts[6])
        if d_init_mu is not None and (dk_p != m["dk"] or dv_p != m["dv"]):
            d_init_mu = d_init_mu[:, :, :m["dv"], :m["dk"]].contiguous()
            d_init_I = d_init_I[:, :, :m["dv"], :m["dk"]].contiguous()
        return (dq, dk, dv, db, dgt, dg, dIp, d_init_mu, d_init_I,
                None, None, None, None, None, None, None, None)


def _assume_constant(fn):
    mark = getattr(getattr(torch, "_dynamo", None), "assume_constant_result", None)
    return mark(fn) if mark is not None else fn


@_assume_constant
def _bwd_supported_code(dk_p: int, dv_p: int, dtype: int, flags: int) -> int:
    """pal_chunk_bwd_supported as a plain int; a tracer evaluates it once on its constant arguments instead of
    following the ctypes call."""
    return int(L.load().pal_chunk_bwd_supported(dk_p, dv_p, dtype, flags))


def chunk_palimpsa(q, k, v, b, gt, g, Ip, initial_mu_state=None, initial_I_state=None, scale=None,
                   chunk_size=16, output_final_state=False, output_uncertainty=False, cu_seqlens=None):
    """Chunked Palimpsa attention; calling convention of chunk_palimpsa in the reference
    (chunk...py:623-667).  Returns ``o`` (or ``(o, o_var)``), plus the final ``(mu, I)``
    states when ``output_final_state`` is set."""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    if not isinstance(chunk_size, int) or chunk_size <= 0:
        raise ValueError(f"chunk_size must be a positive int, got {chunk_size!r}")
    if _ops.available() and torch.compiler.is_compiling():
        # under a tracer the work is handed over as opaque library ops (see _custom_ops.py)
        if cu_seqlens is not None and q.shape[0] != 1:
            raise ValueError(f"Batch size must be 1 for Varlen, got {q.shape[0]}")
        mode_flags = L.state_pass_flags()
        if torch.is_grad_enabled() and any(isinstance(x, torch.Tensor) and x.requires_grad
                                           for x in (q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state)):
            # refuse here what the backward could not serve, as the eager route does
            rows_bf16 = all(x.dtype == torch.bfloat16 for x in (q, k, v, b))
            rc = _bwd_supported_code(cm.padded_dk(q.shape[-1], False), cm.padded_dv(v.shape[-1]),
                                     L.PAL_DTYPE_BF16 if rows_bf16 else L.PAL_DTYPE_F32, mode_flags)
            if rc != 0:
                raise ValueError(f"chunk_palimpsa (backward head dims): unsupported by pal_chunk_bwd (code {rc})")
        o, o_var, final_mu_state, final_I_state, _, _ = _ops.chunk_fwd(
            q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, float(scale), bool(output_uncertainty), cu_seqlens,
            mode_flags)
        out = (o, o_var) if output_uncertainty else o
        if output_final_state:
            return out, final_mu_state, final_I_state
        return out
    return _eager_chunk(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, scale, chunk_size,
                        output_final_state, output_uncertainty, cu_seqlens)


@cm.no_compile
def _eager_chunk(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, scale, chunk_size, output_final_state,
                 output_uncertainty, cu_seqlens):
    chunk_offsets = None
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(f"Batch size must be 1 for Varlen, got {q.shape[0]}")
        chunk_offsets, total_chunks = cm.chunk_meta(cu_seqlens, q.shape[1], q.device)
    else:
        total_chunks = _count_chunks(q.shape[1], q.shape[0])
    H = v.shape[-2]
    dk_p, dv_p = cm.padded_dk(q.shape[-1], False), cm.padded_dv(v.shape[-1])
    # chunk-start states, allocated outside the autograd Function as in the reference (chunk...py:652-653);
    # a long single sequence that no backward will follow is run in windows instead (see _windowed_forward)
    needs_grad = torch.is_grad_enabled() and any(
        isinstance(x, torch.Tensor) and x.requires_grad for x in (q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state))
    if needs_grad:
        # refuse here what the backward could not serve, instead of at .backward() time
        rows_bf16 = all(x.dtype == torch.bfloat16 for x in (q, k, v, b))
        L.check(L.load().pal_chunk_bwd_supported(dk_p, dv_p, L.PAL_DTYPE_BF16 if rows_bf16 else L.PAL_DTYPE_F32,
                                                 L.state_pass_flags()), "chunk_palimpsa (backward head dims)")
    if not needs_grad and cu_seqlens is None and q.shape[0] == 1 and total_chunks > _window_tiles(H, dv_p, dk_p):
        int_mu = int_I = None
    else:
        int_mu = torch.empty(total_chunks, H, dv_p, dk_p, dtype=torch.float32, device=q.device)
        int_I = torch.empty(total_chunks, H, dv_p, dk_p, dtype=torch.float32, device=q.device)
    o, o_var, final_mu_state, final_I_state = ChunkPalimpsa.apply(
        q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, scale, chunk_size,
        output_final_state, output_uncertainty, cu_seqlens, chunk_offsets, int_mu, int_I)
    out = (o, o_var) if output_uncertainty else o
    if output_final_state:
        return out, final_mu_state, final_I_state
    return out
