"""Scalar-gated linear attention: the layer's operator pair without the precision state.

The reference layer falls back to ``fla.ops.simple_gla`` when its precision state is switched off
(``metaplasticity=False``: palimpsa/layers/palimpsa.py:18, :293-300).  With ``b = 0`` and ``Ip = 1``
the Palimpsa recurrence has ``I = 1`` everywhere, so ``mu = M`` and

    S_t = exp(g_t) S_{t-1} + k_t^T v_t ,   o_t = scale * q_t S_t .

``chunk_simple_gla`` and ``fused_recurrent_simple_gla`` keep the keyword names of the layer's call sites
(``q, k, v, g, scale, initial_state, output_final_state, cu_seqlens``), the default
``scale = dk ** -0.5`` and the ``(o, final_state)`` return; the state is ``[N, H, dk, dv]`` fp32 (the
transpose of the kernels' ``[N, H, dv, dk]``).  flash-linear-attention itself is not part of the reference
tree, so its own conventions beyond these call sites are not pinned; the arithmetic is pinned by the
closed form ``o = scale * ((Q K^T) * L) V`` in the tests.

``chunk_simple_gla`` runs kernels of its own (``pal_gla_chunk_fwd`` / ``pal_gla_chunk_bwd``): without the
division by ``I`` a tile's output is two plain matrix products, so the per-token state never has to exist.
``fused_recurrent_simple_gla`` without autograd runs ``pal_gla_recurrent_fwd``, which keeps the state in the
caller's ``[N, H, dk, dv]`` layout; with autograd it runs the Palimpsa token-serial kernels with ``b = 0``,
``Ip = 1`` and ``gt = -g`` under a unit per-head rate (the precision branch then works on zeros).

``q`` and ``k`` may carry fewer heads than ``v`` (``[B, T, Hq, dk]`` with ``Hq`` a divisor of ``H``): a group of
``H / Hq`` value heads then shares one q/k head, which is what the reference's MetaMamba2 layer obtains by repeating
its ``B``, ``C`` groups before the call (layers/meta_mamba2.py:281-282); the kernels index the shared rows and
``dq``, ``dk`` come back summed over each group.  ``g`` is always ``[B, T, H]``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ... import _lib as L
from ..palimpsa import _common as cm
from ..palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
from ..palimpsa.chunk import _count_chunks

__all__ = ["chunk_simple_gla", "fused_recurrent_simple_gla", "ChunkSimpleGLA", "SimpleGlaDecodeStep"]


_RATE_CACHE: dict = {}


def _minus_one_rate(H: int, dev: torch.device) -> torch.Tensor:
    """fp32 [H] tensor of -1 (the kernels compute f_t = exp(-gt_t * rate) and take g itself as gt); kept per device."""
    key = (dev.type, dev.index if dev.index is not None else torch.cuda.current_device(), H)
    t = _RATE_CACHE.get(key)
    if t is None:
        with torch.inference_mode(False):     # a tensor made under inference mode could not be saved for a later backward
            t = _RATE_CACHE[key] = torch.full((H,), -1.0, dtype=torch.float32, device=dev)
    return t


def _run(op, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens, **kw):
    if g is None:
        raise ValueError("g (log decay per token and head, [B, T, H]) is required")
    if g.shape != v.shape[:3]:
        raise ValueError(f"g must have shape {tuple(v.shape[:3])}, got {tuple(g.shape)}")
    H = v.shape[2]
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


class ChunkSimpleGLA(torch.autograd.Function):
    """forward(ctx, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens) -> (o, final_state | None)
    on ``pal_gla_chunk_fwd`` / ``pal_gla_chunk_bwd``.  The state is ``[N, H, dk, dv]`` at this boundary and
    ``[N, H, dv, dk]`` inside.  Gradients reaching the final state are not propagated (as in ChunkPalimpsa)."""

    @staticmethod
    def forward(ctx, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens):
        H = v.shape[2]
        dev = q.device
        rate = _minus_one_rate(H, dev)
        S0 = None
        if initial_state is not None:
            S0 = initial_state.float().transpose(-1, -2).contiguous()       # [N,H,dk,dv] -> [N,H,dv,dk]
        p = cm.prepare_inputs(q, k, v, v, g, rate, rate, S0, S0, cu_seqlens, recurrent=False)
        B, T = p.q.shape[:2]
        table = offsets = None
        flags = 0
        if p.cu_seqlens is not None:
            meta, total_chunks = cm.chunk_meta(cu_seqlens, T, dev)
            offsets, table = meta[: p.n_seqs + 1], meta[p.n_seqs + 1:]
            flags |= L.PAL_FLAG_VARLEN
        else:
            total_chunks = _count_chunks(T, B)
        if p.init_mu is not None:
            flags |= L.PAL_FLAG_HAS_INIT
        o = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev)
        # per-tile contributions (fp32, only needed inside the call) and tile-start states (bf16, kept for the backward)
        tile_S = torch.empty(total_chunks, H, p.dv_p, p.dk_p, dtype=torch.bfloat16, device=dev)
        final = None
        if output_final_state:
            final = torch.empty(p.n_seqs, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        dims = cm.make_dims(p, scale, flags | (L.PAL_FLAG_STORE_FINAL if output_final_state else 0), total_chunks)
        # the fp32 scratch (4 bytes per state entry and tile) only exists for the two-kernel form of the tile states
        scratch = None
        if not L.load().pal_state_pass_applies(dims, 0):
            scratch = torch.empty(total_chunks, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        pt = cm._ptr
        tens = L.PalFwdTensors(q=pt(p.q), k=pt(p.k), v=pt(p.v), gt=pt(p.gt), g=pt(p.g), o=pt(o), init_mu=pt(p.init_mu),
                               final_mu=pt(final), cu_seqlens=pt(p.cu_seqlens), chunk_table=pt(table),
                               chunk_offsets=pt(offsets), chunk_mu=pt(scratch), chunk_I=pt(tile_S))
        with torch.cuda.device(dev):
            rc = L.load().pal_gla_chunk_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_gla_chunk_fwd")
        if any(ctx.needs_input_grad):
            ctx.set_materialize_grads(False)
            ctx.save_for_backward(p.q, p.k, p.v, p.gt, p.g, p.init_mu, p.cu_seqlens, table, offsets, tile_S)
            ctx.meta = dict(dk=p.dk, dv=p.dv, n_seqs=p.n_seqs, compute_dtype=p.compute_dtype, scale=float(scale),
                            flags=flags | L.state_pass_flags(), total_chunks=total_chunks, in_dtypes=(q.dtype, k.dtype, v.dtype, g.dtype),
                            init_dtype=None if initial_state is None else initial_state.dtype)
        o = cm.unpad_last(o, p.dv).to(q.dtype)
        if final is not None:
            final = cm.unpad_state(final, p).transpose(-1, -2).contiguous()
        return o, final

    @staticmethod
    def backward(ctx, do, d_final=None):
        q, k, v, gt, rate, init, cu, table, offsets, tile_S = ctx.saved_tensors
        m = ctx.meta
        dev = q.device
        B, T, Hq, dk_p = q.shape
        H, dv_p = v.shape[2], v.shape[-1]
        cd = m["compute_dtype"]
        if do is None:
            do = torch.zeros(B, T, H, m["dv"], dtype=cd, device=dev)
        do = do.to(cd)
        if dv_p != m["dv"]:
            do = torch.nn.functional.pad(do, (0, dv_p - m["dv"]))
        do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dg_tok = torch.empty(B, T, H, dtype=torch.float32, device=dev)
        d_rate = torch.empty(H, dtype=torch.float32, device=dev)
        d_init = torch.empty_like(init) if init is not None else None
        dims = L.PalDims(batch=B, seq_len=T, n_seqs=m["n_seqs"], n_heads=H, dk=dk_p, dv=dv_p,
                         total_chunks=m["total_chunks"], dtype=cm._pal_dtype(cd), gate_dtype=cm._pal_dtype(gt.dtype),
                         var_dtype=cm._pal_dtype(cd), flags=m["flags"], scale=m["scale"], n_qk_heads=Hq)
        pt = cm._ptr
        tens = L.PalFwdTensors(q=pt(q), k=pt(k), v=pt(v), gt=pt(gt), g=pt(rate), o=pt(do), init_mu=pt(init),
                               cu_seqlens=pt(cu), chunk_table=pt(table), chunk_offsets=pt(offsets), chunk_I=pt(tile_S))
        grads = L.PalBwdTensors(d_o=pt(do), dq=pt(dq), dk=pt(dk), dv=pt(dv), dgt=pt(dg_tok), dg=pt(d_rate),
                                d_init_mu=pt(d_init))
        lib = L.load()
        ws_bytes = int(lib.pal_gla_chunk_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_gla_chunk_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_gla_chunk_bwd")
        dts = m["in_dtypes"]
        dq = cm.unpad_last(dq, m["dk"]).to(dts[0])
        dk = cm.unpad_last(dk, m["dk"]).to(dts[1])
        dv = cm.unpad_last(dv, m["dv"]).to(dts[2])
        if d_init is not None:
            d_init = d_init[:, :, :m["dv"], :m["dk"]].transpose(-1, -2).contiguous().to(m["init_dtype"])
        return dq, dk, dv, dg_tok.to(dts[3]), None, d_init, None, None


def _check_chunk_args(q, v, g, cu_seqlens):
    if g is None:
        raise ValueError("g (log decay per token and head, [B, T, H]) is required")
    if v.dim() != 4 or g.shape != v.shape[:3]:
        raise ValueError(f"g must have shape {tuple(v.shape[:3])}, got {tuple(g.shape)}")
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(f"Batch size must be 1 for Varlen, got {q.shape[0]}")
        cm.chunk_meta(cu_seqlens, q.shape[1], q.device)   # validates; the table is kept for the call below
    cm._require_gpu(q, g)


@cm.no_compile
def chunk_simple_gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: Optional[torch.Tensor] = None,
                     scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                     output_final_state: bool = False, cu_seqlens: Optional[torch.Tensor] = None):
    """Chunked (training / prefill) form; returns ``(o, final_state | None)``."""
    _check_chunk_args(q, v, g, cu_seqlens)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    return ChunkSimpleGLA.apply(q, k, v, g, scale, initial_state, output_final_state, cu_seqlens)


@cm.no_compile
def fused_recurrent_simple_gla(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: Optional[torch.Tensor] = None,
                               scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                               output_final_state: bool = False, cu_seqlens: Optional[torch.Tensor] = None):
    """Token-serial (decode) form; returns ``(o, final_state | None)``.  Without autograd it runs a kernel that keeps
    the state in the ``[N, H, dk, dv]`` layout of the caller (one read and one write of the state per call; the
    result may be written over ``initial_state`` by passing it again as the next call's initial state)."""
    needs_grad = torch.is_grad_enabled() and any(
        isinstance(x, torch.Tensor) and x.requires_grad for x in (q, k, v, g, initial_state))
    if needs_grad:
        return _run(fused_recurrent_palimpsa, q, k, v, g, scale, initial_state, output_final_state, cu_seqlens)
    _check_chunk_args(q, v, g, cu_seqlens)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    H = v.shape[2]
    dev = q.device
    rate = _minus_one_rate(H, dev)
    p = cm.prepare_inputs(q, k, v, v, g, rate, rate, None, None, cu_seqlens, recurrent=False)
    S0 = None
    if initial_state is not None:
        if tuple(initial_state.shape) != (p.n_seqs, H, p.dk, p.dv):
            raise ValueError(f"initial_state must be {(p.n_seqs, H, p.dk, p.dv)}, got {tuple(initial_state.shape)}")
        S0 = initial_state.float().contiguous()
        if p.dk_p != p.dk or p.dv_p != p.dv:
            S0 = torch.nn.functional.pad(S0, (0, p.dv_p - p.dv, 0, p.dk_p - p.dk))
    B, T = p.q.shape[:2]
    o = torch.empty(B, T, H, p.dv_p, dtype=p.compute_dtype, device=dev)
    final = torch.empty(p.n_seqs, H, p.dk_p, p.dv_p, dtype=torch.float32, device=dev) if output_final_state else None
    flags = (L.PAL_FLAG_VARLEN if p.cu_seqlens is not None else 0) | (L.PAL_FLAG_HAS_INIT if S0 is not None else 0) \
        | (L.PAL_FLAG_STORE_FINAL if output_final_state else 0)
    dims = cm.make_dims(p, scale, flags)
    pt = cm._ptr
    tens = L.PalFwdTensors(q=pt(p.q), k=pt(p.k), v=pt(p.v), gt=pt(p.gt), g=pt(p.g), o=pt(o), init_mu=pt(S0),
                           final_mu=pt(final), cu_seqlens=pt(p.cu_seqlens))
    with torch.cuda.device(dev):
        rc = L.load().pal_gla_recurrent_fwd(dims, tens, cm.current_stream_ptr(dev))
    L.check(rc, "pal_gla_recurrent_fwd")
    o = cm.unpad_last(o, p.dv).to(q.dtype)
    if final is not None and (p.dk_p != p.dk or p.dv_p != p.dv):
        final = final[:, :, :p.dk, :p.dv].contiguous()
    return o, final


class SimpleGlaDecodeStep:
    """Bound decode step of the path without the precision state (the counterpart of
    ``palimpsa_amd.ops.palimpsa.DecodeStep``): shapes and dtypes are checked once in ``bind``, ``step`` only issues
    ``pal_gla_recurrent_fwd`` on the current stream.  The state ``S`` ``[B, H, dk, dv]`` fp32 is updated in place, the
    output buffer is reused and nothing is allocated per step, so a step can be recorded into a HIP graph.
    ``dk`` and ``dv`` must be multiples of 16; ``tokens`` > 1 takes that many tokens per sequence and step."""

    def __init__(self, B: int, H: int, dk: int, dv: int, device, rows_dtype=torch.bfloat16,
                 scale: Optional[float] = None, tokens: int = 1):
        dev = torch.device(device)
        if dev.type != "cuda":
            raise RuntimeError("palimpsa_amd runs on an AMD GPU only; there is no CPU fallback")
        if dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        if dk % 16 or dv % 16 or not (16 <= dk <= 256 and 16 <= dv <= 256):
            raise ValueError(f"dk and dv must be multiples of 16 in [16, 256]; got dk={dk}, dv={dv}")
        if rows_dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("rows_dtype must be torch.bfloat16 or torch.float32")
        if not isinstance(tokens, int) or tokens < 1:
            raise ValueError(f"tokens must be a positive int, got {tokens!r}")
        self.B, self.H, self.dk, self.dv, self.device, self.rows_dtype, self.tokens = B, H, dk, dv, dev, rows_dtype, tokens
        self.o = torch.empty(B, tokens, H, dv, dtype=rows_dtype, device=dev)
        self._rate = _minus_one_rate(H, dev)
        self._dims = L.PalDims(batch=B, seq_len=tokens, n_seqs=B, n_heads=H, dk=dk, dv=dv, total_chunks=0,
                               dtype=cm._pal_dtype(rows_dtype), gate_dtype=L.PAL_DTYPE_F32, var_dtype=L.PAL_DTYPE_F32,
                               flags=L.PAL_FLAG_HAS_INIT | L.PAL_FLAG_STORE_FINAL,
                               scale=float(dk ** -0.5 if scale is None else scale))
        self._tens = L.PalFwdTensors(o=cm._ptr(self.o), g=cm._ptr(self._rate))
        self._fn = L.load().pal_gla_recurrent_fwd

    def _check(self, name, x, shape, dtype):
        if tuple(x.shape) != shape or x.dtype != dtype or x.device != self.device or not x.is_contiguous():
            raise ValueError(f"{name}: expected contiguous {dtype} {shape} on {self.device}, "
                             f"got {x.dtype} {tuple(x.shape)} on {x.device}")

    def bind(self, q, k, v, g, S) -> "SimpleGlaDecodeStep":
        """Check the tensors once and remember their addresses (q, k ``[B,tokens,H,dk]``, v ``[B,tokens,H,dv]``, g fp32
        ``[B,tokens,H]``, S fp32 ``[B,H,dk,dv]``); write the next tokens' rows into the same tensors before each step."""
        rs = (self.B, self.tokens, self.H)
        self._check("q", q, rs + (self.dk,), self.rows_dtype)
        self._check("k", k, rs + (self.dk,), self.rows_dtype)
        self._check("v", v, rs + (self.dv,), self.rows_dtype)
        self._check("g", g, rs, torch.float32)
        self._check("S", S, (self.B, self.H, self.dk, self.dv), torch.float32)
        t = self._tens
        t.q, t.k, t.v, t.gt = q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr()
        t.init_mu = t.final_mu = S.data_ptr()
        self._keep = (q, k, v, g, S)
        return self

    def step(self, stream: Optional[int] = None) -> torch.Tensor:
        """Advance every sequence by ``tokens`` tokens; returns the (reused) output buffer ``[B,tokens,H,dv]``."""
        sp = cm.current_stream_ptr(self.device) if stream is None else C.c_void_p(stream)
        rc = self._fn(self._dims, self._tens, sp)
        if rc:
            L.check(rc, "pal_gla_recurrent_fwd")
        return self.o
