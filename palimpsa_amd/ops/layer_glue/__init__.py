"""The element-wise work of the reference layer either side of the operator, as fused HIP kernels.

``Palimpsa.forward`` of the reference (palimpsa/layers/palimpsa.py) turns the projections into the
operator's inputs with about a dozen framework kernels (:266-279) and post-processes the operator's
output with a residual and a gated RMS norm (:337-343).  Here each side is one kernel forward and one
backward behind the C ABI (``pal_prologue_fwd/bwd``, ``pal_epilogue_fwd/bwd``):

    q, k, v, b, gt = palimpsa_inputs(q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw, b_scale)
    o = chunk_palimpsa(q, k, v, b, gt, A, Ip, ...)
    y = palimpsa_output_norm(o, x, D, gate, weight, eps)

A maintainer of the reference would replace lines :266-279 and :337-343 of the layer by these two calls;
the projections, the short convolutions and ``o_proj`` stay as they are.  There is no CPU fallback.

The reference's other caller of the operator, ``MetaMamba2.forward`` (palimpsa/layers/meta_mamba2.py), wraps it
in different element-wise work (:283-299 before, :355-363 after); the same kernels serve it in a second form:

    v, b, dt = metamamba2_inputs(x, dt_raw, dt_bias, b_raw, b_scale, dt_limit)     # dt clamped, v = x dt, b = .. dt
    o = chunk_palimpsa(C, B, v, b, dt, A, Ip, scale=1.0, ...)                       # B, C rows as they are
    y = metamamba2_output_norm(o, x, D, gate, weight, eps)                          # gate first, norm over the token
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ... import _lib as L
from ..palimpsa import _common as cm

__all__ = ["palimpsa_inputs", "palimpsa_output_norm", "PalimpsaInputs", "PalimpsaOutputNorm",
           "metamamba2_inputs", "metamamba2_output_norm", "MetaMamba2Inputs", "MetaMamba2OutputNorm"]


def _rows_dtype(*tensors) -> torch.dtype:
    return torch.bfloat16 if all(t is None or t.dtype == torch.bfloat16 for t in tensors) else torch.float32


def _check_dims(dk: int, dv: int) -> None:
    for name, d in (("dk", dk), ("dv", dv)):
        if d % 8 or not 8 <= d <= 256:
            raise ValueError(f"{name} must be a multiple of 8 in [8, 256], got {d}")


def _glue_dims(tokens, H, Hqk, dk, dv, dtype, eps, dt_min=0.0, dt_max=0.0, norm_over_heads=False):
    return L.PalGlueDims(tokens=tokens, n_heads=H, n_qk_heads=Hqk, dk=dk, dv=dv, dtype=cm._pal_dtype(dtype), eps=float(eps),
                         dt_min=float(dt_min), dt_max=float(dt_max), norm_over_heads=1 if norm_over_heads else 0)


class PalimpsaInputs(torch.autograd.Function):
    """forward(ctx, q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw, b_scale, eps) -> (q, k, v, b | None, gt)."""

    @staticmethod
    def forward(ctx, q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw, b_scale, eps):
        dev = cm._require_gpu(q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw, b_scale)
        if q_raw.shape != k_raw.shape or q_raw.shape[:-2] != x.shape[:-2]:
            raise ValueError("expected q_raw, k_raw [..., Hqk, dk] and x [..., H, dv] with the same leading dims")
        lead = tuple(x.shape[:-2])
        H, dv = x.shape[-2:]
        Hqk, dk = q_raw.shape[-2:]
        if H % Hqk:
            raise ValueError(f"the {H} value heads must be a multiple of the {Hqk} query/key heads")
        if tuple(dt_raw.shape) != lead + (H,) or tuple(bs_raw.shape) != lead + (H,):
            raise ValueError(f"dt_raw and bs_raw must be {lead + (H,)}")
        if (b_raw is None) != (b_scale is None):
            raise ValueError("b_raw and b_scale go together")
        if b_raw is not None and b_raw.shape != x.shape:
            raise ValueError("b_raw must have the shape of x")
        _check_dims(dk, dv)
        cd = _rows_dtype(q_raw, k_raw, x, dt_raw, bs_raw, b_raw)
        prep = lambda t: None if t is None else t.to(cd).contiguous()
        q_raw_c, k_raw_c, x_c, dt_c, bs_c, b_c = (prep(t) for t in (q_raw, k_raw, x, dt_raw, bs_raw, b_raw))
        bias = dt_bias.reshape(H).float().contiguous()
        bsc = None if b_scale is None else b_scale.reshape(H).float().contiguous()
        tokens = x_c.numel() // (H * dv)
        q = torch.empty(lead + (H, dk), dtype=cd, device=dev)
        k = torch.empty_like(q)
        v = torch.empty(lead + (H, dv), dtype=cd, device=dev)
        b = torch.empty_like(v) if b_raw is not None else None
        gt = torch.empty(lead + (H,), dtype=torch.float32, device=dev)
        dims = _glue_dims(tokens, H, Hqk, dk, dv, cd, eps)
        pt = cm._ptr
        tens = L.PalPrologueTensors(q_raw=pt(q_raw_c), k_raw=pt(k_raw_c), x=pt(x_c), dt_raw=pt(dt_c), bs_raw=pt(bs_c),
                                    b_raw=pt(b_c), dt_bias=pt(bias), b_scale=pt(bsc), q=pt(q), k=pt(k), v=pt(v), b=pt(b),
                                    gt=pt(gt))
        with torch.cuda.device(dev):
            rc = L.load().pal_prologue_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_prologue_fwd")
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(q_raw_c, k_raw_c, x_c, dt_c, bs_c, b_c, bias, bsc)
        ctx.meta = dict(tokens=tokens, H=H, Hqk=Hqk, dk=dk, dv=dv, cd=cd, eps=float(eps), lead=lead,
                        dtypes=[None if t is None else t.dtype for t in (q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw, b_scale)],
                        bias_shape=tuple(dt_bias.shape), bscale_shape=None if b_scale is None else tuple(b_scale.shape))
        return q, k, v, b, gt

    @staticmethod
    def backward(ctx, dq, dk, dv, db, dgt):
        q_raw, k_raw, x, dt_raw, bs_raw, b_raw, bias, bsc = ctx.saved_tensors
        m = ctx.meta
        dev = x.device
        cd, lead, H, Hqk = m["cd"], m["lead"], m["H"], m["Hqk"]

        def grad_in(g, shape, dtype):
            if g is None:
                return torch.zeros(shape, dtype=dtype, device=dev)
            return g.to(dtype).contiguous()

        dq = grad_in(dq, lead + (H, m["dk"]), cd)
        dk = grad_in(dk, lead + (H, m["dk"]), cd)
        dv = grad_in(dv, lead + (H, m["dv"]), cd)
        db = grad_in(db, lead + (H, m["dv"]), cd) if b_raw is not None else None
        dgt = grad_in(dgt, lead + (H,), torch.float32)
        dq_raw, dk_raw, dx = torch.empty_like(q_raw), torch.empty_like(k_raw), torch.empty_like(x)
        db_raw = torch.empty_like(b_raw) if b_raw is not None else None
        ddt_raw, dbs_raw = torch.empty_like(dt_raw), torch.empty_like(bs_raw)
        ddt_bias = torch.empty(H, dtype=torch.float32, device=dev)
        db_scale = torch.empty(H, dtype=torch.float32, device=dev) if b_raw is not None else None
        dims = _glue_dims(m["tokens"], H, Hqk, m["dk"], m["dv"], cd, m["eps"])
        pt = cm._ptr
        tens = L.PalPrologueTensors(q_raw=pt(q_raw), k_raw=pt(k_raw), x=pt(x), dt_raw=pt(dt_raw), bs_raw=pt(bs_raw),
                                    b_raw=pt(b_raw), dt_bias=pt(bias), b_scale=pt(bsc), q=pt(dq), k=pt(dk), v=pt(dv),
                                    b=pt(db), gt=pt(dgt))   # outputs are not touched by the backward; any valid pointers
        grads = L.PalPrologueGrads(dq=pt(dq), dk=pt(dk), dv=pt(dv), db=pt(db), dgt=pt(dgt), dq_raw=pt(dq_raw),
                                   dk_raw=pt(dk_raw), dx=pt(dx), db_raw=pt(db_raw), ddt_raw=pt(ddt_raw), dbs_raw=pt(dbs_raw),
                                   ddt_bias=pt(ddt_bias), db_scale=pt(db_scale))
        lib = L.load()
        ws_bytes = int(lib.pal_prologue_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_prologue_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_prologue_bwd")
        dt = m["dtypes"]
        return (dq_raw.to(dt[0]), dk_raw.to(dt[1]), dx.to(dt[2]), ddt_raw.to(dt[3]),
                ddt_bias.reshape(m["bias_shape"]).to(dt[4]), dbs_raw.to(dt[5]),
                None if db_raw is None else db_raw.to(dt[6]),
                None if db_scale is None else db_scale.reshape(m["bscale_shape"]).to(dt[7]), None)


class PalimpsaOutputNorm(torch.autograd.Function):
    """forward(ctx, o, x, D, gate, weight, eps) -> y = rmsnorm(o + x * D) * weight * gate * sigmoid(gate)."""

    @staticmethod
    def forward(ctx, o, x, D, gate, weight, eps):
        dev = cm._require_gpu(o, x, D, gate, weight)
        lead = tuple(o.shape[:-2])
        H, dv = o.shape[-2:]
        if (x is None) != (D is None):
            raise ValueError("x and D go together")
        for name, t in (("x", x), ("gate", gate)):
            if t is not None and t.shape != o.shape:
                raise ValueError(f"{name} must have the shape of o")
        if weight.numel() != dv:
            raise ValueError(f"weight must have {dv} entries")
        _check_dims(8, dv)
        cd = _rows_dtype(o, x, gate)
        prep = lambda t: None if t is None else t.to(cd).contiguous()
        o_c, x_c, g_c = prep(o), prep(x), prep(gate)
        Dc = None if D is None else D.reshape(H).float().contiguous()
        w = weight.reshape(dv).float().contiguous()
        tokens = o_c.numel() // (H * dv)
        y = torch.empty_like(o_c)
        rstd = torch.empty(lead + (H,), dtype=torch.float32, device=dev)
        dims = _glue_dims(tokens, H, H, 8, dv, cd, eps)
        pt = cm._ptr
        tens = L.PalEpilogueTensors(o=pt(o_c), x=pt(x_c), D=pt(Dc), gate=pt(g_c), weight=pt(w), y=pt(y), rstd=pt(rstd))
        with torch.cuda.device(dev):
            rc = L.load().pal_epilogue_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_epilogue_fwd")
        ctx.save_for_backward(o_c, x_c, Dc, g_c, w, rstd)
        ctx.meta = dict(tokens=tokens, H=H, dv=dv, cd=cd, eps=float(eps),
                        dtypes=[None if t is None else t.dtype for t in (o, x, D, gate, weight)],
                        D_shape=None if D is None else tuple(D.shape), w_shape=tuple(weight.shape))
        return y

    @staticmethod
    def backward(ctx, dy):
        o, x, D, gate, w, rstd = ctx.saved_tensors
        m = ctx.meta
        dev = o.device
        cd, H, dv = m["cd"], m["H"], m["dv"]
        dy = dy.to(cd).contiguous()
        d_o = torch.empty_like(o)
        dx = torch.empty_like(x) if x is not None else None
        dgate = torch.empty_like(gate) if gate is not None else None
        dD = torch.empty(H, dtype=torch.float32, device=dev) if x is not None else None
        dw = torch.empty(dv, dtype=torch.float32, device=dev)
        dims = _glue_dims(m["tokens"], H, H, 8, dv, cd, m["eps"])
        pt = cm._ptr
        tens = L.PalEpilogueTensors(o=pt(o), x=pt(x), D=pt(D), gate=pt(gate), weight=pt(w), y=pt(d_o), rstd=pt(rstd))
        grads = L.PalEpilogueGrads(dy=pt(dy), d_o=pt(d_o), dx=pt(dx), dgate=pt(dgate), dD=pt(dD), dweight=pt(dw))
        lib = L.load()
        ws_bytes = int(lib.pal_epilogue_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_epilogue_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_epilogue_bwd")
        dt = m["dtypes"]
        return (d_o.to(dt[0]), None if dx is None else dx.to(dt[1]),
                None if dD is None else dD.reshape(m["D_shape"]).to(dt[2]),
                None if dgate is None else dgate.to(dt[3]), dw.reshape(m["w_shape"]).to(dt[4]), None)


class MetaMamba2Inputs(torch.autograd.Function):
    """forward(ctx, x, dt_raw, dt_bias, b_raw, b_scale, dt_min, dt_max) -> (v, b | None, dt)."""

    @staticmethod
    def forward(ctx, x, dt_raw, dt_bias, b_raw, b_scale, dt_min, dt_max):
        dev = cm._require_gpu(x, dt_raw, dt_bias, b_raw, b_scale)
        lead = tuple(x.shape[:-2])
        H, dv = x.shape[-2:]
        if tuple(dt_raw.shape) != lead + (H,):
            raise ValueError(f"dt_raw must be {lead + (H,)}")
        if (b_raw is None) != (b_scale is None):
            raise ValueError("b_raw and b_scale go together")
        if b_raw is not None and b_raw.shape != x.shape:
            raise ValueError("b_raw must have the shape of x")
        if not dt_min <= dt_max:
            raise ValueError(f"dt_limit must be an ordered pair, got ({dt_min}, {dt_max})")
        _check_dims(8, dv)
        cd = _rows_dtype(x, dt_raw, b_raw)
        prep = lambda t: None if t is None else t.to(cd).contiguous()
        x_c, dt_c, b_c = prep(x), prep(dt_raw), prep(b_raw)
        bias = dt_bias.reshape(H).float().contiguous()
        bsc = None if b_scale is None else b_scale.reshape(H).float().contiguous()
        tokens = x_c.numel() // (H * dv)
        v = torch.empty(lead + (H, dv), dtype=cd, device=dev)
        b = torch.empty_like(v) if b_raw is not None else None
        gt = torch.empty(lead + (H,), dtype=torch.float32, device=dev)
        dims = _glue_dims(tokens, H, H, 8, dv, cd, 0.0, dt_min, dt_max)
        pt = cm._ptr
        tens = L.PalPrologueTensors(x=pt(x_c), dt_raw=pt(dt_c), b_raw=pt(b_c), dt_bias=pt(bias), b_scale=pt(bsc),
                                    v=pt(v), b=pt(b), gt=pt(gt))
        with torch.cuda.device(dev):
            rc = L.load().pal_prologue_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_prologue_fwd")
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(x_c, dt_c, b_c, bias, bsc)
        ctx.meta = dict(tokens=tokens, H=H, dv=dv, cd=cd, lead=lead, dt_min=float(dt_min), dt_max=float(dt_max),
                        dtypes=[None if t is None else t.dtype for t in (x, dt_raw, dt_bias, b_raw, b_scale)],
                        bias_shape=tuple(dt_bias.shape), bscale_shape=None if b_scale is None else tuple(b_scale.shape))
        return v, b, gt

    @staticmethod
    def backward(ctx, dv, db, dgt):
        x, dt_raw, b_raw, bias, bsc = ctx.saved_tensors
        m = ctx.meta
        dev = x.device
        cd, lead, H = m["cd"], m["lead"], m["H"]

        def grad_in(g, shape, dtype):
            if g is None:
                return torch.zeros(shape, dtype=dtype, device=dev)
            return g.to(dtype).contiguous()

        dv = grad_in(dv, lead + (H, m["dv"]), cd)
        db = grad_in(db, lead + (H, m["dv"]), cd) if b_raw is not None else None
        dgt = grad_in(dgt, lead + (H,), torch.float32)
        dx = torch.empty_like(x)
        db_raw = torch.empty_like(b_raw) if b_raw is not None else None
        ddt_raw = torch.empty_like(dt_raw)
        ddt_bias = torch.empty(H, dtype=torch.float32, device=dev)
        db_scale = torch.empty(H, dtype=torch.float32, device=dev) if b_raw is not None else None
        dims = _glue_dims(m["tokens"], H, H, 8, m["dv"], cd, 0.0, m["dt_min"], m["dt_max"])
        pt = cm._ptr
        tens = L.PalPrologueTensors(x=pt(x), dt_raw=pt(dt_raw), b_raw=pt(b_raw), dt_bias=pt(bias), b_scale=pt(bsc),
                                    v=pt(dv), b=pt(db), gt=pt(dgt))   # outputs are not touched by the backward
        grads = L.PalPrologueGrads(dv=pt(dv), db=pt(db), dgt=pt(dgt), dx=pt(dx), db_raw=pt(db_raw), ddt_raw=pt(ddt_raw),
                                   ddt_bias=pt(ddt_bias), db_scale=pt(db_scale))
        lib = L.load()
        ws_bytes = int(lib.pal_prologue_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_prologue_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_prologue_bwd")
        dt = m["dtypes"]
        return (dx.to(dt[0]), ddt_raw.to(dt[1]), ddt_bias.reshape(m["bias_shape"]).to(dt[2]),
                None if db_raw is None else db_raw.to(dt[3]),
                None if db_scale is None else db_scale.reshape(m["bscale_shape"]).to(dt[4]), None, None)


class MetaMamba2OutputNorm(torch.autograd.Function):
    """forward(ctx, o, x, D, gate, weight, eps) -> y = rmsnorm over all heads of ((o + x * D) * gate * sigmoid(gate)) * weight."""

    @staticmethod
    def forward(ctx, o, x, D, gate, weight, eps):
        dev = cm._require_gpu(o, x, D, gate, weight)
        lead = tuple(o.shape[:-2])
        H, dv = o.shape[-2:]
        if (x is None) != (D is None):
            raise ValueError("x and D go together")
        for name, t in (("x", x), ("gate", gate)):
            if t is not None and tuple(t.shape) not in (tuple(o.shape), lead + (H * dv,)):
                raise ValueError(f"{name} must have the entries of o ({tuple(o.shape)} or {lead + (H * dv,)})")
        if weight.numel() != H * dv:
            raise ValueError(f"weight must have {H * dv} entries")
        if H * dv > 4096:
            raise ValueError(f"the norm over all heads serves up to 4096 entries per token, got {H * dv}")
        _check_dims(8, dv)
        cd = _rows_dtype(o, x, gate)
        prep = lambda t: None if t is None else t.to(cd).contiguous()
        o_c, x_c, g_c = prep(o), prep(x), prep(gate)
        Dc = None if D is None else D.reshape(H).float().contiguous()
        w = weight.reshape(H * dv).float().contiguous()
        tokens = o_c.numel() // (H * dv)
        y = torch.empty_like(o_c)
        rstd = torch.empty(lead, dtype=torch.float32, device=dev)
        dims = _glue_dims(tokens, H, H, 8, dv, cd, eps, norm_over_heads=True)
        pt = cm._ptr
        tens = L.PalEpilogueTensors(o=pt(o_c), x=pt(x_c), D=pt(Dc), gate=pt(g_c), weight=pt(w), y=pt(y), rstd=pt(rstd))
        with torch.cuda.device(dev):
            rc = L.load().pal_epilogue_fwd(dims, tens, cm.current_stream_ptr(dev))
        L.check(rc, "pal_epilogue_fwd")
        ctx.save_for_backward(o_c, x_c, Dc, g_c, w, rstd)
        ctx.meta = dict(tokens=tokens, H=H, dv=dv, cd=cd, eps=float(eps),
                        dtypes=[None if t is None else t.dtype for t in (o, x, D, gate, weight)],
                        shapes=[None if t is None else tuple(t.shape) for t in (o, x, D, gate, weight)])
        return y

    @staticmethod
    def backward(ctx, dy):
        o, x, D, gate, w, rstd = ctx.saved_tensors
        m = ctx.meta
        dev = o.device
        cd, H, dv = m["cd"], m["H"], m["dv"]
        dy = dy.to(cd).contiguous()
        d_o = torch.empty_like(o)
        dx = torch.empty_like(x) if x is not None else None
        dgate = torch.empty_like(gate) if gate is not None else None
        dD = torch.empty(H, dtype=torch.float32, device=dev) if x is not None else None
        dw = torch.empty(H * dv, dtype=torch.float32, device=dev)
        dims = _glue_dims(m["tokens"], H, H, 8, dv, cd, m["eps"], norm_over_heads=True)
        pt = cm._ptr
        tens = L.PalEpilogueTensors(o=pt(o), x=pt(x), D=pt(D), gate=pt(gate), weight=pt(w), y=pt(d_o), rstd=pt(rstd))
        grads = L.PalEpilogueGrads(dy=pt(dy), d_o=pt(d_o), dx=pt(dx), dgate=pt(dgate), dD=pt(dD), dweight=pt(dw))
        lib = L.load()
        ws_bytes = int(lib.pal_epilogue_bwd_workspace_bytes(dims))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = lib.pal_epilogue_bwd(dims, tens, grads, C.c_void_p(ws.data_ptr()), ws_bytes, cm.current_stream_ptr(dev))
        L.check(rc, "pal_epilogue_bwd")
        dt, sh = m["dtypes"], m["shapes"]
        return (d_o.to(dt[0]), None if dx is None else dx.reshape(sh[1]).to(dt[1]),
                None if dD is None else dD.reshape(sh[2]).to(dt[2]),
                None if dgate is None else dgate.reshape(sh[3]).to(dt[3]), dw.reshape(sh[4]).to(dt[4]), None)


@cm.no_compile
def palimpsa_inputs(q_raw: torch.Tensor, k_raw: torch.Tensor, x: torch.Tensor, dt_raw: torch.Tensor,
                    dt_bias: torch.Tensor, bs_raw: torch.Tensor, b_raw: Optional[torch.Tensor] = None,
                    b_scale: Optional[torch.Tensor] = None, eps: float = 1e-12):
    """Operator inputs from the layer's projections (layers/palimpsa.py:266-279 of the reference).

    q_raw, k_raw ``[..., Hqk, dk]`` and x ``[..., H, dv]`` are the (convolved, activated) q/k/v projections
    split into heads; dt_raw, bs_raw ``[..., H]`` the outputs of ``dt_proj`` / ``bs_proj``; b_raw ``[..., H, dv]``
    the output of ``b_proj`` (None with metaplasticity off).  Returns ``(q, k, v, b | None, gt)``: q, k
    L2-normalised with their heads repeated ``H / Hqk`` times, ``v = x * bs``, ``b = sigmoid(b_raw) *
    softplus(b_scale) * bs`` with ``bs = sigmoid(bs_raw)`` rounded to the row dtype, and
    ``gt = softplus(dt_raw + dt_bias)`` in fp32."""
    return PalimpsaInputs.apply(q_raw, k_raw, x, dt_raw, dt_bias, bs_raw, b_raw, b_scale, eps)


@cm.no_compile
def palimpsa_output_norm(o: torch.Tensor, x: Optional[torch.Tensor], D: Optional[torch.Tensor],
                         gate: Optional[torch.Tensor], weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """Residual and output norm of the layer (layers/palimpsa.py:337-343): ``rmsnorm(o + x * D) * weight``,
    times ``gate * sigmoid(gate)`` when a gate is given; o, x, gate ``[..., H, dv]``, D ``[H]``, weight ``[dv]``."""
    return PalimpsaOutputNorm.apply(o, x, D, gate, weight, eps)


@cm.no_compile
def metamamba2_inputs(x: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, b_raw: Optional[torch.Tensor] = None,
                      b_scale: Optional[torch.Tensor] = None, dt_limit=(0.0, float("inf"))):
    """Operator inputs of ``MetaMamba2.forward`` from its projections (layers/meta_mamba2.py:283-299 of the reference).

    x ``[..., H, dv]`` is the convolved value stream split into heads, dt_raw ``[..., H]`` the time-step columns of
    ``in_proj``, b_raw ``[..., H, dv]`` the output of ``b_proj`` (None with metaplasticity off).  Returns
    ``(v, b | None, dt)``: ``dt = clamp(softplus(dt_raw + dt_bias), *dt_limit)`` in fp32 (the operator's ``gt``),
    ``v = x * dt`` and ``b = sigmoid(b_raw) * softplus(b_scale) * dt`` in the row dtype.  The layer's ``B`` and ``C``
    rows go to the operator as they are (``k = B``, ``q = C``; fewer heads than ``H`` are shared inside the kernels)."""
    return MetaMamba2Inputs.apply(x, dt_raw, dt_bias, b_raw, b_scale, float(dt_limit[0]), float(dt_limit[1]))


@cm.no_compile
def metamamba2_output_norm(o: torch.Tensor, x: Optional[torch.Tensor], D: Optional[torch.Tensor],
                           gate: Optional[torch.Tensor], weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """Residual, gate and output norm of ``MetaMamba2.forward`` (layers/meta_mamba2.py:355-363):
    ``rmsnorm((o + x * D) * gate * sigmoid(gate)) * weight`` with the mean square taken over all ``H * dv`` entries of a
    token (``RMSNormGated(intermediate_size, norm_before_gate=False)``); o ``[..., H, dv]``, x and gate with the same
    entries (``[..., H, dv]`` or ``[..., H * dv]``), D ``[H]``, weight ``[H * dv]``.  Returns ``[..., H, dv]``."""
    return MetaMamba2OutputNorm.apply(o, x, D, gate, weight, eps)
